"""int8 compute formats: the per-row int8 quantizer and the int8 GEMM of the `int8_linear` op.

An operand is 2-D `[rows, K]` with K the contraction axis; a row's scale is
`max(amax, 1e-12) / 127` (correctly rounded fp32 division) and its codes
`round_half_even(x / s)` clamped to +-127; `col_scale` multiplies the columns first, in fp32.
Interface and arithmetic follow reference `src/kohakumoss_kernels/int8/formats.py:21-58`.
`quantize_rows` runs the hand-written HIP quantizer for bf16 / fp16 device tensors and plain
torch ops otherwise; both produce the same bytes.
"""

import torch
from torch import Tensor

INT8_MAX = 127.0
AMAX_FLOOR = 1e-12
_HIP_DTYPES = (torch.bfloat16, torch.float16)


def row_scale(amax: Tensor) -> Tensor:
    """`max(amax, 1e-12) / 127` per row, fp32."""
    a = amax.float().clamp_min(AMAX_FLOOR)
    return a / torch.full_like(a, INT8_MAX)


def quantize_rows(x: Tensor, col_scale: Tensor | None = None) -> tuple[Tensor, Tensor]:
    """`(q int8 [rows, K], s fp32 [rows])` of a 2-D operand, its columns times `col_scale` [K]
    first when given."""
    if x.dim() != 2:
        raise ValueError(f"int8 operand must be 2-D, got {tuple(x.shape)}")
    if x.device.type == "cuda" and x.dtype in _HIP_DTYPES and x.numel():
        from kohakumosstrainer_amd import native

        return native.quant_rows_i8(x.detach(), col_scale)
    v = x.detach().float()
    if col_scale is not None:
        v = v * col_scale.float()[None, :]
    s = row_scale(v.abs().amax(1))
    return torch.round(v / s[:, None]).clamp_(-INT8_MAX, INT8_MAX).to(torch.int8), s


def int_mm(a: Tensor, b: Tensor) -> Tensor:
    """int8 `a` [M, K] @ int8 `b` [K, N] -> int32 [M, N]. Host tensors: the fp64 product of the
    codes, which is exact (|acc| <= K * 127^2 < 2^53); device tensors go through the HIP GEMM in
    the launchers, not through here."""
    if a.device.type != "cpu":
        raise ValueError("int_mm is the host reference; device operands use the HIP int8 GEMM")
    return (a.double() @ b.double()).to(torch.int32)


def col_major(q: Tensor) -> Tensor:
    """`q` [N, K] as a column-major `[N, K]` view (one transposed copy)."""
    return q.t().contiguous().t()
