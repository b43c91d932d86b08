"""int8 compute format: per-row symmetric int8 codes of an activation and the integer product.

    s[r] = max(amax of row r, 1e-12) / 127          (a correctly rounded fp32 division)
    q[r] = clamp(round_half_even(x[r] / s[r]), -127, 127)

`quantize_rows` takes an optional per-column factor (the weight scales, for the int8 input
gradient `Q(dy * scale) q`). On gfx950 it is the HIP quantizer (`km_quant_rows_i8`), elsewhere
torch. Replaces reference `src/kohakumoss_kernels/int8/formats.py:21-58`.
"""

from __future__ import annotations

import torch
from torch import Tensor

INT8_MAX = 127.0
AMAX_FLOOR = 1e-12
_HIP_DTYPES = (torch.bfloat16, torch.float16)


def row_scale(amax: Tensor) -> Tensor:
    """Tensor divided by tensor: torch rounds that quotient correctly; a Python divisor would go
    through a reciprocal and can be one unit off."""
    floor = amax.to(torch.float32).clamp_min(AMAX_FLOOR)
    return floor / torch.full_like(floor, INT8_MAX)


def _on_gfx950(x: Tensor) -> bool:
    if not (x.is_cuda and x.dtype in _HIP_DTYPES):
        return False
    from kohakumosstrainer_amd.kernels.arch import arch_of

    return arch_of(x.device).name == "gfx950"


def quantize_rows(x: Tensor, col_scale: Tensor | None = None) -> tuple[Tensor, Tensor]:
    """`(q int8 [rows, K], s fp32 [rows])` of a 2-D activation, its columns times `col_scale` first."""
    if x.dim() != 2:
        raise ValueError(f"int8 operand must be 2-D, got {tuple(x.shape)}")
    if _on_gfx950(x):
        from kohakumosstrainer_amd import native

        return native.quant_rows_i8(x.detach(), col_scale)
    v = x.detach().to(torch.float32)
    if col_scale is not None:
        v = v * col_scale.to(torch.float32).unsqueeze(0)
    s = row_scale(v.abs().amax(dim=1))
    codes = torch.round(v / s.unsqueeze(1)).clamp_(-INT8_MAX, INT8_MAX)
    return codes.to(torch.int8), s


def int_mm(a: Tensor, b: Tensor) -> Tensor:
    """int8 `[M, K] @ [K, N]` with an exact int32 result. The host path multiplies in fp64
    (|sum| <= K * 127^2 stays far below 2^53); a device without the HIP backend uses the
    library's int8 GEMM."""
    if a.is_cuda:
        return torch._int_mm(a.contiguous(), b)
    return (a.to(torch.float64) @ b.to(torch.float64)).to(torch.int32)


def col_major(q: Tensor) -> Tensor:
    """The same `[N, K]` matrix laid out with N contiguous (the `[K, N]` operand an int8 GEMM
    over N wants), as a view with strides `(1, N)`."""
    return q.t().contiguous().t()
