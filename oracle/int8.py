"""Oracle (test infrastructure): the int8 compute linear on the CPU with torch.

per-row quantizer   reference `src/kohakumoss_kernels/int8/formats.py:21-38`
int8 GEMM           reference `int8/formats.py:41-52` (`torch._int_mm`, int32 accumulation; here
                    the fp64 matmul of the codes, exact because |acc| <= K * 127^2 < 2^53)
forward / dgrad     reference `src/kohakumoss_kernels/int8/op.py:40-60`; `group` > 0 rotates x
                    before the quantizer and dx afterwards (`oracle/hadamard.py`; `rotation`
                    picks the reference's eager form or its kernels' butterfly form)

Pinned by `tests/test_oracle_int8.py`: the reference's half-to-even known answers and floor
scale (`tests/kernels/quant/test_int8_linear.py:142-148`), a definition-level numpy restatement,
exact agreement with an fp64 model of the scheme on inputs that quantize without error
(`test_int8_linear.py:84-113`), closeness to that model off the grid with broken designs failing
(`:116-130`). No function here is "parity unpinned".
"""

import torch
from torch import Tensor

from oracle import hadamard

INT8_MAX = 127.0
AMAX_FLOOR = 1e-12
DGRAD = ("int8", "16bit")


def row_scale(amax: Tensor) -> Tensor:
    """`max(amax, 1e-12) / 127` as a tensor-by-tensor (correctly rounded) fp32 division."""
    a = amax.to(torch.float32).clamp_min(AMAX_FLOOR)
    return a / torch.full_like(a, INT8_MAX)


def quantize_rows(x: Tensor, col_scale: Tensor | None = None) -> tuple[Tensor, Tensor]:
    """`(q int8 [rows, K], s fp32 [rows])`; the columns are multiplied by `col_scale` [K] in
    fp32 first when given; codes round half to even and are clamped to +-127."""
    if x.dim() != 2:
        raise ValueError(f"int8 operand must be 2-D, got {tuple(x.shape)}")
    v = x.detach().to(torch.float32)
    if col_scale is not None:
        v = v * col_scale.to(torch.float32)[None, :]
    s = row_scale(v.abs().amax(dim=1))
    q = torch.round(v / s[:, None]).clamp_(-INT8_MAX, INT8_MAX)
    return q.to(torch.int8), s


def int_mm(a: Tensor, b_t: Tensor) -> Tensor:
    """int8 `a` [M, K] times int8 `b_t` [K, N], exact int32 result."""
    return (a.to(torch.float64) @ b_t.to(torch.float64)).to(torch.int32)


def dequantize_weight(q: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    return (q.to(torch.float32) * scale.to(torch.float32)[:, None]).to(dtype)


def _rotate(t: Tensor, group: int, rotation: str) -> Tensor:
    if not group:
        return t
    return hadamard.butterflies(t, group) if rotation == "butterflies" else hadamard.rotate(t, group)


def forward(x: Tensor, q: Tensor, scale: Tensor, bias: Tensor | None, group: int = 0, rotation: str = "eager") -> Tensor:
    """`(int32(Q(x R) q^T) * s_x) * s_w (+ bias)` in fp32, each operation rounded on its own,
    rounded once to x's dtype; x R is rounded to x's dtype before it is quantized."""
    xq, xs = quantize_rows(_rotate(x, group, rotation))
    y = int_mm(xq, q.t()).to(torch.float32) * xs[:, None] * scale.to(torch.float32)[None, :]
    if bias is not None:
        y = y + bias.to(torch.float32)
    return y.to(x.dtype)


def dgrad(dy: Tensor, q: Tensor, scale: Tensor, mode: str, group: int = 0, rotation: str = "eager") -> Tensor:
    """int8: `Q(dy * scale) q` (int32) times dy's row scales; 16bit: `dy (q * scale)`, the
    weight-only input gradient; both rotated back when the base is a rotated one."""
    if mode not in DGRAD:
        raise ValueError(f"int8 dgrad {mode!r} not in {DGRAD}")
    if mode == "16bit":
        return _rotate(dy @ dequantize_weight(q, scale, dy.dtype), group, rotation)
    gq, gs = quantize_rows(dy, scale)
    return _rotate((int_mm(gq, q).to(torch.float32) * gs[:, None]).to(dy.dtype), group, rotation)
