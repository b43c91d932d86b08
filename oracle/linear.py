"""Oracle (test infrastructure): the eager quantized linears on the CPU with torch.

fp8 compute linear   reference `src/kohakumoss_kernels/fp8/op.py:25-40`
bias / weight grads  reference `fp8/op.py:110-119`, `fp8/train.py:75-86`,
                     `backends/_master.py:35-38`
weight-only linear   reference `src/kohakumoss_kernels/quant/__init__.py:26-44`
weight quantizer     reference `src/kohakumoss/quant/weights.py:31-49`
LoRA bypass          reference `src/kohakumoss/adapters/bind/forwards.py:15-22` (the
                     arithmetic lives in the un-vendored `lycoris-lora>=4.1.3`; the closed
                     form `y = base(x) + gamma * (x A^T) B^T` is the one the reference's
                     `tests/adapters/test_stored_bypass.py:103-111` pins)
exact products       reference `tests/_util/fp8.py:30-46`
"""

import torch
import torch.nn.functional as F
from torch import Tensor

from oracle import formats

INT8_MAX = 127.0
FP8_MAX = 448.0
WEIGHT_FORMATS = ("int8", "fp8")


# ---- fp8 / MXFP8 compute linear -------------------------------------------------------


def fp8_forward(x, q, scale, aux, bias, recipe):
    """Quantize `x`, dequantize both operands to x's dtype, dense linear; the bias is
    cast to x's dtype first. `aux` (a vendor-layout scale copy) is not read."""
    xq, xs = formats.quantize(x, recipe, "act")
    a = formats.dequantize(xq, xs, recipe, x.dtype)
    w = formats.dequantize(q, scale, recipe, x.dtype)
    return F.linear(a, w, None if bias is None else bias.to(x.dtype))


def fp8_dgrad(dy, q, scale, q_t, scale_t, aux_t, recipe):
    """Input gradient: through the `[K, N]` copy quantized along N when one is stored
    (`dy` is quantized per call), else 16-bit `dy @ dequant(W)`."""
    if q_t is None:
        return dy @ formats.dequantize(q, scale, recipe, dy.dtype)
    gq, gs = formats.quantize(dy, recipe, "act")
    g = formats.dequantize(gq, gs, recipe, dy.dtype)
    return F.linear(g, formats.dequantize(q_t, scale_t, recipe, dy.dtype))


def bias_grad(dy: Tensor, dtype: torch.dtype) -> Tensor:
    """Column sum of the incoming gradient in fp32, stored in the bias dtype."""
    return dy.to(torch.float32).sum(0).to(dtype)


def weight_grad(dy: Tensor, x: Tensor, dtype: torch.dtype) -> Tensor:
    """`dy^T x` of 16-bit operands accumulated in fp32, stored in `dtype`. The reference
    asks the BLAS for an fp32-accumulated product with `out_dtype`; on the CPU that is
    the fp32 matmul of the exactly widened operands."""
    return (dy.to(torch.float32).t() @ x.to(torch.float32)).to(dtype)


def exact64(q: Tensor, scale: Tensor, recipe: str) -> Tensor:
    """The exact fp64 value `q * scale` of every element of a quantized operand."""
    rows, k = q.shape
    r = torch.arange(rows)[:, None]
    c = torch.arange(k)[None, :]
    v = q.to(torch.float64)
    if recipe == "tensor":
        return v * scale.to(torch.float64).reshape(())
    if recipe == "row":
        return v * scale.to(torch.float64)[:, None]
    if recipe == "mx":
        return v * torch.pow(2.0, scale.to(torch.float64)[r, c // 32] - 127)
    if scale.shape[0] == rows:
        return v * scale.to(torch.float64)[r, c // 128]
    return v * scale.to(torch.float64)[r // 128, c // 128]


# ---- weight-only int8 / fp8 linear ----------------------------------------------------


def quantize_weight(w: Tensor, fmt: str) -> tuple[Tensor, Tensor]:
    """Per-output-row quantizer of a frozen base: `(q, scale[N] fp32)`. int8 rounds
    `w / s` half to even and clips to +-127 with `s = max(amax, 1e-12) / 127`; fp8 rounds
    `w / s` once to e4m3 with `s = max(amax, 1e-12) / 448` (here the divisor is a Python
    scalar, as in the reference's module quantizer)."""
    v = w.detach().to(torch.float32)
    amax = v.abs().amax(dim=1).clamp_min(1e-12)
    if fmt == "int8":
        s = amax / INT8_MAX
        q = torch.round(v / s[:, None]).clamp_(-INT8_MAX, INT8_MAX)
        return q.to(torch.int8), s
    if fmt == "fp8":
        s = amax / FP8_MAX
        q = (v / s[:, None]).clamp_(-FP8_MAX, FP8_MAX)
        return q.to(torch.float8_e4m3fn), s
    raise ValueError(f"quant format {fmt!r} not in {WEIGHT_FORMATS}")


def dequantize_weight(q: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    """`q * scale[:, None]` in fp32 rounded once to `dtype`."""
    return (q.to(torch.float32) * scale.to(torch.float32)[:, None]).to(dtype)


def wo_forward(x: Tensor, q: Tensor, scale: Tensor, bias: Tensor | None) -> Tensor:
    """Weight-only forward: the weight is rounded to x's dtype before the matmul."""
    b = None if bias is None else bias.to(x.dtype)
    return F.linear(x, dequantize_weight(q, scale, x.dtype), b)


def wo_dgrad(dy: Tensor, q: Tensor, scale: Tensor) -> Tensor:
    return dy @ dequantize_weight(q, scale, dy.dtype)


def wo_exact64(q: Tensor, scale: Tensor) -> Tensor:
    return q.to(torch.float64) * scale.to(torch.float64)[:, None]


# ---- LoRA bypass over a quantized base ------------------------------------------------


def lora_bypass(base_y: Tensor, x: Tensor, down: Tensor, up: Tensor, gamma: float):
    """`base(x) + gamma * (x down^T) up^T`, the factors cast to x's dtype per call;
    `down` is `[r, K]`, `up` is `[N, r]`."""
    d = down.to(x.dtype)
    u = up.to(x.dtype)
    return base_y + F.linear(F.linear(x, d), u) * gamma
