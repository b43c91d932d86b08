"""Weight-only quantized frozen bases: int8 or e4m3 codes with one fp32 scale per output row.

    quantize(w, fmt)          -> (q [N, K], scale [N])
    QuantWeight               a module holding them; `linear(x, bias)` = x @ (q * scale)^T + bias

`rotation` > 0 marks codes of `W R` (R the group Hadamard of that size: ConvRot files); the
linear then rotates x. `int8_dgrad` set ("int8" or "16bit") routes an int8 base through the int8
*compute* linear instead (activations quantized per row, integer GEMM). On the host the linear is
plain torch with a custom backward that keeps only `(q, scale)` alive; on a GPU it is the
registry's op. Replaces reference `src/kohakumoss/quant/weights.py:31-190`.
"""

from __future__ import annotations

import torch
from torch import Tensor, nn

from kohakumosstrainer_amd.kernels import hadamard, registry

FORMATS = ("int8", "fp8")
_LIMIT = {"int8": 127.0, "fp8": 448.0}
_FLOOR = 1e-12


def _hip_rows(w: Tensor) -> bool:
    if not (w.is_cuda and w.dtype in (torch.bfloat16, torch.float16)):
        return False
    from kohakumosstrainer_amd.kernels.arch import arch_of

    return arch_of(w.device).name == "gfx950"


def quantize(w: Tensor, fmt: str) -> tuple[Tensor, Tensor]:
    """Per-output-row symmetric quantizer. The scale is `max(amax, 1e-12) / limit` with the limit
    a Python number (127 for int8: codes round half to even; 448 for e4m3: one rounding of w / s)."""
    if fmt not in FORMATS:
        raise ValueError(f"quant format {fmt!r} not in {FORMATS}")
    if w.dim() == 2 and _hip_rows(w):
        # 16-bit weights on the card: the per-row quantizer kernels (same scale, same single rounding)
        from kohakumosstrainer_amd import native

        return native.quant_rows_i8(w.detach(), None) if fmt == "int8" else native.quant_rows(w.detach())
    v = w.detach().to(torch.float32)
    scale = v.abs().amax(dim=1).clamp_min(_FLOOR) / _LIMIT[fmt]
    ratio = v / scale.unsqueeze(1)
    if fmt == "int8":
        return torch.round(ratio).clamp_(-127.0, 127.0).to(torch.int8), scale
    return ratio.clamp_(-448.0, 448.0).to(torch.float8_e4m3fn), scale


def dequantize(q: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    return (q.to(torch.float32) * scale.to(torch.float32).unsqueeze(1)).to(dtype)


class _HostLinear(torch.autograd.Function):
    """x @ dequant(q, scale)^T on the host. The dequantized weight is rebuilt in backward: the
    graph holds the codes and the scale, never a 16-bit matrix."""

    @staticmethod
    def forward(ctx, x, q, scale, bias):
        ctx.save_for_backward(q, scale)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return torch.nn.functional.linear(x, dequantize(q, scale, x.dtype), None if bias is None else bias.to(x.dtype))

    @staticmethod
    def backward(ctx, grad):
        q, scale = ctx.saved_tensors
        dx = grad @ dequantize(q, scale, grad.dtype) if ctx.needs_input_grad[0] else None
        db = None
        if ctx.bias_dtype is not None and ctx.needs_input_grad[3]:
            db = grad.reshape(-1, grad.shape[-1]).to(torch.float32).sum(0).to(ctx.bias_dtype)
        return dx, None, None, db


class QuantWeight(nn.Module):
    """Codes and scales of a frozen weight as buffers, and the way to multiply by them."""

    def __init__(self, q: Tensor, scale: Tensor, fmt: str, rotation: int = 0, int8_dgrad: str | None = None):
        super().__init__()
        if fmt not in FORMATS:
            raise ValueError(f"quant format {fmt!r} not in {FORMATS}")
        if rotation:
            hadamard.stages(rotation)
        if int8_dgrad is not None and fmt != "int8":
            raise ValueError("the int8 compute linear needs an int8 base")
        self.fmt, self.rotation, self.int8_dgrad = fmt, int(rotation), int8_dgrad
        self.register_buffer("q", q)
        self.register_buffer("scale", scale.to(torch.float32))
        self._call = None
        self._bound_for = None

    @classmethod
    def from_weight(cls, w: Tensor, fmt: str) -> "QuantWeight":
        return cls(*quantize(w, fmt), fmt)

    def weight(self, dtype: torch.dtype) -> Tensor:
        """The dense weight this base stands for (rotated back when the codes are of W R)."""
        dense = dequantize(self.q, self.scale, torch.float32)
        if self.rotation:
            dense = hadamard.group_hadamard_eager(dense, self.rotation)  # R is its own inverse
        return dense.to(dtype)

    def materialize(self) -> Tensor:
        return self.weight(torch.float32)

    def bind(self, dtype: torch.dtype, device=None) -> None:
        """Pick how `linear` runs for `(device, dtype)`, once."""
        device = torch.device(device) if device is not None else self.q.device
        self._bound_for = (device, dtype)
        if self.int8_dgrad is not None:
            op = registry.resolve("int8_linear", device, dtype, group=self.rotation, dgrad=self.int8_dgrad)
            self._call = lambda x, bias: op(x, self.q, self.scale, bias, self.rotation, self.int8_dgrad)
        elif device.type == "cpu":
            self._call = self._on_host
        elif self.rotation:
            op = registry.resolve("quant_linear_rotated", device, dtype, fmt=self.fmt, group=self.rotation)
            self._call = lambda x, bias: op(x, self.q, self.scale, bias, self.fmt, self.rotation)
        else:
            op = registry.resolve("quant_linear", device, dtype, fmt=self.fmt)
            self._call = lambda x, bias: op(x, self.q, self.scale, bias, self.fmt)

    def _on_host(self, x: Tensor, bias: Tensor | None) -> Tensor:
        if self.rotation:
            x = hadamard.group_hadamard(x, self.rotation)
        return _HostLinear.apply(x, self.q, self.scale, bias)

    def linear(self, x: Tensor, bias: Tensor | None) -> Tensor:
        if self._call is None or self._bound_for != (x.device, x.dtype):
            self.bind(x.dtype, x.device)
        return self._call(x, bias)

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.q, self.scale))
