"""Quantized frozen base weights (per-output-row scales) as MossLinear base storage.

int8: q = round(w / s) clamped to [-127, 127], s = max|w_row| / 127.
fp8 (e4m3fn): q = fp8(w / s), s = max|w_row| / 448.
`linear` is bound once per (device, dtype): on the host the plain-op composition (dequantize,
then a dense linear, saving only `q` / `scale` for the input gradient); on a GPU the
`quant_linear` op the registry resolves (the HIP dequant-GEMM on gfx950) or, for an int8 base
with `int8_dgrad` set (int8 compute), the `int8_linear` op (activations quantized per row, int8
MFMA GEMM). `rotation` > 0 marks a ConvRot base: the stored codes are those of W R with
R = blockdiag(H_rotation) over K, and the linear rotates x first (`quant_linear_rotated`, or the
`group` of `int8_linear`). Mirrors reference `src/kohakumoss/quant/weights.py:31-140,159-202`.
"""

from functools import partial

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from kohakumosstrainer_amd.kernels import registry

FP8_MAX = 448.0
INT8_MAX = 127.0
FORMATS = ("int8", "fp8")


def quantize(w: Tensor, fmt: str) -> tuple[Tensor, Tensor]:
    """`(q, scale[out])` of a 2-D weight; scale is fp32."""
    v = w.detach().float()
    amax = v.abs().amax(dim=1).clamp_min(1e-12)
    if fmt == "int8":
        scale = amax / INT8_MAX
        return torch.round(v / scale[:, None]).clamp_(-INT8_MAX, INT8_MAX).to(torch.int8), scale
    if fmt == "fp8":
        scale = amax / FP8_MAX
        return (v / scale[:, None]).clamp_(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn), scale
    raise ValueError(f"quant format {fmt!r} not in {FORMATS}")


def dequantize(q: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    return (q.to(torch.float32) * scale.float()[:, None]).to(dtype)


class QuantWeight(nn.Module):
    """BaseWeight holding `q` and `scale` as buffers (they follow `.to(device)`); `int8_dgrad`
    is None (weight-only) or the input-gradient mode of int8 compute ("int8" | "16bit")."""

    def __init__(self, q: Tensor, scale: Tensor, fmt: str, rotation: int = 0, int8_dgrad: str | None = None):
        super().__init__()
        if fmt not in FORMATS:
            raise ValueError(f"quant format {fmt!r} not in {FORMATS}")
        if int8_dgrad is not None and fmt != "int8":
            raise ValueError("int8 compute needs an int8 base")
        self.fmt = fmt
        self.rotation = int(rotation)
        self.int8_dgrad = int8_dgrad
        self.register_buffer("q", q)
        self.register_buffer("scale", scale.float())
        self.shape = q.shape
        self._linear = _host_linear

    @classmethod
    def from_weight(cls, w: Tensor, fmt: str) -> "QuantWeight":
        return cls(*quantize(w, fmt), fmt)

    def weight(self, dtype: torch.dtype) -> Tensor:
        """W in `dtype` (the rotation undone: W = (q * s) R, R its own inverse)."""
        if not self.rotation:
            return dequantize(self.q, self.scale, dtype)
        from kohakumosstrainer_amd.kernels.hadamard import group_hadamard_eager

        return group_hadamard_eager(dequantize(self.q, self.scale, torch.float32), self.rotation).to(dtype)

    def materialize(self) -> Tensor:
        return self.weight(torch.float32)

    def bind(self, dtype: torch.dtype, device=None) -> None:
        """Bind `linear` for (device, dtype) once."""
        device = self.q.device if device is None else torch.device(device)
        if device.type == "cpu":
            self._linear = _host_linear
            return
        if self.int8_dgrad is not None:
            kernel = registry.resolve("int8_linear", device, dtype, group=self.rotation, dgrad=self.int8_dgrad)
            self._linear = partial(_int8_linear, kernel)
            return
        if self.rotation:
            kernel = registry.resolve("quant_linear_rotated", device, dtype, fmt=self.fmt, group=self.rotation)
            self._linear = partial(_rotated_linear, kernel)
            return
        kernel = registry.resolve("quant_linear", device, dtype, fmt=self.fmt)
        self._linear = partial(_kernel_linear, kernel)

    def linear(self, x: Tensor, bias: Tensor | None) -> Tensor:
        """x W^T (+ bias) through the bound implementation."""
        return self._linear(self, x, bias)

    def nbytes(self) -> int:
        return self.q.nbytes + self.scale.numel() * 4


class _HostLinear(torch.autograd.Function):
    """Dequantize for this call, dense linear; only `q` / `scale` are saved."""

    @staticmethod
    def forward(ctx, x, q, scale, bias):
        ctx.save_for_backward(q, scale)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return F.linear(x, dequantize(q, scale, x.dtype), None if bias is None else bias.to(x.dtype))

    @staticmethod
    def backward(ctx, grad):
        q, scale = ctx.saved_tensors
        gx = grad @ dequantize(q, scale, grad.dtype) if ctx.needs_input_grad[0] else None
        gb = grad.float().sum(0).to(ctx.bias_dtype) if ctx.bias_dtype is not None and ctx.needs_input_grad[3] else None
        return gx, None, None, gb


def _host_linear(qw: QuantWeight, x: Tensor, bias: Tensor | None) -> Tensor:
    if qw.rotation:
        from kohakumosstrainer_amd.kernels.rotated import quant_linear_rotated_eager

        return quant_linear_rotated_eager(x, qw.q, qw.scale, bias, qw.fmt, qw.rotation)
    lead = x.shape[:-1]
    y = _HostLinear.apply(x.reshape(-1, x.shape[-1]), qw.q, qw.scale, bias)
    return y.reshape(*lead, qw.q.shape[0])


def _kernel_linear(kernel, qw: QuantWeight, x: Tensor, bias: Tensor | None) -> Tensor:
    return kernel(x, qw.q, qw.scale, bias, qw.fmt)


def _rotated_linear(kernel, qw: QuantWeight, x: Tensor, bias: Tensor | None) -> Tensor:
    return kernel(x, qw.q, qw.scale, bias, qw.fmt, qw.rotation)


def _int8_linear(kernel, qw: QuantWeight, x: Tensor, bias: Tensor | None) -> Tensor:
    return kernel(x, qw.q, qw.scale, bias, qw.rotation, qw.int8_dgrad)
