"""Quantizing the plain `nn.Linear`s of a frozen text encoder.

    per output channel (`group` 0)   `QuantLinear` over a `QuantWeight` (int8 / fp8, the weight-only
                                      kernels) or a `ComputeWeight` (fp8_compute / mxfp8, the fp8 op)
    per `group` input columns         `GroupQuantLinear`: codes `[out, in]`, scales `[out, in / group]`,
                                      the weight widened to the activation's type on every call

`linear_fate` says what happens to one module; `quantize_text_linears` does it to every linear under a
module and reports counts and bytes. The reference can also quantize from the values a checkpoint
stores instead of the loaded weight (`source=`); that loader is not part of this package, so only the
loaded weight is ever read here.
Replaces reference `src/kohakumoss/quant/text.py:31-152`.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from kohakumosstrainer_amd.quant.compute import COMPUTE
from kohakumosstrainer_amd.quant.convert import QuantLinear, accepts

_CODES = {"int8": (torch.int8, 127.0), "fp8": (torch.float8_e4m3fn, 448.0)}


def _format(fmt: str) -> tuple[torch.dtype, float]:
    try:
        return _CODES[fmt]
    except KeyError:
        raise ValueError(f"group quantization takes {tuple(_CODES)}, got {fmt!r}") from None


def quantize_groups(w: Tensor, fmt: str, group: int) -> tuple[Tensor, Tensor]:
    """`(q [out, in], scale [out, in / group] fp32)`: one scale `max(amax, 1e-12) / limit` per run of
    `group` input columns; int8 codes round half to even and clamp to +-127, e4m3 codes are the
    quotient clamped to +-448 and rounded once."""
    dtype, limit = _format(fmt)
    if w.dim() != 2 or group <= 0 or w.shape[1] % group:
        raise ValueError(f"a [out, in] weight with in % group == 0 is needed, got {tuple(w.shape)} and group {group}")
    runs = w.detach().to(torch.float32).unflatten(1, (-1, group))
    scale = runs.abs().amax(dim=-1).clamp_min(1e-12) / limit
    ratio = runs / scale.unsqueeze(-1)
    if fmt == "int8":
        ratio = torch.round(ratio)
    return ratio.clamp_(-limit, limit).flatten(1).to(dtype), scale


def dequantize_groups(q: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    """`q * scale` per group in fp32, rounded once to `dtype`."""
    group = q.shape[1] // scale.shape[1]
    return (q.to(torch.float32).unflatten(1, (-1, group)) * scale.unsqueeze(-1)).flatten(1).to(dtype)


class GroupQuantLinear(nn.Module):
    """`y = x W^T + b` with W stored as per-group codes and widened on every call."""

    def __init__(self, linear: nn.Linear, fmt: str, group: int):
        super().__init__()
        self.in_features, self.out_features = linear.in_features, linear.out_features
        q, scale = quantize_groups(linear.weight, fmt, group)
        self.register_buffer("q", q.to(linear.weight.device))
        self.register_buffer("scale", scale.to(linear.weight.device))
        self.bias = None if linear.bias is None else nn.Parameter(linear.bias.detach(), requires_grad=False)

    def forward(self, x: Tensor) -> Tensor:
        bias = None if self.bias is None else self.bias.to(x.dtype)
        return F.linear(x, dequantize_groups(self.q, self.scale, x.dtype), bias)


def linear_fate(module: nn.Module, precision: str, group: int, min_features: int = 256) -> str | None:
    """What `quantize_text_linears` does with `module`: "quantize"; "skip" (a large plain linear
    whose shape the fp8 compute op cannot take); None (not a plain linear, too small, or its input
    width is no multiple of the group: left as it is)."""
    if type(module) is not nn.Linear or min(module.in_features, module.out_features) < min_features:
        return None
    if group and module.in_features % group:
        return None
    return "quantize" if accepts(precision, module.out_features, module.in_features) else "skip"


def quantizes(module: nn.Module, precision: str, group: int, min_features: int = 256) -> bool:
    """Whether `quantize_text_linears` would replace anything under `module`."""
    return any(linear_fate(m, precision, group, min_features) == "quantize" for m in module.modules())


@torch.no_grad()
def quantize_text_linears(module: nn.Module, precision: str, group: int, compute_dtype: torch.dtype, min_features: int = 256,
                          recipe: str = "row", work_device=None) -> dict[str, int]:
    """Replace, in place, every plain `nn.Linear` under `module` whose fate is "quantize": per-group
    storage when `group` is set and the precision is weight-only, a `QuantLinear` otherwise (quantized
    on `work_device`). Each dense linear is let go as soon as it is replaced. Returns `layers`,
    `dense_bytes`, `quant_bytes` and `skipped` (large linears fp8 compute could not take)."""
    report = {"layers": 0, "dense_bytes": 0, "quant_bytes": 0, "skipped": 0}
    holders = [m for m in module.modules() if type(m) is not nn.Linear]
    for holder in holders:
        for name, child in list(holder.named_children()):
            fate = linear_fate(child, precision, group, min_features)
            if fate == "skip":
                report["skipped"] += 1
            if fate != "quantize":
                continue
            if group and precision not in COMPUTE:
                new = GroupQuantLinear(child, precision, group)
            else:
                new = QuantLinear(child, precision, compute_dtype, recipe, work_device)
            report["layers"] += 1
            report["dense_bytes"] += child.weight.numel() * child.weight.element_size()
            report["quant_bytes"] += sum(t.numel() * t.element_size() for t in new.buffers())
            setattr(holder, name, new)
            del child, new
    return report
