"""Turning a model's linears into quantized ones.

    make_base(w, fmt, ...)           a QuantWeight (int8 / fp8) or ComputeWeight (fp8_compute / mxfp8)
    quantize_model(model, fmt, ...)  every accepted MossLinear gets a frozen base; returns a report
    attach_compute(model, fmt, ...)  every accepted MossLinear keeps its weight and gets an fp8 cache
    QuantLinear / quantize_torch_linears   the same for plain nn.Linear modules (text encoder)

A layer is accepted when the filter says so (`default_filter`: not a kept-fp32 name, both sides at
least `min_features`) and, for compute precisions, when its shape tiles by 128.
Replaces reference `src/kohakumoss/quant/convert.py:29-244`.
"""

from __future__ import annotations

from collections.abc import Callable

import torch
from torch import nn

from kohakumosstrainer_amd.model.linear import MossLinear, placeholder
from kohakumosstrainer_amd.quant.bind import work_device as default_work_device
from kohakumosstrainer_amd.quant.compute import COMPUTE, ComputeCache, ComputeWeight, eligible, recipe_of
from kohakumosstrainer_amd.quant.weights import FORMATS, QuantWeight

PRECISIONS = (*FORMATS, *COMPUTE)


def make_base(w: torch.Tensor, fmt: str, recipe: str = "row", dgrad: bool = False):
    if fmt in COMPUTE:
        return ComputeWeight.from_weight(w, recipe_of(fmt, recipe), dgrad)
    if fmt in FORMATS:
        return QuantWeight.from_weight(w, fmt)
    raise ValueError(f"base precision {fmt!r} not in {PRECISIONS}")


def accepts(fmt: str, out_features: int, in_features: int) -> bool:
    """Shape rule of a precision: compute bases need both sides to tile by 128."""
    return fmt not in COMPUTE or eligible(out_features, in_features) is None


def default_filter(keep_fp32: tuple[str, ...], min_features: int = 256) -> Callable[[str, nn.Linear], bool]:
    """Accept a linear unless it is one of `keep_fp32` or lies under one (`name == key` or
    `name` starts with `key.`; a name that merely contains a key is not kept), or it is narrower
    than `min_features` on either side."""

    def accept(name: str, lin: nn.Linear) -> bool:
        if any(name == key or name.startswith(key + ".") for key in keep_fp32):
            return False
        return min(lin.in_features, lin.out_features) >= min_features

    return accept


class QuantLinear(nn.Module):
    """A plain `nn.Linear` replaced by a quantized base and its (dense) bias. The base is the
    submodule `qweight`: state keys are `qweight.q`, `qweight.scale`, ... and `bias`."""

    def __init__(self, linear: nn.Linear, fmt: str, compute_dtype: torch.dtype, recipe: str = "row", work_device=None):
        super().__init__()
        where = linear.weight.device if work_device is None else torch.device(work_device)
        base = make_base(linear.weight.detach().to(where), fmt, recipe).to(linear.weight.device)
        self._adopt(linear.in_features, linear.out_features, base, linear.bias, compute_dtype)

    def _adopt(self, in_features, out_features, base, bias, compute_dtype) -> None:
        self.in_features, self.out_features, self.compute_dtype = in_features, out_features, compute_dtype
        self.qweight = base
        base.bind(compute_dtype)
        self.bias = None if bias is None else nn.Parameter(bias.detach().clone(), requires_grad=False)

    @classmethod
    def from_base(cls, in_features: int, out_features: int, base, bias, compute_dtype: torch.dtype) -> "QuantLinear":
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self._adopt(in_features, out_features, base, bias, compute_dtype)
        return self

    def forward(self, x):
        bias = None if self.bias is None else self.bias.to(x.dtype)
        return self.qweight.linear(x, bias)


def _walk_children(module: nn.Module, prefix: str = ""):
    for name, child in module.named_children():
        path = f"{prefix}.{name}" if prefix else name
        yield module, name, path, child
        yield from _walk_children(child, path)


@torch.no_grad()
def quantize_torch_linears(module: nn.Module, fmt: str, compute_dtype: torch.dtype, min_features: int = 256) -> int:
    """Replace every plain `nn.Linear` under `module` that passes the size and shape rules by a
    `QuantLinear`; returns how many were replaced."""
    accept = default_filter((), min_features)
    swaps = [(parent, name, child) for parent, name, path, child in _walk_children(module)
             if type(child) is nn.Linear and accept(path, child) and accepts(fmt, child.out_features, child.in_features)]
    for parent, name, child in swaps:
        setattr(parent, name, QuantLinear(child, fmt, compute_dtype))
    return len(swaps)


def _accepted(model: nn.Module, fmt: str, accept) -> tuple[list[tuple[str, MossLinear]], int]:
    taken, skipped = [], 0
    for path, layer in model.named_modules():
        if not isinstance(layer, MossLinear) or not layer.is_plain:
            continue
        if accept is not None and not accept(path, layer):
            continue
        if accepts(fmt, layer.out_features, layer.in_features):
            taken.append((path, layer))
        else:
            skipped += 1
    return taken, skipped


@torch.no_grad()
def attach_compute(model: nn.Module, fmt: str, accept, compute_dtype: torch.dtype, recipe: str = "row", dgrad: bool = True) -> list[MossLinear]:
    """Give every accepted trainable MossLinear an fp8 cache of its weight (quantized now; the
    trainer refreshes it after each optimizer step). Returns the layers that got one."""
    if fmt not in COMPUTE:
        raise ValueError(f"compute precision {fmt!r} not in {COMPUTE}")
    taken, _ = _accepted(model, fmt, accept)
    for _, layer in taken:
        cache = ComputeCache(recipe_of(fmt, recipe), dgrad)
        cache.refresh(layer.weight)
        cache.bind(compute_dtype, layer.weight.device)
        layer.set_compute(cache)
    return [layer for _, layer in taken]


@torch.no_grad()
def quantize_model(model: nn.Module, fmt: str, accept=None, compute_dtype: torch.dtype | None = None, recipe: str = "row", dgrad: bool = False, work_device=None) -> dict:
    """Swap the weight of every accepted MossLinear for a frozen base. Quantization runs on
    `work_device` (default: the layer's own device if it is a GPU); the base ends up where the
    layer was. Report: layers converted, layers skipped for their shape, bytes before / after."""
    if fmt not in PRECISIONS:
        raise ValueError(f"base precision {fmt!r} not in {PRECISIONS}")
    taken, skipped = _accepted(model, fmt, accept if accept is not None else default_filter(()))
    dense_bytes = quant_bytes = 0
    for _, layer in taken:
        home = layer.weight.device
        where = default_work_device(home) if work_device is None else torch.device(work_device)
        dense_bytes += layer.weight.numel() * layer.weight.element_size()
        base = make_base(layer.weight.detach().to(where), fmt, recipe, dgrad).to(home)
        quant_bytes += base.nbytes()
        layer.weight = placeholder(layer.weight)
        layer.set_base(base)
        if compute_dtype is not None:
            base.bind(compute_dtype, home)
    return {"layers": len(taken), "skipped": skipped, "dense_bytes": dense_bytes, "quant_bytes": quant_bytes, "format": fmt}
