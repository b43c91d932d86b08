"""Quantize the frozen linears of a model in place: weight-only (int8 / fp8, `QuantWeight`) or
fp8 compute (fp8_compute / mxfp8, `ComputeWeight`); attach trainable fp8 compute caches.
Mirrors reference `src/kohakumoss/quant/convert.py:29-244` without the checkpoint-source
plumbing (weights are always quantized from the module's own parameter).
"""

from collections.abc import Callable

import torch
from torch import nn

from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant.compute import COMPUTE, ComputeCache, ComputeWeight, eligible, recipe_of
from kohakumosstrainer_amd.quant.weights import QuantWeight


def make_base(w: torch.Tensor, fmt: str, recipe: str = "row", dgrad: bool = False):
    """The quantized base of weight `w` under precision `fmt` (`recipe` and `dgrad` apply to
    fp8_compute / mxfp8)."""
    if fmt in COMPUTE:
        return ComputeWeight.from_weight(w, recipe_of(fmt, recipe), dgrad)
    return QuantWeight.from_weight(w, fmt)


def accepts(fmt: str, out_features: int, in_features: int) -> bool:
    """Whether a [N, K] weight can take `fmt` (fp8 compute needs aligned shapes)."""
    return fmt not in COMPUTE or eligible(out_features, in_features) is None


def default_filter(keep_fp32: tuple[str, ...], min_features: int = 256) -> Callable[[str, nn.Linear], bool]:
    """Quantize every linear except those under a kept name and small ones."""

    def accept(name: str, lin: nn.Linear) -> bool:
        if any(name == k or name.startswith(k + ".") for k in keep_fp32):
            return False
        return min(lin.in_features, lin.out_features) >= min_features

    return accept


class QuantLinear(nn.Module):
    """Inference replacement of a plain nn.Linear by a quantized weight (+ bias)."""

    def __init__(self, linear: nn.Linear, fmt: str, compute_dtype: torch.dtype, recipe: str = "row", work_device=None):
        super().__init__()
        self.in_features, self.out_features = linear.in_features, linear.out_features
        home = linear.weight.device
        self.qweight = make_base(linear.weight.detach().to(work_device or home), fmt, recipe).to(home)
        self.qweight.bind(compute_dtype)
        self.bias = None if linear.bias is None else nn.Parameter(linear.bias.detach(), requires_grad=False)

    @classmethod
    def from_base(cls, in_features: int, out_features: int, base, bias, compute_dtype: torch.dtype) -> "QuantLinear":
        """A QuantLinear over an already-quantized base."""
        self = cls.__new__(cls)
        nn.Module.__init__(self)
        self.in_features, self.out_features = in_features, out_features
        self.qweight = base
        self.qweight.bind(compute_dtype)
        self.bias = None if bias is None else nn.Parameter(bias, requires_grad=False)
        return self

    def forward(self, x):
        return self.qweight.linear(x, None if self.bias is None else self.bias.to(x.dtype))


@torch.no_grad()
def quantize_torch_linears(module: nn.Module, fmt: str, compute_dtype: torch.dtype, min_features: int = 256) -> int:
    """Replace every large plain nn.Linear inside `module` (e.g. a frozen text encoder);
    returns how many."""
    count = 0
    for name, child in list(module.named_children()):
        big = type(child) is nn.Linear and min(child.in_features, child.out_features) >= min_features
        if big and accepts(fmt, child.out_features, child.in_features):
            setattr(module, name, QuantLinear(child, fmt, compute_dtype))
            count += 1
        elif not big:
            count += quantize_torch_linears(child, fmt, compute_dtype, min_features)
    return count


@torch.no_grad()
def attach_compute(model: nn.Module, fmt: str, accept, compute_dtype: torch.dtype, recipe: str = "row", dgrad: bool = True) -> list[MossLinear]:
    """Trainable fp8 compute: a ComputeCache, quantized from the current weight, on every
    accepted dense MossLinear of an fp8-compute shape; returns those linears (their caches
    need `refresh` after every optimizer step)."""
    out = []
    for name, lin in list(model.named_modules()):
        if not isinstance(lin, MossLinear) or lin.base is not None:
            continue
        if not accept(name, lin) or not accepts(fmt, lin.out_features, lin.in_features):
            continue
        cache = ComputeCache(recipe_of(fmt, recipe), dgrad)
        cache.refresh(lin.weight)
        cache.bind(compute_dtype, lin.weight.device)
        lin.set_compute(cache)
        out.append(lin)
    return out


@torch.no_grad()
def quantize_model(model: nn.Module, fmt: str, accept=None, compute_dtype: torch.dtype | None = None, recipe: str = "row", dgrad: bool = False, work_device=None) -> dict[str, int]:
    """Replace accepted dense MossLinear bases with QuantWeight (int8 / fp8) or ComputeWeight
    (fp8_compute / mxfp8), quantizing on `work_device` (default: where the weight is); the dense
    parameter becomes an empty placeholder. Returns counts and bytes (`skipped`: accepted
    layers whose shape fp8 compute cannot take)."""
    accept = accept or default_filter(())
    report = {"layers": 0, "dense_bytes": 0, "quant_bytes": 0, "skipped": 0}
    for name, lin in list(model.named_modules()):
        if not isinstance(lin, MossLinear) or lin.base is not None or not accept(name, lin):
            continue
        if not accepts(fmt, lin.out_features, lin.in_features):
            report["skipped"] += 1
            continue
        w = lin.weight.detach()
        home = w.device
        base = make_base(w.to(work_device or home), fmt, recipe, dgrad).to(home)
        report["layers"] += 1
        report["dense_bytes"] += w.nbytes
        report["quant_bytes"] += base.nbytes()
        lin.weight = nn.Parameter(torch.empty(0, dtype=w.dtype, device=home), requires_grad=False)
        lin.set_base(base)
        base.bind(compute_dtype or w.dtype)
    return report
