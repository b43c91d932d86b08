"""Error statistics of a result against an fp64 truth, and the comparison of a kernel's error
with the eager path's on the same inputs (what `tuning` reports and the parity tests judge by).
Same quantities as reference `src/kohakumoss_kernels/error_stats.py:15-59`.
"""

from __future__ import annotations

import torch
from torch import Tensor

KEYS = ("cos_deficit", "abs_mean", "abs_median", "rel_mean", "rel_median")
PAIRS = (("abs_mean", "rel_mean"), ("abs_median", "rel_median"))


def _summary(values: Tensor) -> dict[str, float]:
    if values.numel() == 0:
        values = values.new_zeros(1)
    return {"mean": values.mean().item(), "median": values.median().item(), "min": values.min().item(), "max": values.max().item()}


def stats(out: Tensor, ref: Tensor) -> dict[str, float]:
    """Cosine to `ref`, and mean / median / min / max of the absolute error and of the error
    relative to |ref| where ref is not zero; everything in fp64."""
    got = out.detach().double().flatten()
    want = ref.detach().double().flatten()
    err = (got - want).abs()
    nz = want != 0
    table = {"finite": bool(torch.isfinite(got).all())}
    cosine = torch.nn.functional.cosine_similarity(got, want, dim=0).item() if got.numel() else 1.0
    table["cos"], table["cos_deficit"] = cosine, 1.0 - cosine
    for prefix, values in (("abs", err), ("rel", err[nz] / want[nz].abs())):
        table.update({f"{prefix}_{k}": v for k, v in _summary(values).items()})
    return table


def floors(out: Tensor, ref64: Tensor) -> dict[str, float]:
    """What one rounding step of `out`'s dtype amounts to in each statistic: an eager error below
    it is not a meaningful yardstick."""
    eps = float(torch.finfo(out.dtype).eps) if out.is_floating_point() else 0.0
    typical = ref64.detach().double().abs().flatten().median().item() if ref64.numel() else 0.0
    return {"cos_deficit": eps, "abs_mean": eps * typical, "abs_median": eps * typical, "rel_mean": eps, "rel_median": eps}


def compare(out: Tensor, eager: Tensor, ref64: Tensor) -> dict[str, dict]:
    return {"kernel": stats(out, ref64), "eager": stats(eager, ref64), "floor": floors(out, ref64)}


def worse(table: dict[str, dict], ratio: float = 10.0) -> list[str]:
    """The statistics on which the kernel is `ratio` times the eager path (or the rounding floor)
    off: the cosine on its own, absolute and relative error only when both of a pair are."""
    kernel, eager, floor = table["kernel"], table["eager"], table.get("floor", {})
    if eager["finite"] and not kernel["finite"]:
        return ["non-finite"]
    far = {k for k in KEYS if kernel[k] > 0 and kernel[k] > ratio * max(eager[k], floor.get(k, 0.0))}
    found = [k for k in ("cos_deficit",) if k in far]
    for a, b in PAIRS:
        if a in far and b in far:
            found += [a, b]
    return found
