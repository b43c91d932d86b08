"""Error statistics of a result against an fp64 reference, next to the same statistics of
the eager reference: cosine deficit and mean / median / min / max of the absolute and the
relative error (interface of reference `src/kohakumoss_kernels/error_stats.py:15-59`)."""

import torch
from torch import Tensor

KEYS = ("cos_deficit", "abs_mean", "abs_median", "rel_mean", "rel_median")
PAIRS = (("abs_mean", "rel_mean"), ("abs_median", "rel_median"))


def stats(out: Tensor, ref: Tensor) -> dict[str, float]:
    o, r = out.detach().double().flatten(), ref.detach().double().flatten()
    err = (o - r).abs()
    keep = r != 0
    rel = err[keep] / r[keep].abs() if bool(keep.any()) else err.new_zeros(1)
    cos = torch.nn.functional.cosine_similarity(o, r, dim=0).item() if o.numel() else 1.0
    row = {"finite": bool(torch.isfinite(o).all()), "cos": cos, "cos_deficit": 1.0 - cos}
    for name, v in (("abs", err if err.numel() else err.new_zeros(1)), ("rel", rel)):
        row.update({f"{name}_mean": v.mean().item(), f"{name}_median": v.median().item(), f"{name}_min": v.min().item(), f"{name}_max": v.max().item()})
    return row


def floors(out: Tensor, ref64: Tensor) -> dict[str, float]:
    eps = torch.finfo(out.dtype).eps if out.is_floating_point() else 0.0
    mid = ref64.detach().double().abs().flatten().median().item() if ref64.numel() else 0.0
    return {"cos_deficit": eps, "abs_mean": eps * mid, "abs_median": eps * mid, "rel_mean": eps, "rel_median": eps}


def compare(out: Tensor, eager: Tensor, ref64: Tensor) -> dict[str, dict]:
    return {"kernel": stats(out, ref64), "eager": stats(eager, ref64), "floor": floors(out, ref64)}


def worse(table: dict[str, dict]) -> list[str]:
    k, e = table["kernel"], table["eager"]
    out = [s for s in k if s not in ("finite", "cos") and s in e and k[s] > e[s]]
    return ["non-finite", *out] if e.get("finite", True) and not k.get("finite", True) else out
