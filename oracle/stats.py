"""Oracle (test infrastructure): the error statistics a result is judged by.

Restates reference `src/kohakumoss_kernels/error_stats.py:15-59` (the statistics) and
`tests/_util/error_stats.py:30-64` (the pass rule): against an fp64 truth a kernel
result regresses when it is non-finite where the eager result is finite, when its
cosine deficit is 10x the eager result's or more, or when both the absolute and the
relative error of the same summary (mean, or median) are; an eager statistic below one
rounding step of the output dtype counts as one rounding step.
"""

import torch
from torch import Tensor

SUMMARIES = ("cos_deficit", "abs_mean", "abs_median", "rel_mean", "rel_median")
PAIRED = (("abs_mean", "rel_mean"), ("abs_median", "rel_median"))
MAX_RATIO = 10.0


def stats(out: Tensor, truth: Tensor) -> dict[str, float]:
    """Cosine to `truth` and mean / median / min / max of |out-truth| and of
    |out-truth|/|truth| over the nonzero truth entries."""
    o = out.detach().to(torch.float64).flatten()
    t = truth.detach().to(torch.float64).flatten()
    err = (o - t).abs()
    nonzero = t != 0
    rel = err[nonzero] / t[nonzero].abs() if bool(nonzero.any()) else err.new_zeros(1)
    cos = F_cos(o, t) if o.numel() else 1.0
    row = {"finite": bool(torch.isfinite(o).all()), "cos": cos, "cos_deficit": 1.0 - cos}
    for name, v in (("abs", err), ("rel", rel)):
        v = v if v.numel() else err.new_zeros(1)
        row[f"{name}_mean"] = v.mean().item()
        row[f"{name}_median"] = v.median().item()
        row[f"{name}_min"] = v.min().item()
        row[f"{name}_max"] = v.max().item()
    return row


def F_cos(a: Tensor, b: Tensor) -> float:
    return torch.nn.functional.cosine_similarity(a, b, dim=0).item()


def floors(out: Tensor, truth: Tensor) -> dict[str, float]:
    """One rounding step of `out`'s dtype per statistic: eps * median|truth| for the
    absolute ones, eps for the relative ones and the cosine."""
    eps = torch.finfo(out.dtype).eps if out.is_floating_point() else 0.0
    mid = truth.detach().to(torch.float64).abs().flatten().median().item() if truth.numel() else 0.0
    return {
        "cos_deficit": eps,
        "abs_mean": eps * mid,
        "abs_median": eps * mid,
        "rel_mean": eps,
        "rel_median": eps,
    }


def compare(out: Tensor, eager: Tensor, truth: Tensor) -> dict[str, dict]:
    return {"kernel": stats(out, truth), "eager": stats(eager, truth), "floor": floors(out, truth)}


def regressions(table: dict[str, dict], ratio: float = MAX_RATIO) -> list[str]:
    k, e, floor = table["kernel"], table["eager"], table.get("floor", {})
    if not k["finite"] and e["finite"]:
        return ["non-finite"]
    away = {s for s in SUMMARIES if k[s] > ratio * max(e[s], floor.get(s, 0.0)) and k[s] > 0}
    bad = ["cos_deficit"] if "cos_deficit" in away else []
    for a, r in PAIRED:
        if a in away and r in away:
            bad += [a, r]
    return bad


def assert_no_regression(out: Tensor, eager: Tensor, truth: Tensor, name: str = "") -> dict:
    """Assert `out` is not 10x worse than `eager` against `truth`; returns the table."""
    assert truth.abs().max() > 0, f"{name}: the truth is all zero"
    table = compare(out, eager, truth)
    bad = regressions(table)
    assert not bad, f"{name}: regresses on {bad}: {table}"
    return table


def rel_l2(out: Tensor, truth: Tensor) -> float:
    """`||out - truth||_2 / ||truth||_2` in fp64 (the headline GEMM tolerance)."""
    o = out.detach().to(torch.float64)
    t = truth.detach().to(torch.float64)
    return ((o - t).norm() / t.norm()).item()
