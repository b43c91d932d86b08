"""Declarative support checks for `registry.register(..., supports=...)`.

`requires(...)` returns a function of the query that answers None ("can serve this") or the
first reason it cannot. Reasons are sentences for `registry.available()`; they name what was
asked and what would have been accepted. The reference keys its checks on a CUDA sm range
(`src/kohakumoss_kernels/constraints.py:10-31`); here a backend names the device kinds and arch
names it was written for.
"""

from __future__ import annotations

from collections.abc import Callable, Iterable

import torch

Check = Callable[[object], "str | None"]


def requires(kinds: Iterable[str] | None = None, archs: Iterable[str] | None = None, dtypes: Iterable[torch.dtype] | None = None,
             fp8: bool = False, mx: bool = False, extra: Check | Iterable[Check] = ()) -> Check:
    """kinds   device kinds served ("hip", "cpu")
    archs   arch names served ("gfx950")
    dtypes  activation dtypes served
    fp8/mx  the arch must have fp8 / block-scaled matrix instructions
    extra   one more check of the query, or several, run in order after the ones above"""
    kinds = None if kinds is None else tuple(kinds)
    archs = None if archs is None else tuple(archs)
    dtypes = None if dtypes is None else tuple(dtypes)
    rules: list[Check] = []
    if kinds is not None:
        rules.append(lambda q: None if q.arch.kind in kinds else f"device kind {q.arch.kind} is not one of {kinds}")
    if archs is not None:
        rules.append(lambda q: None if q.arch.name in archs else f"arch {q.arch.name} is not one of {archs}")
    if dtypes is not None:
        rules.append(lambda q: None if q.dtype in dtypes else f"dtype {q.dtype} is not one of {tuple(str(d) for d in dtypes)}")
    if fp8:
        rules.append(lambda q: None if q.arch.has_fp8 else f"arch {q.arch.name} has no fp8 matrix instructions")
    if mx:
        rules.append(lambda q: None if q.arch.has_mx else f"arch {q.arch.name} has no block-scaled matrix instructions")
    rules.extend([extra] if callable(extra) else list(extra))

    def supports(query) -> str | None:
        for rule in rules:
            why = rule(query)
            if why is not None:
                return why
        return None

    return supports
