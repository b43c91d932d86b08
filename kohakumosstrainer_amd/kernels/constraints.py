"""Declarative `supports(query)` builders shared by backends (reference
`src/kohakumoss_kernels/constraints.py:10-31`)."""

from collections.abc import Callable

import torch


def requires(
    kinds: tuple[str, ...] = ("hip",),
    archs: tuple[str, ...] | None = None,
    dtypes: tuple[torch.dtype, ...] = (torch.float16, torch.bfloat16),
    extra: Callable | None = None,
) -> Callable:
    """A `supports` function gating on device kind, arch name, dtype and an extra check;
    it returns None when the query is served, else the reason."""

    def supports(query) -> str | None:
        arch = query.arch
        if arch.kind not in kinds:
            return f"device kind {arch.kind} not in {kinds}"
        if archs is not None and arch.name not in archs:
            return f"{arch.name} not in {archs}"
        if query.dtype not in dtypes:
            return f"dtype {query.dtype} not in {dtypes}"
        if query.dtype == torch.bfloat16 and not arch.has_bf16:
            return f"{arch.name} has no bf16"
        return None if extra is None else extra(query)

    return supports
