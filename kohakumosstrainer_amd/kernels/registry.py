"""Per-op dispatch: backends register implementations, callers `resolve` once at build time
to a `Bound` op that walks the arch's backend priority when a backend turns out unable to run.

Mirrors the public interface of reference `src/kohakumoss_kernels/registry.py`
(`register / resolve / available / set_priority / Bound / OpQuery`, :50-72, :101-223,
:345-429). Backends here are `hip` (hand-written gfx950 kernels behind the C ABI) and `eager`
(the torch reference launchers, what a host-resident tensor runs). On `gfx950` the priority is
`("hip",)` alone: a GPU op never drops to torch behind the caller's back; if the HIP library is
missing or a launch fails, `resolve` / the call raises.
"""

import importlib
import threading
import weakref
from collections.abc import Callable
from dataclasses import dataclass, field

import torch

from kohakumosstrainer_amd.kernels.arch import Arch, arch_of
from kohakumosstrainer_amd.kernels.errors import (
    LAUNCH_ERRORS,
    BackendUnavailable,
    InputError,
    describe,
    is_sticky_error,
    unavailable,
)

BACKENDS = ("hip", "eager")
DEFAULT_PRIORITY: dict[str, tuple[str, ...]] = {
    "gfx950": ("hip",),
    "cpu": ("eager",),
}
CAUGHT = (BackendUnavailable, *LAUNCH_ERRORS)


class NoImplementationError(RuntimeError):
    """No registered backend can serve the query; the message lists every reason."""


@dataclass(frozen=True)
class OpQuery:
    """What a caller asks for: op name, arch, compute dtype and static options."""

    op: str
    arch: Arch
    dtype: torch.dtype
    static: tuple[tuple[str, object], ...] = ()

    def get(self, key: str, default=None):
        return dict(self.static).get(key, default)


@dataclass
class Impl:
    """One backend's implementation of one op; `supports(query)` gives a reason or None."""

    backend: str
    fn: Callable
    supports: Callable[[OpQuery], str | None] | None = None

    def reason(self, query: OpQuery) -> str | None:
        return None if self.supports is None else self.supports(query)


@dataclass
class _Tables:
    impls: dict[str, dict[str, Impl]] = field(default_factory=dict)
    unavailable: dict[str, str] = field(default_factory=dict)
    priority: dict[str, tuple[str, ...]] = field(default_factory=lambda: dict(DEFAULT_PRIORITY))
    failed: dict[tuple, str] = field(default_factory=dict)  # (op, backend, arch, dtype, static) -> why


_T = _Tables()
_LIVE: "weakref.WeakSet[Bound]" = weakref.WeakSet()
_load_lock = threading.RLock()
_loaded: list[bool] = []


def _priority(arch: Arch) -> tuple[str, ...]:
    order = _T.priority.get(arch.name)
    if order is None:
        raise NoImplementationError(f"no backend priority for arch {arch.name}: only gfx950 and the host are served")
    return order


class Bound:
    """A resolved op. Calling it runs the bound backend's implementation; a build / launch
    failure is recorded and the op, together with every live `Bound` of the same query on the
    failed backend, moves to the next backend of `order`. With no backend left (or a pinned
    one) the failure is raised."""

    def __init__(self, query: OpQuery, device, order: tuple[str, ...], backend: str):
        self.op, self.query, self.device, self.order = query.op, query, device, order
        self._bind(backend)
        _LIVE.add(self)

    def _bind(self, backend: str) -> None:
        self.backend = backend
        self.fn = _T.impls[self.op][backend].fn

    def __call__(self, *args, **kwargs):
        while True:
            try:
                return self.fn(*args, **kwargs)
            except CAUGHT as err:
                self.fall_back(err, args, kwargs)

    def __getattr__(self, name: str):
        if name in ("fn", "backend"):
            raise AttributeError(name)
        return getattr(self.fn, name)

    def fall_back(self, err: BaseException, args=None, kwargs=None) -> None:
        if is_sticky_error(err, self.device):
            raise err
        if args is not None and not isinstance(err, BackendUnavailable):  # a failed build says nothing about the inputs
            self._reject_bad_inputs(err, args, kwargs or {})
        err = unavailable(self.op, err, self.backend)
        _T.failed[_failure_key(self.query, self.backend)] = describe(err)
        rest = self.order[self.order.index(self.backend) + 1 :]
        if not rest:
            raise err
        try:
            name, _ = _first(self.query, self.device, rest)
        except NoImplementationError as none_left:
            raise none_left from err
        failed = self.backend
        for op in [o for o in list(_LIVE) if o.backend == failed and o.query == self.query and o.order == self.order]:
            op._bind(name)

    def _reject_bad_inputs(self, err: BaseException, args, kwargs) -> None:
        eager = _T.impls[self.op].get("eager")
        if eager is None or self.backend == "eager":
            return
        detached = [a.detach() if isinstance(a, torch.Tensor) else a for a in args]
        try:
            with torch.no_grad():
                eager.fn(*detached, **kwargs)
        except torch.OutOfMemoryError:
            return
        except Exception as rejected:  # noqa: BLE001 - any rejection by the reference counts
            raise InputError(self.op, self.backend, err, rejected) from err


def _failure_key(query: OpQuery, backend: str) -> tuple:
    return (query.op, backend, query.arch.name, query.dtype, query.static)


def register(op: str, backend: str, fn: Callable, supports: Callable[[OpQuery], str | None] | None = None) -> None:
    """Register `fn` as `backend`'s implementation of `op`."""
    _T.impls.setdefault(op, {})[backend] = Impl(backend, fn, supports)


def mark_unavailable(backend: str, reason: str) -> None:
    """Record why a whole backend cannot be used in this process."""
    _T.unavailable[backend] = reason


def set_priority(arch_name: str, order: tuple[str, ...] | list[str]) -> None:
    _T.priority[arch_name] = tuple(order)


def reset_priority() -> None:
    _T.priority.clear()
    _T.priority.update(DEFAULT_PRIORITY)


def failures() -> dict[tuple, str]:
    """`{(op, backend, arch, dtype, static): error}` recorded in this process."""
    return dict(_T.failed)


def clear_failures() -> None:
    _T.failed.clear()


def _reason(name: str, query: OpQuery, device) -> str | None:
    if name in _T.unavailable:
        return f"unavailable ({_T.unavailable[name]})"
    impl = _T.impls.get(query.op, {}).get(name)
    if impl is None:
        return "not implemented"
    why = impl.reason(query)
    if why is not None:
        return why
    failed = _T.failed.get(_failure_key(query, name))
    return None if failed is None else f"failed here ({failed[:300]})"


def _first(query: OpQuery, device, order: tuple[str, ...]) -> tuple[str, Impl]:
    reasons = []
    for name in order:
        why = _reason(name, query, device)
        if why is None:
            return name, _T.impls[query.op][name]
        reasons.append(f"{name}: {why}")
    raise NoImplementationError(f"{query.op} on {query.arch.name}/{query.dtype}: " + "; ".join(reasons))


def available(op: str, device: torch.device | str, dtype: torch.dtype, **static) -> dict[str, str | None]:
    """`{backend: None | reason}` for `op` on `device`."""
    load_backends()
    query = OpQuery(op, arch_of(device), dtype, tuple(sorted(static.items())))
    return {b: _reason(b, query, device) for b in BACKENDS}


def resolve(op: str, device: torch.device | str, dtype: torch.dtype, backend: str | None = None, **static) -> Bound:
    """The implementation of `op` for (device, dtype, static), resolved once; a pinned
    `backend` gets no fallback. The first call loads the backends."""
    load_backends()
    query = OpQuery(op, arch_of(device), dtype, tuple(sorted(static.items())))
    order = (backend,) if backend else _priority(query.arch)
    name, _ = _first(query, device, order)
    return Bound(query, device, order, name)


def load_backends() -> None:
    """Once per process: import the op modules (they register the eager launchers) and the
    backend packages; a backend whose import fails is marked unavailable with the reason."""
    if _loaded:
        return
    with _load_lock:
        if _loaded:
            return
        _loaded.append(True)
        for mod in ("fp8.op", "fp8.train", "quant", "hadamard", "rotated", "int8.op"):
            importlib.import_module(f"kohakumosstrainer_amd.kernels.{mod}")
        try:
            importlib.import_module("kohakumosstrainer_amd.kernels.backends.hip")
        except (ImportError, RuntimeError, OSError) as err:
            mark_unavailable("hip", describe(err))
