"""Per-op dispatch: which backend serves an op on a device, and what happens when it cannot.

    register(op, backend, fn, supports)   a backend offers `fn` for `op`; `supports(query)` says why not, or None
    resolve(op, device, dtype, **static)  -> Bound: the first backend of the arch's priority list that
                                             is loaded, has not failed this query before, and supports it
    available(op, device, dtype, **static) -> {backend: None | reason}

A `Bound` is what a module keeps and calls. When its backend raises "cannot build / launch here"
it records the failure, moves itself and every live `Bound` of the same query to the next backend
and repeats the call there; a pinned backend (`resolve(..., backend=...)`), a device fault and an
out-of-memory condition are re-raised instead, and arguments the eager implementation rejects as
well are reported as the caller's `InputError`. Semantics of reference
`src/kohakumoss_kernels/registry.py:32-454`; the arch table here has `gfx950`, served by the `hip`
backend alone, so that an op on the GPU never ends up in torch code without anyone noticing.
"""

from __future__ import annotations

import importlib
import threading
import weakref
from collections.abc import Callable
from dataclasses import dataclass

import torch

from kohakumosstrainer_amd.kernels.arch import Arch, arch_of
from kohakumosstrainer_amd.kernels.errors import BackendUnavailable, InputError, LAUNCH_ERRORS, describe, is_build_error, is_sticky_error

BACKENDS = ("hip", "eager")
DEFAULT_PRIORITY: dict[str, tuple[str, ...]] = {"gfx950": ("hip",), "cpu": ("eager",)}
FALLBACK_PRIORITY = ("eager",)  # an arch without an entry of its own


class NoImplementationError(RuntimeError):
    """No backend serves the query; the message lists every backend's reason."""


@dataclass(frozen=True)
class OpQuery:
    """What a backend is asked to serve: the op, the arch-table entry of the device, the
    activation dtype and the op's static options as sorted `(name, value)` pairs."""

    op: str
    arch: Arch
    dtype: torch.dtype
    static: tuple[tuple[str, object], ...] = ()

    def get(self, key: str, default=None):
        return dict(self.static).get(key, default)

    def describe(self) -> str:
        opts = ", ".join(f"{k}={v}" for k, v in self.static)
        return f"{self.op}[{self.arch.name}, {self.dtype}{', ' + opts if opts else ''}]"


@dataclass(frozen=True)
class Impl:
    fn: Callable
    supports: Callable[[OpQuery], str | None] | None = None

    def reason(self, query: OpQuery) -> str | None:
        return None if self.supports is None else self.supports(query)


class _State:
    """Everything mutable, behind one lock: offers, priority overrides, backends that did not
    load, failures seen, and the live bound ops per query (so that siblings move together)."""

    def __init__(self):
        self.lock = threading.RLock()
        self.impls: dict[str, dict[str, Impl]] = {}
        self.priority: dict[str, tuple[str, ...]] = {}
        self.not_loaded: dict[str, str] = {}
        self.failed: dict[tuple, str] = {}
        self.live: dict[tuple, weakref.WeakSet] = {}
        self.loaded = False


_S = _State()


def _order_for(arch: Arch) -> tuple[str, ...]:
    if arch.name in _S.priority:
        return _S.priority[arch.name]
    return DEFAULT_PRIORITY.get(arch.name, FALLBACK_PRIORITY)


def _failure_key(query: OpQuery, backend: str) -> tuple:
    return (query.op, backend, query.arch.name, str(query.dtype), query.static)


def _why_not(backend: str, query: OpQuery) -> str | None:
    """None when `backend` can be bound for `query` right now."""
    if backend in _S.not_loaded:
        return _S.not_loaded[backend]
    impl = _S.impls.get(query.op, {}).get(backend)
    if impl is None:
        return f"backend {backend} does not implement {query.op}"
    seen = _S.failed.get(_failure_key(query, backend))
    if seen is not None:
        return f"failed earlier: {seen}"
    return impl.reason(query)


class Bound:
    """An op bound to one backend, callable like the backend's function. `order` is the chain it
    may walk (one entry when pinned), `backend` where it stands."""

    def __init__(self, query: OpQuery, device: torch.device, order: tuple[str, ...], backend: str, pinned: bool):
        self.query, self.device, self.order, self.pinned = query, device, order, pinned
        self._move_to(backend)
        with _S.lock:
            _S.live.setdefault((query, str(device)), weakref.WeakSet()).add(self)

    def _move_to(self, backend: str) -> None:
        self.backend = backend
        self._fn = _S.impls[self.query.op][backend].fn

    def __call__(self, *args, **kwargs):
        while True:
            try:
                return self._fn(*args, **kwargs)
            except LAUNCH_ERRORS as err:
                self.fall_back(err, args, kwargs)  # raises when there is nowhere to go

    def __getattr__(self, name: str):
        if name.startswith("_"):
            raise AttributeError(name)
        return getattr(self._fn, name)

    def __repr__(self) -> str:
        return f"<{self.query.describe()} on {self.backend} of {self.order}>"

    def fall_back(self, err: BaseException, args=None, kwargs=None) -> None:
        """Leave the current backend after `err`. Returns with the op (and its siblings) bound to
        the next usable backend, or raises: `err` itself when it must not be answered by moving on,
        `InputError` when the arguments are at fault, `NoImplementationError`-free `err` when the chain ends."""
        if self.pinned or not is_build_error(err) or is_sticky_error(err, self.device):
            raise err
        if not isinstance(err, BackendUnavailable) and args is not None:
            self._blame_arguments(err, args, kwargs or {})
        with _S.lock:
            _S.failed[_failure_key(self.query, self.backend)] = describe(err)
            left = self.backend
            here = self.order.index(left) if left in self.order else len(self.order)
            for candidate in self.order[here + 1 :]:
                if _why_not(candidate, self.query) is None:
                    for sibling in list(_S.live.get((self.query, str(self.device)), ())):
                        if sibling.backend == left and not sibling.pinned:
                            sibling._move_to(candidate)
                    return
        raise err

    def _blame_arguments(self, err: BaseException, args, kwargs) -> None:
        """Run the eager implementation on the same arguments: if it refuses them too, nothing is
        wrong with the backend."""
        eager = _S.impls.get(self.query.op, {}).get("eager")
        if eager is None or self.backend == "eager":
            return
        try:
            eager.fn(*args, **kwargs)
        except (ValueError, TypeError, IndexError, RuntimeError) as verdict:
            if isinstance(verdict, BackendUnavailable):
                return
            raise InputError(self.query.op, self.backend, err, verdict) from err


# ---- registration ---------------------------------------------------------------------------


def register(op: str, backend: str, fn: Callable, supports: Callable[[OpQuery], str | None] | None = None) -> None:
    with _S.lock:
        _S.impls.setdefault(op, {})[backend] = Impl(fn, supports)


def unregister(op: str, backend: str | None = None) -> None:
    """Withdraw one backend's offer for `op`, or every offer."""
    with _S.lock:
        if backend is None:
            _S.impls.pop(op, None)
        else:
            _S.impls.get(op, {}).pop(backend, None)


def mark_unavailable(backend: str, reason: str) -> None:
    """The backend as a whole cannot be used in this process (its library did not load)."""
    with _S.lock:
        _S.not_loaded[backend] = reason


def set_priority(arch_name: str, order: tuple[str, ...] | list[str]) -> None:
    with _S.lock:
        _S.priority[arch_name] = tuple(order)


def reset_priority() -> None:
    with _S.lock:
        _S.priority.clear()


def failures() -> dict[tuple, str]:
    with _S.lock:
        return dict(_S.failed)


def clear_failures() -> None:
    with _S.lock:
        _S.failed.clear()


# ---- queries ----------------------------------------------------------------------------------


def _query(op: str, device, dtype: torch.dtype, static: dict) -> tuple[OpQuery, torch.device]:
    device = torch.device(device)
    return OpQuery(op, arch_of(device), dtype, tuple(sorted(static.items()))), device


def available(op: str, device: torch.device | str, dtype: torch.dtype, **static) -> dict[str, str | None]:
    """Every backend that offers `op` or stands in the arch's priority list -> None (usable) or why not."""
    load_backends()
    query, _ = _query(op, device, dtype, static)
    with _S.lock:
        names = list(dict.fromkeys([*_order_for(query.arch), *_S.impls.get(op, {}), *BACKENDS]))
        return {name: _why_not(name, query) for name in names}


def resolve(op: str, device: torch.device | str, dtype: torch.dtype, backend: str | None = None, **static) -> Bound:
    load_backends()
    query, device = _query(op, device, dtype, static)
    with _S.lock:
        order = (backend,) if backend is not None else _order_for(query.arch)
        reasons = {}
        for name in order:
            reasons[name] = _why_not(name, query)
            if reasons[name] is None:
                return Bound(query, device, order, name, pinned=backend is not None)
    listing = "; ".join(f"{n}: {why}" for n, why in reasons.items())
    raise NoImplementationError(f"no backend serves {query.describe()} ({listing})")


# ---- backends ---------------------------------------------------------------------------------

_OP_MODULES = ("kohakumosstrainer_amd.kernels.fp8.op", "kohakumosstrainer_amd.kernels.quant", "kohakumosstrainer_amd.kernels.rotated",
               "kohakumosstrainer_amd.kernels.int8.op")
_BACKEND_MODULES = {"hip": "kohakumosstrainer_amd.kernels.backends.hip"}


def load_backends() -> None:
    """Import the op modules (each registers its eager launchers) and then the backends, once. A
    backend whose import fails is marked unavailable with the error as its reason."""
    if _S.loaded:
        return
    with _S.lock:
        if _S.loaded:
            return
        _S.loaded = True  # set first: the imports below call register()
        for module in _OP_MODULES:
            importlib.import_module(module)
        for name, module in _BACKEND_MODULES.items():
            try:
                importlib.import_module(module)
            except Exception as err:  # noqa: BLE001 - any import-time failure disables the backend, with its text
                mark_unavailable(name, describe(err))
