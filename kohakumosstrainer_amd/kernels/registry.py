"""Per-op dispatch: which backend serves an op on a device, and what happens when it cannot.

    register(op, backend, fn, supports)   a backend offers `fn` for `op`; `supports(query)` says why not, or None
    resolve(op, device, dtype, **static)  -> Bound: the first backend of the arch's priority list that
                                             is loaded, has not failed this query before, and supports it
    available(op, device, dtype, **static) -> {backend: None | reason}

A `Bound` is what a module keeps and calls. When its backend raises "cannot build / launch here"
it records the failure, moves itself and every live `Bound` of the same query to the next backend
and repeats the call there; a pinned backend (`resolve(..., backend=...)`), a device fault and an
out-of-memory condition are re-raised instead, and arguments the eager implementation rejects as
well are reported as the caller's `InputError`. The same holds for a failure inside backward: while
a `Bound` still has a backend to give way to, a call that records an autograd graph runs under a
guard whose backward, if the backend fails there, moves the op on and computes forward and backward
again through the next backend from the saved inputs (`settle_guards` lifts the guard once a
backward has gone through; `exercise` does all of that on scratch inputs at build time). Failures of
the toolchain class met at build time are kept on disk and not tried again by a later process with
the same library and torch. Semantics of reference `src/kohakumoss_kernels/registry.py:32-454` and
`status.py:42-133`; the arch table here has `gfx950`, served by the `hip` backend alone, so that an
op on the GPU never ends up in torch code without anyone noticing.
"""

from __future__ import annotations

import hashlib
import importlib
import json
import os
import threading
import time
import weakref
from collections.abc import Callable
from contextlib import contextmanager
from dataclasses import dataclass
from pathlib import Path

import torch

from kohakumosstrainer_amd.kernels.arch import Arch, arch_of
from kohakumosstrainer_amd.kernels.errors import BackendUnavailable, InputError, LAUNCH_ERRORS, describe, is_build_error, is_sticky_error, is_toolchain_error

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
        self.build_depth = 0  # inside `build_phase()`: toolchain failures go to disk
        self.disk: dict[str, dict] | None = None  # failures of earlier processes, read once
        self.proven: weakref.WeakSet = weakref.WeakSet()  # guarded ops whose backward went through


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
    kept = _disk_records().get(_disk_key(query, backend))
    if kept is not None:
        return f"failed in an earlier process: {kept.get('error', '?')}"
    return impl.reason(query)


# ---- failures that outlive the process ----------------------------------------------------------
# Only what would fail the same way next time: a build / toolchain failure (`is_toolchain_error`) met
# at build time (`build_phase`, the prewarm). A record holds for one fingerprint: the kernel library's
# file (size and modification time), the torch version and the Python version.


def _status_path() -> Path:
    root = os.environ.get("KOHAKUMOSS_KERNEL_CACHE")
    base = Path(root) if root else Path.home() / ".cache" / "kohakumoss_kernels"
    return base / "failures" / "backends.json"


def fingerprint() -> str:
    from kohakumosstrainer_amd import native

    try:
        st = native.LIB_PATH.stat()
        lib = f"{st.st_size}:{st.st_mtime_ns}"
    except OSError:
        lib = "no-library"
    import sys

    return hashlib.sha1(f"{lib}|{torch.__version__}|{sys.version.split()[0]}".encode()).hexdigest()[:12]


def _disk_key(query: OpQuery, backend: str) -> str:
    options = ",".join(f"{k}={v}" for k, v in query.static) or "-"
    return "|".join((query.op, backend, query.arch.name, str(query.dtype), options))


def _disk_records() -> dict[str, dict]:
    if _S.disk is None:
        try:
            raw = json.loads(_status_path().read_text())
        except (OSError, ValueError):
            raw = {}
        fp = fingerprint()
        _S.disk = {k: v for k, v in raw.items() if isinstance(v, dict) and v.get("fingerprint") == fp}
    return _S.disk


def _persist(query: OpQuery, backend: str, err: BaseException) -> None:
    records = _disk_records()
    records[_disk_key(query, backend)] = {"error": describe(err), "time": time.time(), "fingerprint": fingerprint()}
    path = _status_path()
    try:
        path.parent.mkdir(parents=True, exist_ok=True)
        tmp = path.with_suffix(f".{os.getpid()}.tmp")
        tmp.write_text(json.dumps(records, indent=1, sort_keys=True))
        os.replace(tmp, path)
    except OSError:
        pass  # a cache that cannot be written is no reason to fail the call


@contextmanager
def build_phase():
    """Inside, a recorded failure of the build / toolchain class is also written to disk."""
    with _S.lock:
        _S.build_depth += 1
    try:
        yield
    finally:
        with _S.lock:
            _S.build_depth -= 1


def forget_disk_failures() -> None:
    """Drop the on-disk records (and the copy read from them)."""
    with _S.lock:
        _S.disk = None
        try:
            _status_path().unlink()
        except OSError:
            pass


# ---- backward under guard -----------------------------------------------------------------------


def _records_grad(args) -> bool:
    """A call that records a plain autograd graph: grad on, not traced, no saved-tensor hooks
    (checkpointing and activation offload keep their own graph semantics), a tensor needing grad."""
    return (
        torch.is_grad_enabled()
        and not torch.compiler.is_compiling()
        and not _saved_tensor_hooks_active()
        and any(isinstance(a, torch.Tensor) and a.requires_grad for a in args)
    )


def _saved_tensor_hooks_active() -> bool:
    probe = getattr(torch._C._autograd, "_top_saved_tensors_default_hooks", None)
    if probe is None:
        return True  # cannot tell: leave such a call unguarded rather than change what its hooks see
    return probe(False) is not None


def _as_leaves(args) -> list:
    return [a.detach().requires_grad_(a.requires_grad) if isinstance(a, torch.Tensor) else a for a in args]


def _backprop(outs, leaves, grads) -> tuple:
    need = [i for i, a in enumerate(leaves) if isinstance(a, torch.Tensor) and a.requires_grad]
    pairs = [(o, g) for o, g in zip(outs, grads) if g is not None and o.requires_grad]
    got = torch.autograd.grad([o for o, _ in pairs], [leaves[i] for i in need], [g for _, g in pairs], allow_unused=True)
    result: list = [None] * len(leaves)
    for i, g in zip(need, got):
        result[i] = g
    return tuple(result)


class _Guarded(torch.autograd.Function):
    """The op on detached copies of its arguments, its backward through `autograd.grad` over that
    inner graph. A backend failure there moves the op on (`fall_back`) and runs forward and backward
    again through the next backend from the saved arguments (autograd refuses them if they were
    written to in between). Afterwards the inner graph, its outputs and the arguments are let go."""

    @staticmethod
    def forward(ctx, bound, kwargs, *args):
        leaves = _as_leaves(args)
        with torch.enable_grad():
            out = bound._run(leaves, kwargs)
        ctx.save_for_backward(*(a for a in args if isinstance(a, torch.Tensor)))
        ctx.others = [None if isinstance(a, torch.Tensor) else (a,) for a in args]
        ctx.bound, ctx.kwargs, ctx.leaves = bound, kwargs, leaves
        ctx.outs = out if isinstance(out, tuple) else (out,)
        return tuple(o.detach() for o in out) if isinstance(out, tuple) else out.detach()

    @staticmethod
    def backward(ctx, *grads):
        bound = ctx.bound
        try:
            try:
                got = _backprop(ctx.outs, ctx.leaves, grads)
                with _S.lock:  # backward runs on autograd's threads
                    _S.proven.add(bound)
            except LAUNCH_ERRORS as err:
                saved = iter(ctx.saved_tensors)
                args = [next(saved) if slot is None else slot[0] for slot in ctx.others]
                bound.fall_back(err, args, ctx.kwargs)  # raises when there is nowhere to go
                leaves = _as_leaves(args)
                with torch.enable_grad():
                    out = bound._run(leaves, ctx.kwargs)
                got = _backprop(out if isinstance(out, tuple) else (out,), leaves, grads)
        finally:
            ctx.bound = ctx.kwargs = ctx.leaves = ctx.outs = ctx.others = None
        return (None, None, *got)


def settle_guards() -> int:
    """Lift the guard from every op whose guarded backward went through (call it at a step boundary,
    so that a step runs one call path per op); returns how many."""
    with _S.lock:
        ops = list(_S.proven)
        _S.proven.clear()
    for op in ops:
        op.guard = False
    return len(ops)


def exercise(op: "Bound", run: Callable[["Bound"], object]) -> object:
    """`run(op)`, a forward and backward on scratch inputs, as build time: a backend failure anywhere
    in it, the backward included, moves `op` on and runs it again; toolchain failures met here are
    kept on disk; a backward that went through lifts the guard at once (no step is running)."""
    with build_phase():
        while True:
            try:
                out = run(op)
            except LAUNCH_ERRORS as err:
                op.fall_back(err)
                continue
            with _S.lock:
                if op in _S.proven:
                    _S.proven.discard(op)
                    op.guard = False
            return out


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
        # a backward can only be answered by moving on while there is somewhere to go
        self.guard = not self.pinned and backend in self.order and backend != self.order[-1]

    def _run(self, args, kwargs):
        while True:
            try:
                return self._fn(*args, **kwargs)
            except LAUNCH_ERRORS as err:
                self.fall_back(err, args, kwargs)  # raises when there is nowhere to go

    def __call__(self, *args, **kwargs):
        if self.guard and _records_grad(args):
            return _Guarded.apply(self, kwargs, *args)
        return self._run(args, kwargs)

    def __getattr__(self, name: str):
        if name.startswith("_"):
            raise AttributeError(name)
        return getattr(self._fn, name)

    def __repr__(self) -> str:
        return f"<{self.query.describe()} on {self.backend} of {self.order}>"

    def fall_back(self, err: BaseException, args=None, kwargs=None) -> None:
        """Leave the current backend after `err`. Returns with the op (and its siblings) bound to
        the next usable backend, or raises: `err` itself when it must not be answered by moving on,
        `InputError` when the arguments are at fault, `err` again when no backend is left in the chain."""
        if self.pinned or not is_build_error(err) or is_sticky_error(err, self.device):
            raise err
        if not isinstance(err, BackendUnavailable) and args is not None:
            self._blame_arguments(err, args, kwargs or {})
        with _S.lock:
            _S.failed[_failure_key(self.query, self.backend)] = describe(err)
            if _S.build_depth > 0 and is_toolchain_error(err):
                _persist(self.query, self.backend, err)
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
