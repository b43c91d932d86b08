"""Error vocabulary of the kernel layer.

A backend that cannot build or launch on this machine raises one of `BUILD_ERRORS`; a launcher
that has run out of configurations raises `BackendUnavailable` (`ConfigsFailed` when a tuned
kernel tried them all). The registry answers those by moving to the next backend. Two kinds of
failure are never a reason to move on: an out-of-memory condition (the next backend would only
hit it later) and a device fault that leaves the context unusable. A call the eager path rejects
too is the caller's mistake and surfaces as `InputError`.
Convention of reference `src/kohakumoss_kernels/errors.py:12-136`.
"""

from __future__ import annotations

import re

import torch

from kohakumosstrainer_amd.native import KernelError, KernelLibraryMissing

# what "cannot build or launch here" looks like (the C ABI's error codes arrive as KernelError)
BUILD_ERRORS: tuple[type[BaseException], ...] = (RuntimeError, OSError, UnicodeError, KernelError, KernelLibraryMissing)
LAUNCH_ERRORS = BUILD_ERRORS

_TEXT_LIMIT = 400
# a library that is not there or a compiler that failed: the same on every call of this process and the next
_TOOLCHAIN = re.compile(r"hipcc|compil|toolchain|not built|cannot load|codegen|out of resources", re.I)
# the device context is gone: every later call on it fails too
_STICKY = re.compile(
    r"memory access fault|illegal memory access|hsa_status_error|device-side assert|unspecified launch failure|"
    r"hardware exception|gpu hang|ecc error|device lost|hiperrorillegaladdress|launch timed out",
    re.I,
)


def describe(err: BaseException) -> str:
    """One line naming the error, short enough for a table row or a log line."""
    text = " ".join(str(err).split())
    if len(text) > _TEXT_LIMIT:
        text = text[: _TEXT_LIMIT - 3] + "..."
    return f"{type(err).__name__}: {text}" if text else type(err).__name__


def _join(errors: dict[str, str]) -> str:
    return "; ".join(f"{where}: {why}" for where, why in errors.items()) or "no attempt recorded"


class BackendUnavailable(RuntimeError):
    """`op` cannot run on this backend here. `errors` maps what was tried to why it failed;
    `persist` says whether a later process would fail the same way (a missing library does, a
    shape that does not fit does not); `problem` names the shape when the reason is one."""

    def __init__(self, op: str, errors: dict[str, str], what: str = "unavailable", persist: bool = True, problem: str | None = None):
        self.op, self.errors, self.persist, self.problem = op, dict(errors), persist, problem
        where = f" for {problem}" if problem else ""
        super().__init__(f"{op} {what}{where}: {_join(self.errors)}")


class ConfigsFailed(BackendUnavailable):
    """Every configuration of a tuned kernel failed to build or launch."""

    def __init__(self, kernel: str, errors: dict[str, str], persist: bool = True, problem: str | None = None):
        super().__init__(kernel, errors, what="has no configuration that runs", persist=persist, problem=problem)
        self.kernel = kernel


class InputError(ValueError):
    """The backend failed and the eager implementation rejected the same arguments: the call is
    wrong, no backend is to blame."""

    def __init__(self, op: str, backend: str, err: BaseException, eager: BaseException):
        self.op, self.backend, self.error, self.eager_error = op, backend, err, eager
        super().__init__(f"{op}: bad arguments ({describe(eager)}); the {backend} backend had failed with {describe(err)}")


def is_build_error(err: BaseException) -> bool:
    """Something a backend may answer by giving way. Running out of memory is not."""
    if isinstance(err, torch.OutOfMemoryError):
        return False
    return isinstance(err, BUILD_ERRORS)


def is_toolchain_error(err: BaseException) -> bool:
    """A build error that does not depend on the call: worth remembering across processes."""
    if isinstance(err, KernelLibraryMissing):
        return True
    if isinstance(err, BackendUnavailable):
        return err.persist
    return is_build_error(err) and _TOOLCHAIN.search(str(err)) is not None


def is_sticky_error(err: BaseException, device=None) -> bool:
    """A device fault after which the context cannot be trusted: by the words of the message, or,
    given a device, by whether it still synchronizes."""
    if isinstance(err, (BackendUnavailable, KernelLibraryMissing)):
        return False
    if _STICKY.search(str(err)):
        return True
    dev = torch.device(device) if device is not None else None
    if dev is not None and dev.type == "cuda" and torch.cuda.is_available():
        try:
            torch.cuda.synchronize(dev)
        except Exception:  # noqa: BLE001 - whatever it raises, the device is not well
            return True
    return False


def unavailable(op: str, err: BaseException, where: str = "") -> BackendUnavailable:
    """Wrap a build / launch error as `BackendUnavailable`, keeping the cause."""
    if isinstance(err, BackendUnavailable):
        return err
    out = BackendUnavailable(op, {where or "launch": describe(err)}, persist=is_toolchain_error(err))
    out.__cause__ = err
    return out
