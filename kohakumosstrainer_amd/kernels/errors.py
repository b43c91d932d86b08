"""Errors of the kernel layer and the classification the dispatch relies on.

Mirrors reference `src/kohakumoss_kernels/errors.py`: a backend that cannot build or launch
an op raises one of `BUILD_ERRORS`; the registry turns it into `BackendUnavailable` and moves
to the next backend of the arch's priority. Out-of-memory is never such an error, a sticky
device fault is re-raised, and arguments the eager reference rejects too are the caller's bug
(`InputError`).
"""

import torch

BUILD_ERRORS: tuple[type[BaseException], ...] = (RuntimeError, OSError, UnicodeError)
# what a *launch* may raise and still mean "this backend cannot run here": a bare
# RuntimeError from a call is only trusted when the backend wrapped it (BackendUnavailable)
LAUNCH_ERRORS: tuple[type[BaseException], ...] = (OSError, UnicodeError)

_TOOLCHAIN_WORDS = ("hipcc", "compiler", "compilation", "toolchain", "not built", "cannot load", "out of resources", "codegen")
_STICKY_WORDS = (
    "illegal memory access",
    "illegal address",
    "misaligned address",
    "illegal instruction",
    "device-side assert",
    "unspecified launch failure",
    "memory access fault",
    "hardware exception",
)


def describe(err: BaseException) -> str:
    return f"{type(err).__name__}: {err}"[:2000]


class BackendUnavailable(RuntimeError):
    """A backend cannot run `op` here. `errors` maps each attempt to its error text;
    `persist` says the cause is the build / toolchain (it holds for later processes), not one
    call's arguments; `problem` names the single tuned problem that failed, if any."""

    def __init__(self, op: str, errors: dict[str, str], what: str = "unavailable", persist: bool = True, problem: str | None = None):
        self.op, self.errors, self.persist, self.problem = op, dict(errors), persist, problem
        super().__init__(f"{op}: {what}: {self.errors}")


class ConfigsFailed(BackendUnavailable):
    """Every shortlisted config of a tuned kernel failed on one problem."""

    def __init__(self, kernel: str, errors: dict[str, str], persist: bool = True, problem: str | None = None):
        super().__init__(kernel, errors, "every shortlisted config failed", persist, problem)


class InputError(ValueError):
    """A backend failed on arguments the eager reference rejects as well: a caller bug, never
    a backend failure (no fallback, nothing recorded)."""

    def __init__(self, op: str, backend: str, err: BaseException, eager: BaseException):
        super().__init__(
            f"{op}: backend {backend} failed on arguments the eager reference also rejects: "
            f"{describe(err)[:1000]}; eager: {describe(eager)[:1000]}"
        )


def is_build_error(err: BaseException) -> bool:
    return isinstance(err, BUILD_ERRORS) and not isinstance(err, torch.OutOfMemoryError)


def is_toolchain_error(err: BaseException) -> bool:
    if isinstance(err, BackendUnavailable):
        return err.persist
    if isinstance(err, torch.OutOfMemoryError):
        return False
    if isinstance(err, (OSError, UnicodeError)):
        return True
    text = str(err).lower()
    return any(word in text for word in _TOOLCHAIN_WORDS)


def is_sticky_error(err: BaseException, device=None) -> bool:
    """The error left the device context unusable (its text names a fault, or synchronizing
    the device raises): falling back onto the same context would fail too."""
    text = str(err).lower()
    if any(word in text for word in _STICKY_WORDS):
        return True
    if device is None or torch.device(device).type != "cuda" or not torch.cuda.is_available():
        return False
    try:
        torch.cuda.synchronize(device)
    except RuntimeError:
        return True
    return False


def unavailable(op: str, err: BaseException, where: str = "") -> BackendUnavailable:
    """`err` as BackendUnavailable when it is a build / launch failure; anything else
    (out-of-memory, bugs) is re-raised unchanged."""
    if isinstance(err, BackendUnavailable):
        return err
    if not is_build_error(err):
        raise err
    return BackendUnavailable(op, {where or op: describe(err)}, persist=is_toolchain_error(err))
