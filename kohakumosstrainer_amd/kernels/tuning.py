"""Shape tuning table: pick one config per (kernel, problem key) - a stored winner if it is
still a candidate, else the fastest of a timed shortlist - and keep the winners per card on
disk.

Mirrors the semantics of reference `src/kohakumoss_kernels/tuning/tuner.py` (`select` :217-288,
`decided` :534-537, `forget` :521-524, `table` :201-205, `TuneTable` :104-151), `buckets.pow2`
(:18-23), the freeze / defer windows (`tuning/window.py:12-72`) and the event timing
(`tuning/timing.py:37-58`):

  1. a choice settled in this process wins;
  2. else a stored row whose config is still among the candidates;
  3. else, where timing is not allowed (mode "off", a torch.compile trace or graph capture,
     inside an autograd backward unless `in_backward`), the first candidate - settled only
     under mode "off" or when it is the only candidate;
  4. else, when frozen or deferring, the first candidate that runs once (unstored);
  5. else every config of the shortlist is timed (>= 25 ms busy warm-up, best of 10 event-timed
     calls), the winner is stored with every timing and failure, and settled.

Table file: `<KOHAKUMOSS_KERNEL_CACHE or ~/.cache/kohakumoss_kernels>/tuning/<card key>/<tag>/<kernel>.json`,
rows `{key: {"config", "timings_ms", "failures"}}`, merged on write and replaced atomically.
"""

import hashlib
import json
import os
import tempfile
import threading
import time
from collections.abc import Callable, Sequence
from contextlib import contextmanager
from pathlib import Path

import torch

from kohakumosstrainer_amd.kernels.errors import BUILD_ERRORS, ConfigsFailed, describe, is_toolchain_error

MODES = ("table", "off")
WARMUP_MS = 25.0
_state = {"mode": "table", "frozen": False, "defer": False}
_chosen: dict[tuple[str, str, str], dict] = {}
_failed: dict[tuple[str, str, str], ConfigsFailed] = {}
_tables: dict[tuple[str, str], "TuneTable"] = {}
_resets: list[Callable[[], None]] = []
DEFERRED: set[tuple[str, str, str]] = set()
TIMED: dict[str, int] = {}


def pow2(n: int, floor: int) -> int:
    """Smallest power of two >= max(n, floor) (`floor` a power of two)."""
    b = floor
    while b < n:
        b *= 2
    return b


def cdiv(a: int, b: int) -> int:
    return -(-a // b)


def set_mode(mode: str) -> None:
    if mode not in MODES:
        raise ValueError(f"TUNE={mode!r} not in {MODES}")
    _state["mode"] = mode


def get_mode() -> str:
    return _state["mode"]


def freeze() -> None:
    """From here `select` times nothing outside `tuning_window()`."""
    _state["frozen"] = True


def defer(on: bool) -> None:
    _state["defer"] = bool(on)


def reopen() -> None:
    _state.update(frozen=False, defer=False)


@contextmanager
def tuning_window():
    was = _state["frozen"]
    _state["frozen"] = False
    try:
        yield
    finally:
        _state["frozen"] = was


def on_reset(fn: Callable[[], None]) -> None:
    """Register a clear of a binding cache built from tuned choices (run by `reset`)."""
    _resets.append(fn)


def reset() -> None:
    """Forget every settled choice and every binding built from one."""
    _chosen.clear()
    _failed.clear()
    DEFERRED.clear()
    for fn in _resets:
        fn()


# ---- tables on disk ---------------------------------------------------------------------


def cache_dir() -> Path:
    root = os.environ.get("KOHAKUMOSS_KERNEL_CACHE")
    return Path(root) if root else Path.home() / ".cache" / "kohakumoss_kernels"


def _table_tag() -> str:
    from kohakumosstrainer_amd import native

    try:
        abi = str(native.load().km_abi_version())
    except RuntimeError:
        abi = "-"
    return hashlib.sha1(f"kohakumosstrainer_amd|abi={abi}".encode()).hexdigest()[:10]


def card_key(device: torch.device | str) -> str:
    """Cache key of a card: name, arch, HIP and torch versions."""
    device = torch.device(device)
    if device.type != "cuda":
        return f"cpu-torch{torch.__version__.split('+')[0]}"
    props = torch.cuda.get_device_properties(device)
    name = props.name.replace(" ", "_").replace("/", "_")
    arch = str(getattr(props, "gcnArchName", "")).split(":")[0] or f"sm{props.major}{props.minor}"
    return f"{name}-{arch}-hip{torch.version.hip or 'none'}-torch{torch.__version__.split('+')[0]}"


def _read_json(path: Path) -> dict | None:
    try:
        with open(path, encoding="utf-8") as fh:
            return json.load(fh)
    except (OSError, ValueError):
        return None


def _write_json_atomic(path: Path, data: dict) -> bool:
    try:
        path.parent.mkdir(parents=True, exist_ok=True)
        fd, tmp = tempfile.mkstemp(dir=path.parent, suffix=".tmp")
        with os.fdopen(fd, "w", encoding="utf-8") as fh:
            json.dump(data, fh, indent=1, sort_keys=True)
        os.replace(tmp, path)
        return True
    except OSError:
        return False


class TuneTable:
    """Winning configs of one kernel on one card, keyed by problem. A write merges the rows on
    disk first; threads sharing the table write one at a time; a failed write keeps the rows in
    memory."""

    def __init__(self, path: Path):
        self.path = path
        self.rows: dict[str, dict] = _read_json(path) or {}
        self.lock = threading.Lock()

    def get(self, key: str) -> dict | None:
        row = self.rows.get(key)
        return None if row is None else row["config"]

    def put(self, key: str, config: dict, timings: dict, failures: dict) -> None:
        with self.lock:
            self.rows = {**(_read_json(self.path) or {}), **self.rows, key: {"config": config, "timings_ms": timings, "failures": failures}}
            _write_json_atomic(self.path, self.rows)


def table(kernel: str, device: torch.device | str) -> TuneTable:
    """The process-shared table of `kernel` on `device`'s card."""
    card = card_key(device)
    tab = _tables.get((card, kernel))
    if tab is None or tab.path.parent.parent.parent.parent != cache_dir():
        tab = TuneTable(cache_dir() / "tuning" / card / _table_tag() / f"{kernel}.json")
        _tables[(card, kernel)] = tab
    return tab


# ---- timing -----------------------------------------------------------------------------


def _elapsed_ms(fn: Callable[[], object], calls: int, device: torch.device) -> float:
    if device.type != "cuda":
        t = time.perf_counter()
        for _ in range(calls):
            fn()
        return (time.perf_counter() - t) * 1e3
    with torch.cuda.device(device):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(calls):
            fn()
        end.record()
        end.synchronize()
        return start.elapsed_time(end)


def best_ms(fn: Callable[[], object], device: torch.device | str, iters: int = 10, warmup_ms: float = WARMUP_MS) -> float:
    """Best-of-`iters` device time of `fn` in ms after a busy warm-up of `warmup_ms`."""
    device = torch.device(device)
    calls, spent = 2, 0.0
    while spent < warmup_ms:
        spent += _elapsed_ms(fn, calls, device)
        calls *= 2
    return min(_elapsed_ms(fn, 1, device) for _ in range(iters))


def _tracing() -> bool:
    if torch.compiler.is_compiling():
        return True
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def timing_allowed(in_backward: bool = False) -> bool:
    """Whether the calling context permits timing a shortlist."""
    if get_mode() == "off" or _tracing():
        return False
    return in_backward or torch._C._current_graph_task_id() == -1


# ---- selection ---------------------------------------------------------------------------


def config_name(config: dict) -> str:
    return ",".join(f"{k}={v}" for k, v in sorted(config.items()))


def _canon(config: dict) -> str:
    return json.dumps(config, sort_keys=True, default=str)


def select(
    kernel: str,
    device: torch.device | str,
    key: str,
    candidates: Callable[[], Sequence[dict]],
    launch: Callable[[dict], Callable[[], object]],
    shortlist: int = 4,
    errors: tuple[type[BaseException], ...] = BUILD_ERRORS,
    in_backward: bool = False,
) -> dict:
    """The config for problem `key` of `kernel` on `device` (see the module docstring)."""
    ident = (str(device), kernel, key)
    chosen = _chosen.get(ident)
    if chosen is not None:
        return chosen
    failed = _failed.get(ident)
    if failed is not None:
        raise ConfigsFailed(kernel, failed.errors, failed.persist, failed.problem)
    ranked = list(candidates())
    tab = table(kernel, device)
    row = tab.get(key)
    if row is not None:
        match = [c for c in ranked if _canon(c) == _canon(row)]
        if match:
            _chosen[ident] = match[0]
            return match[0]
    if not timing_allowed(in_backward) or len(ranked) == 1:
        if get_mode() == "off" or len(ranked) == 1:
            _chosen[ident] = ranked[0]
        return ranked[0]
    if _state["frozen"] or _state["defer"]:
        return _bind_untimed(ident, ranked, launch, errors)
    TIMED[kernel] = TIMED.get(kernel, 0) + 1
    timings, failures, toolchain, best = {}, {}, [], None
    for config in ranked[:shortlist]:
        try:
            with torch.enable_grad():
                ms = best_ms(launch(config), device)
        except torch.OutOfMemoryError:
            raise
        except errors as err:
            failures[config_name(config)] = describe(err)[:300]
            toolchain.append(is_toolchain_error(err))
            continue
        timings[config_name(config)] = ms
        if best is None or ms < timings[config_name(best)]:
            best = config
    if best is None:
        err = ConfigsFailed(kernel, failures, all(toolchain), f"{kernel}:{key}")
        _failed[ident] = err
        raise err
    tab.put(key, best, timings, failures)
    _chosen[ident] = best
    return best


def _bind_untimed(ident, ranked, launch, errors) -> dict:
    failures, toolchain = {}, []
    for config in ranked:
        try:
            with torch.enable_grad():
                launch(config)()
        except errors as err:
            failures[config_name(config)] = describe(err)[:300]
            toolchain.append(is_toolchain_error(err))
            continue
        _chosen[ident] = config
        DEFERRED.add(ident)
        return config
    err = ConfigsFailed(ident[1], failures, all(toolchain), f"{ident[1]}:{ident[2]}")
    _failed[ident] = err
    raise err


def forget(kernel: str, device: torch.device | str, key: str) -> None:
    """Drop this process's choice for the problem (its config turned out unable to run)."""
    _chosen.pop((str(device), kernel, key), None)


def settled(kernel: str, device: torch.device | str, key: str) -> dict | None:
    chosen = _chosen.get((str(device), kernel, key))
    return chosen if chosen is not None else table(kernel, device).get(key)


def decided(kernel: str, device: torch.device | str, key: str) -> bool:
    """Whether `select` has a settled choice for this problem (callers bind only then)."""
    return (str(device), kernel, key) in _chosen
