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
rows `{key: {"config", "timings_ms", "failures"[, "working_mib"]}}`, merged on write and replaced
atomically. `working_mib` is the peak device memory each timed candidate took beyond what was
allocated before it ran; a candidate whose first run takes more than the caller's `working_bound`
is dropped from the shortlist like one that fails to launch (reference `tuner.py:363-442`).
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

    def put(self, key: str, config: dict, timings: dict, failures: dict, working_mib: dict | None = None) -> None:
        row = {"config": config, "timings_ms": timings, "failures": failures}
        if working_mib:
            row["working_mib"] = working_mib
        with self.lock:
            self.rows = {**(_read_json(self.path) or {}), **self.rows, key: row}
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


class _Problem:
    """One (device, kernel, key) and what `select` learns about it: shared bookkeeping of the
    ways a configuration gets picked."""

    def __init__(self, kernel: str, device: torch.device, key: str):
        self.kernel, self.device, self.key = kernel, device, key
        self.ident = (str(device), kernel, key)
        self.errors: dict[str, str] = {}

    def settle(self, config: dict) -> dict:
        _chosen[self.ident] = config
        DEFERRED.discard(self.ident)
        return config

    def give_up(self) -> ConfigsFailed:
        err = ConfigsFailed(self.kernel, dict(self.errors), persist=all(_TOOLCHAIN_HINT(v) for v in self.errors.values()), problem=self.key)
        _failed[self.ident] = err
        return err

    def try_once(self, config: dict, launch: Callable[[dict], Callable[[], object]]) -> Callable[[], object] | None:
        """Build and run `config` once; None (and the reason noted) when it cannot."""
        try:
            run = launch(config)
            run()
            if self.device.type == "cuda":
                torch.cuda.synchronize(self.device)
            return run
        except BUILD_ERRORS as err:
            if isinstance(err, torch.OutOfMemoryError):
                raise
            self.errors[config_name(config)] = describe(err)
            return None


def _TOOLCHAIN_HINT(text: str) -> bool:
    return is_toolchain_error(RuntimeError(text))


def _peak_mib(device: torch.device) -> float:
    return torch.cuda.max_memory_allocated(device) / 2**20 if device.type == "cuda" else 0.0


def select(
    kernel: str,
    device: torch.device | str,
    key: str,
    candidates: Callable[[], Sequence[dict]],
    launch: Callable[[dict], Callable[[], object]] | None,
    shortlist: int = 4,
    in_backward: bool = False,
    timing: Callable[[Callable[[], object], torch.device], float] | None = None,
    working_bound: float | None = None,
) -> dict:
    """The configuration of `kernel` for problem `key` on `device`.

    `candidates()` lists configurations, the planner's first pick first; `launch(config)` returns
    a zero-argument callable that runs the kernel once on the caller's operands. `working_bound`
    (MiB) drops candidates whose run allocates more than that. See the module docstring for the
    order of the five cases."""
    device = torch.device(device)
    problem = _Problem(kernel, device, key)
    if problem.ident in _chosen:
        return _chosen[problem.ident]
    if problem.ident in _failed:
        raise _failed[problem.ident]
    ranked = list(candidates())
    if not ranked:
        raise ConfigsFailed(kernel, {"candidates": "the planner offered none"}, persist=False, problem=key)

    stored = table(kernel, device).get(key) if get_mode() == "table" else None
    if stored is not None:
        wanted = _canon(stored)
        for config in ranked:
            if _canon(config) == wanted:
                return problem.settle(config)

    if len(ranked) == 1:
        return problem.settle(ranked[0])  # nothing to compare
    if not timing_allowed(in_backward):
        # nothing may be measured here: the planner's first pick serves, and only counts as the
        # answer when no measurement will ever be made (mode off)
        return problem.settle(ranked[0]) if get_mode() == "off" else ranked[0]

    if _state["frozen"] or _state["defer"]:
        DEFERRED.add(problem.ident)
        for config in ranked:
            if problem.try_once(config, launch) is not None:
                return config  # provisional: timed once a tuning window opens
        raise problem.give_up()

    measure = timing or (lambda run, dev: best_ms(run, dev))
    timings: dict[str, float] = {}
    working: dict[str, float] = {}
    by_name = {}
    for config in ranked[: max(1, shortlist)]:
        name = config_name(config)
        if device.type == "cuda":
            torch.cuda.synchronize(device)
            torch.cuda.reset_peak_memory_stats(device)
        before = torch.cuda.memory_allocated(device) / 2**20 if device.type == "cuda" else 0.0
        run = problem.try_once(config, launch)
        if run is None:
            continue
        took = max(0.0, _peak_mib(device) - before)
        if device.type == "cuda":
            working[name] = round(took, 3)
        if working_bound is not None and took > working_bound:
            problem.errors[name] = f"working memory {took:.1f} MiB exceeds the bound of {working_bound:.1f} MiB"
            continue
        try:
            timings[name] = measure(run, device)
        except BUILD_ERRORS as err:
            if isinstance(err, torch.OutOfMemoryError):
                raise
            problem.errors[name] = describe(err)
            continue
        by_name[name] = config
    if not timings:
        # the shortlist is exhausted: anything further down that runs at all still serves
        for config in ranked[max(1, shortlist) :]:
            if problem.try_once(config, launch) is not None:
                table(kernel, device).put(key, config, {}, dict(problem.errors))
                return problem.settle(config)
        raise problem.give_up()
    TIMED[kernel] = TIMED.get(kernel, 0) + 1
    winner = by_name[min(timings, key=timings.get)]
    table(kernel, device).put(key, winner, timings, dict(problem.errors), working)
    return problem.settle(winner)


def forget(kernel: str, device: torch.device | str, key: str) -> None:
    """Drop what this process settled for one problem (a stored row stays on disk)."""
    ident = (str(torch.device(device)), kernel, key)
    _chosen.pop(ident, None)
    _failed.pop(ident, None)
    DEFERRED.discard(ident)


def settled(kernel: str, device: torch.device | str, key: str) -> dict | None:
    return _chosen.get((str(torch.device(device)), kernel, key))


def decided(kernel: str, device: torch.device | str, key: str) -> bool:
    """True once the choice for `key` will not change in this process: callers cache a bound
    runner only then."""
    return (str(torch.device(device)), kernel, key) in _chosen
