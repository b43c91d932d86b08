"""Dispatch and tuning table on the host (no GPU): fake backends registered into the
registry under a patched priority (the way reference `tests/kernels/registry/test_fallback.py`
does), the arch table, and the five cases of `tuning.select`."""

import json

import pytest
import torch

from kohakumosstrainer_amd.kernels import registry, tuning
from kohakumosstrainer_amd.kernels.arch import CPU, GFX950, arch_of, forced_arch
from kohakumosstrainer_amd.kernels.constraints import requires
from kohakumosstrainer_amd.kernels.errors import BackendUnavailable, ConfigsFailed, InputError


@pytest.fixture
def fake_ops():
    registry.load_backends()
    calls = []

    def good(x):
        calls.append("good")
        return x + 1

    def broken(x):
        calls.append("broken")
        raise BackendUnavailable("fake_op", {"broken": "cannot build"})

    def eager(x):
        calls.append("eager")
        return x + 1

    registry.register("fake_op", "hip", broken, supports=lambda q: None)
    registry.register("fake_op", "second", good)
    registry.register("fake_op", "eager", eager)
    registry.set_priority("cpu", ("hip", "second", "eager"))
    yield calls
    registry.reset_priority()
    registry.clear_failures()
    registry.unregister("fake_op")


def test_arch_table():
    assert arch_of("cpu") is CPU and not CPU.has_fp8
    assert GFX950.name == "gfx950" and GFX950.kind == "hip" and GFX950.has_fp8 and GFX950.has_mx and GFX950.has_bf16
    with forced_arch(GFX950):
        assert arch_of("cpu") is GFX950
    assert registry.DEFAULT_PRIORITY["gfx950"] == ("hip",), "a GPU op must never drop to torch silently"


def test_fallback_walks_priority_and_rebinds_siblings(fake_ops):
    a = registry.resolve("fake_op", "cpu", torch.float32)
    b = registry.resolve("fake_op", "cpu", torch.float32)
    assert a.backend == b.backend == "hip"
    assert a(torch.zeros(1)).item() == 1
    assert a.backend == "second" and b.backend == "second", "the sibling moves with it"
    assert fake_ops == ["broken", "good"]
    assert any(k[0] == "fake_op" and k[1] == "hip" for k in registry.failures())
    c = registry.resolve("fake_op", "cpu", torch.float32)
    assert c.backend == "second", "a backend that failed here is skipped at the next resolve"


class _FailsInBackward(torch.autograd.Function):
    """A backend whose forward is fine and whose backward cannot launch."""

    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return x @ w.t()

    @staticmethod
    def backward(ctx, g):
        raise BackendUnavailable("fake_linear", {"dgrad": "kernel does not build"})


@pytest.fixture
def backward_failure():
    registry.load_backends()
    calls = []

    def hip(x, w):
        calls.append("hip")
        return _FailsInBackward.apply(x, w)

    def eager(x, w):
        calls.append("eager")
        return x @ w.t()

    registry.register("fake_linear", "hip", hip)
    registry.register("fake_linear", "eager", eager)
    registry.set_priority("cpu", ("hip", "eager"))
    yield calls
    registry.reset_priority()
    registry.clear_failures()
    registry.forget_disk_failures()
    registry.unregister("fake_linear")


def test_failure_inside_backward_moves_on_and_recomputes(backward_failure):
    """Reference `registry.py:280-314`: the backend fails only in backward; the op and its sibling
    move to the next backend and the gradients come from a second forward + backward there."""
    op = registry.resolve("fake_linear", "cpu", torch.float32)
    sibling = registry.resolve("fake_linear", "cpu", torch.float32)
    assert op.backend == "hip" and op.guard, "an op with somewhere to go runs its backward under guard"
    x = torch.randn(5, 8, requires_grad=True)
    w = torch.randn(3, 8, requires_grad=True)
    y = op(x, w)
    assert op.backend == "hip" and backward_failure == ["hip"]
    g = torch.randn(5, 3)
    y.backward(g)
    assert op.backend == "eager" and sibling.backend == "eager", "the sibling moves with it"
    assert backward_failure == ["hip", "eager"], "forward ran again through the next backend"
    assert torch.allclose(x.grad, g @ w.detach()) and torch.allclose(w.grad, g.t() @ x.detach())
    assert torch.equal(y.detach(), x.detach() @ w.detach().t())
    assert not op.guard, "the last backend of the chain has nothing to give way to"
    assert any(k[0] == "fake_linear" and k[1] == "hip" for k in registry.failures())
    # without grad nothing is guarded, and the next call goes straight to the backend that works
    with torch.no_grad():
        op(x, w)
    assert backward_failure == ["hip", "eager", "eager"]


def test_guard_refuses_inputs_written_between_forward_and_backward(backward_failure):
    op = registry.resolve("fake_linear", "cpu", torch.float32)
    x = torch.randn(5, 8, requires_grad=True)
    w = torch.randn(3, 8)
    y = op(x, w)
    w.add_(1.0)  # the recompute would see another weight: autograd's version check must refuse
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        y.backward(torch.ones(5, 3))


def test_settle_guards_and_exercise(backward_failure):
    registry.unregister("fake_linear", "hip")
    registry.register("fake_linear", "hip", lambda x, w: x @ w.t())  # a backend that works
    op = registry.resolve("fake_linear", "cpu", torch.float32)
    x = torch.randn(2, 8, requires_grad=True)
    w = torch.randn(3, 8)
    assert op.guard
    op(x, w).sum().backward()
    assert op.guard, "proven, but the guard is lifted only at a step boundary"
    assert registry.settle_guards() == 1 and not op.guard and op.backend == "hip"
    op(x, w).sum().backward()  # the plain path
    other = registry.resolve("fake_linear", "cpu", torch.float16)
    ran = registry.exercise(other, lambda o: o(x.detach().half().requires_grad_(True), w.half()).sum().backward())
    assert ran is None and not other.guard, "a prewarm that went through lifts the guard at once"


def test_toolchain_failures_at_build_time_outlive_the_process(backward_failure):
    """Reference `status.py:111-133`: only a build / toolchain failure met at build time is written
    to disk; a later process (here: the in-memory state dropped) does not try that backend again."""
    op = registry.resolve("fake_linear", "cpu", torch.float32)
    x = torch.randn(2, 8, requires_grad=True)
    w = torch.randn(3, 8)
    registry.exercise(op, lambda o: o(x, w).sum().backward())
    assert op.backend == "eager"
    registry.clear_failures()
    registry._S.disk = None  # what a new process starts with: nothing in memory, the file on disk
    why = registry.available("fake_linear", "cpu", torch.float32)
    assert why["hip"] is not None and "earlier process" in why["hip"], why
    assert registry.resolve("fake_linear", "cpu", torch.float32).backend == "eager"
    assert registry.resolve("fake_linear", "cpu", torch.float16).backend == "hip", "another query is not covered by the record"
    # a failure in a live call (outside build time) stays in the process
    registry.forget_disk_failures()
    live = registry.resolve("fake_linear", "cpu", torch.bfloat16)
    xb = x.detach().bfloat16().requires_grad_(True)
    live(xb, w.bfloat16()).sum().backward()
    assert live.backend == "eager"
    registry.clear_failures()
    registry._S.disk = None
    assert registry.available("fake_linear", "cpu", torch.bfloat16)["hip"] is None


def test_pinned_backend_has_no_fallback(fake_ops):
    op = registry.resolve("fake_op", "cpu", torch.float32, backend="hip")
    with pytest.raises(BackendUnavailable):
        op(torch.zeros(1))


def test_bad_inputs_are_the_callers_bug(fake_ops):
    def picky(x):
        raise OSError("launch failed")

    def eager_rejects(x):
        raise ValueError("bad shape")

    registry.register("fake_op", "hip", picky)
    registry.register("fake_op", "eager", eager_rejects)
    op = registry.resolve("fake_op", "cpu", torch.float32)
    with pytest.raises(InputError):
        op(torch.zeros(1))
    assert op.backend == "hip" and not registry.failures(), "nothing recorded, the op stays bound"


def test_sticky_device_fault_is_reraised(fake_ops):
    def faulting(x):
        raise OSError("HSA_STATUS_ERROR: memory access fault by GPU")

    registry.register("fake_op", "hip", faulting)
    op = registry.resolve("fake_op", "cpu", torch.float32)
    with pytest.raises(OSError):
        op(torch.zeros(1))


def test_supports_and_available_reasons():
    registry.load_backends()
    why = registry.available("fp8_linear", "cpu", torch.bfloat16, recipe="mx")
    assert why["eager"] is None and "cpu" in why["hip"]
    with forced_arch(GFX950):
        assert registry.available("fp8_linear", "cpu", torch.bfloat16, recipe="mx")["hip"] is None
        assert registry.available("fp8_linear", "cpu", torch.bfloat16, recipe="row")["hip"] is None
        assert registry.available("fp8_linear", "cpu", torch.bfloat16, recipe="block")["hip"] is None
        assert "not built" in registry.available("fp8_linear", "cpu", torch.bfloat16, recipe="nvfp4")["hip"]
        assert registry.available("fp8_linear", "cpu", torch.float32, recipe="mx")["hip"] is not None
        assert registry.available("quant_linear", "cpu", torch.float16, fmt="fp8")["hip"] is None
        assert "unknown" in registry.available("quant_linear", "cpu", torch.float16, fmt="int4")["hip"]
        with pytest.raises(registry.NoImplementationError):
            registry.resolve("fp8_linear", "cpu", torch.bfloat16, recipe="nvfp4")
    gate = requires(kinds=("hip",), archs=("gfx950",))
    assert gate(registry.OpQuery("x", CPU, torch.bfloat16)) is not None
    assert gate(registry.OpQuery("x", GFX950, torch.bfloat16)) is None


def test_gpu_op_without_a_gpu_fails_loudly():
    """On gfx950 the only backend is hip: handing it host tensors raises, it does not compute
    on the CPU."""
    registry.load_backends()
    with forced_arch(GFX950):
        op = registry.resolve("quant_linear", "cpu", torch.bfloat16, fmt="int8")
    assert op.backend == "hip" and op.order == ("hip",)
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="device tensors"):
        op(x, torch.zeros(8, 64, dtype=torch.int8), torch.ones(8), None, "int8")


# ---- tuning table ------------------------------------------------------------------------


@pytest.fixture
def fresh_tuner(tmp_path, monkeypatch):
    monkeypatch.setenv("KOHAKUMOSS_KERNEL_CACHE", str(tmp_path))
    tuning.reset()
    tuning._tables.clear()
    tuning.reopen()
    tuning.set_mode("table")
    yield tmp_path
    tuning.set_mode("table")
    tuning.reopen()
    tuning.reset()
    tuning._tables.clear()


CANDS = [{"bm": 256, "id": 0}, {"bm": 128, "id": 1}, {"bm": 64, "id": 2}]


def timed_launch(cost):
    import time

    def launch(cfg):
        def run():
            time.sleep(cost[cfg["id"]])

        return run

    return launch


def test_select_times_shortlist_stores_and_settles(fresh_tuner):
    launch = timed_launch({0: 0.004, 1: 0.0005, 2: 0.002})
    cfg = tuning.select("k", "cpu", "m64", lambda: CANDS, launch, shortlist=3)
    assert cfg == CANDS[1] and tuning.decided("k", "cpu", "m64")
    files = list(fresh_tuner.rglob("k.json"))
    assert len(files) == 1 and files[0].parent.parent.parent.name == "tuning"
    row = json.loads(files[0].read_text())["m64"]
    assert row["config"] == CANDS[1] and len(row["timings_ms"]) == 3 and row["failures"] == {}
    # a new process (fresh state) binds the stored winner without timing
    tuning.reset()
    tuning._tables.clear()
    def boom(cfg):
        raise AssertionError("must not launch")
    assert tuning.select("k", "cpu", "m64", lambda: CANDS, boom) == CANDS[1]
    # a stored winner that is no longer a candidate is ignored
    tuning.reset()
    assert tuning.select("k", "cpu", "m64", lambda: CANDS[:1], boom) == CANDS[0]


def test_select_mode_off_binds_first_candidate_untimed(fresh_tuner):
    tuning.set_mode("off")
    def boom(cfg):
        raise AssertionError("must not launch")
    assert tuning.select("k", "cpu", "a", lambda: CANDS, boom) == CANDS[0]
    assert tuning.decided("k", "cpu", "a") and not list(fresh_tuner.rglob("*.json"))


def test_untimed_pick_is_not_settled_then_timed_later(fresh_tuner, monkeypatch):
    launch = timed_launch({0: 0.002, 1: 0.0003, 2: 0.002})
    with monkeypatch.context() as patch:
        patch.setattr(tuning, "timing_allowed", lambda *a, **k: False)
        assert tuning.select("k", "cpu", "b", lambda: CANDS, launch) == CANDS[0]
        assert not tuning.decided("k", "cpu", "b"), "a provisional pick must not be bound"
    assert tuning.select("k", "cpu", "b", lambda: CANDS, launch, shortlist=3) == CANDS[1]
    assert tuning.decided("k", "cpu", "b")


def test_frozen_window_binds_first_config_that_runs(fresh_tuner):
    tuning.freeze()
    def launch(cfg):
        def run():
            if cfg["id"] == 0:
                raise RuntimeError("out of resources")
        return run
    assert tuning.select("k", "cpu", "c", lambda: CANDS, launch) == CANDS[1]
    assert ("cpu", "k", "c") in tuning.DEFERRED and not list(fresh_tuner.rglob("*.json"))
    with tuning.tuning_window():
        assert tuning.select("k", "cpu", "d", lambda: CANDS, timed_launch({0: 0.001, 1: 0.001, 2: 0.0001}), shortlist=3) == CANDS[2]


def test_failures_are_recorded_and_all_failed_raises(fresh_tuner):
    def launch(cfg):
        def run():
            if cfg["id"] != 2:
                raise RuntimeError(f"config {cfg['id']} cannot launch")
        return run
    assert tuning.select("k", "cpu", "e", lambda: CANDS, launch, shortlist=3) == CANDS[2]
    row = json.loads(next(fresh_tuner.rglob("k.json")).read_text())["e"]
    assert len(row["failures"]) == 2 and len(row["timings_ms"]) == 1
    def all_fail(cfg):
        def run():
            raise RuntimeError("no")
        return run
    with pytest.raises(ConfigsFailed):
        tuning.select("k", "cpu", "f", lambda: CANDS, all_fail)
    with pytest.raises(ConfigsFailed):
        tuning.select("k", "cpu", "f", lambda: CANDS, all_fail)


def test_forget_and_reset_hooks(fresh_tuner):
    tuning.set_mode("off")
    cleared = []
    tuning.on_reset(lambda: cleared.append(True))
    tuning.select("k", "cpu", "g", lambda: CANDS, None)
    tuning.forget("k", "cpu", "g")
    assert not tuning.decided("k", "cpu", "g")
    tuning.reset()
    assert cleared
    tuning._resets.pop()


def test_buckets_and_planner_ranking():
    assert [tuning.pow2(n, 16) for n in (1, 16, 17, 300, 16384)] == [16, 16, 32, 512, 16384]
    registry.load_backends()
    from kohakumosstrainer_amd.kernels.backends.hip import fp8_linear, quant

    big = fp8_linear.candidates("mx", 16384)
    assert (big[0]["bm"], big[0]["bn"]) == (256, 256) and all(c["gemm"] == "hip" for c in big)
    small = fp8_linear.candidates("mx", 40)
    assert small[0]["bm"] == 64 and all(c["bm"] <= 64 for c in small)
    assert quant.candidates(4096)[0]["bm"] == 256 and quant.candidates(1)[0]["bm"] == 64
    assert fp8_linear._table_key("fwd", 300, 9216, 3072, torch.empty(0, dtype=torch.bfloat16), "mx", None) == "fwd_m512_n9216_k3072_torch.bfloat16_mx_x"
