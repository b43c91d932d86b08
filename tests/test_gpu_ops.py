"""The registered ops on the GPU: forward / input gradient / bias gradient of the HIP backend
against the fp64 product of the same dequantized operands (oracle), the gradient-free op equal
to the autograd op, one fullgraph torch.compile trace, the weight-only op, the module API end
to end, and one LoRA training step at the M=2048 K=4096 N=12288 r=8 shape.

Tolerances: forward and dgrad within rel-L2 2e-3 of the exact product in bf16 (1e-3 in fp16),
and no error statistic worse than 10x the eager launcher's on the same inputs
(reference `tests/kernels/fp8/test_fp8_linear.py:47-66`, `tests/kernels/_compare.py`)."""

import pytest
import torch
from torch import nn

from kohakumosstrainer_amd.kernels import registry, tuning
from kohakumosstrainer_amd.kernels.fp8 import formats
from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant import ComputeWeight, QuantWeight, attach_compute, default_filter, quantize_model
from kohakumosstrainer_amd.quant.compute import quantize_pair
from oracle import formats as oracle_formats
from oracle import linear as oracle_linear
from oracle import stats as oracle_stats

pytestmark = pytest.mark.gpu
DEV = "cuda"
REL_L2 = {torch.bfloat16: 2e-3, torch.float16: 1e-3}


@pytest.fixture(autouse=True)
def untimed():
    """Bind the planner's first candidate: the ops under test are the same, the shortlist
    timing is covered by its own test."""
    tuning.set_mode("off")
    tuning.reset()
    yield
    tuning.set_mode("table")
    tuning.reset()


def problem(m, n, k, dtype, recipe, dgrad=True, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = (torch.randn(n, k, generator=g) * 0.05).to(dtype)
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    base = ComputeWeight.from_weight(w, recipe, dgrad)
    return x, w, bias, dy, base


def parts(base, device):
    return [None if t is None else t.to(device) for t in (base.q, base.scale, base.aux, base.q_t, base.scale_t, base.aux_t)]


def exact_product(a, q, scale, bias, recipe):
    """fp64 product of the exactly dequantized operands: the activation `a` quantized per call
    (as the op does), the stored codes `q` [rows_out, K] with `scale`."""
    aq, asc = oracle_formats.quantize(a, recipe, "act")
    y = oracle_linear.exact64(aq, asc, recipe) @ oracle_linear.exact64(q, scale, recipe).T
    return y if bias is None else y + bias.double()


def check(got, eager, exact, dtype, what, slack=1.0):
    rel = oracle_stats.rel_l2(got.cpu(), exact)
    assert rel <= REL_L2[dtype] * slack, (what, rel)
    oracle_stats.assert_no_regression(got.cpu(), eager, exact, name=what)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("recipe,dgrad", [("mx", True), ("mx", False), ("tensor", True), ("tensor", False), ("row", True), ("row", False), ("block", True), ("block", False)])
def test_fp8_linear_forward_and_grads(dtype, recipe, dgrad):
    m, n, k = 300, 384, 512
    x, w, bias, dy, base = problem(m, n, k, dtype, recipe, dgrad)
    op = registry.resolve("fp8_linear", DEV, dtype, recipe=recipe)
    assert op.backend == "hip" and op.order == ("hip",)
    xd = x.to(DEV).requires_grad_(True)
    bd = bias.to(DEV).requires_grad_(True)
    q, s, aux, q_t, s_t, aux_t = parts(base, DEV)
    y = op(xd, q, s, aux, q_t, s_t, aux_t, bd, recipe)
    y.backward(dy.to(DEV))
    assert y.dtype == dtype and y.shape == (m, n) and xd.grad.shape == (m, k)

    eager_y = oracle_linear.fp8_forward(x, base.q, base.scale, None, bias, recipe)
    exact_y = exact_product(x, base.q, base.scale, bias, recipe)
    check(y.detach(), eager_y, exact_y, dtype, f"fwd {recipe}")
    eager_dx = oracle_linear.fp8_dgrad(dy, base.q, base.scale, base.q_t, base.scale_t, None, recipe)
    if dgrad:
        exact_dx = exact_product(dy, base.q_t, base.scale_t, None, recipe)
    else:
        exact_dx = dy.double() @ oracle_linear.exact64(base.q, base.scale, recipe)
    # the 16-bit path rounds q * scale to the activation dtype first: exact for mx (powers of
    # two), one more 2^-9 rounding per weight for fp32 scales, in the eager path just the same
    slack = 1.0 if dgrad or recipe == "mx" else 2.0
    check(xd.grad, eager_dx, exact_dx, dtype, f"dgrad {recipe} fp8={dgrad}", slack)
    assert torch.equal(bd.grad.cpu(), oracle_linear.bias_grad(dy, dtype))


def test_infer_op_equals_autograd_op_and_leading_dims():
    x, w, bias, dy, base = problem(256, 256, 384, torch.bfloat16, "mx")
    train = registry.resolve("fp8_linear", DEV, torch.bfloat16, recipe="mx")
    infer = registry.resolve("fp8_linear_infer", DEV, torch.bfloat16, recipe="mx")
    args = parts(base, DEV)
    x3 = x.to(DEV).reshape(2, 128, 384)
    a = train(x3, *args, bias.to(DEV), "mx")
    b = infer(x3, *args, bias.to(DEV), "mx")
    assert a.shape == (2, 128, 256) and torch.equal(a, b) and not b.requires_grad
    assert torch.equal(a.reshape(256, 256), train(x.to(DEV), *args, bias.to(DEV), "mx"))


def test_fullgraph_compile_traces_the_custom_op():
    x, w, bias, dy, base = problem(128, 256, 256, torch.bfloat16, "mx")
    op = registry.resolve("fp8_linear", DEV, torch.bfloat16, recipe="mx")
    args = parts(base, DEV)
    bd = bias.to(DEV)

    def f(t):
        return op(t, *args, bd, "mx") * 2

    want = f(x.to(DEV))
    xg = x.to(DEV).requires_grad_(True)
    got = torch.compile(f, fullgraph=True, backend="aot_eager")(xg)
    assert torch.equal(got, want)
    got.sum().backward()
    xe = x.to(DEV).requires_grad_(True)
    f(xe).sum().backward()
    assert torch.equal(xg.grad, xe.grad)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fmt", ["int8", "fp8"])
def test_quant_linear_op(dtype, fmt):
    m, n, k = 200, 320, 448
    g = torch.Generator().manual_seed(3)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randn(n, k, generator=g) * 0.05
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    q, scale = oracle_linear.quantize_weight(w, fmt)
    op = registry.resolve("quant_linear", DEV, dtype, fmt=fmt)
    assert op.backend == "hip"
    xd = x.to(DEV).requires_grad_(True)
    y = op(xd, q.to(DEV), scale.to(DEV), bias.to(DEV), fmt)
    y.backward(dy.to(DEV))
    w64 = oracle_linear.wo_exact64(q, scale)
    exact_y, exact_dx = x.double() @ w64.T + bias.double(), dy.double() @ w64
    check(y.detach(), oracle_linear.wo_forward(x, q, scale, bias), exact_y, dtype, f"wo fwd {fmt}")
    # the per-row scale lies on the contraction axis of the input gradient, so it is folded into
    # a 16-bit operand (one extra rounding, as in the eager launcher): twice the forward bound
    check(xd.grad, oracle_linear.wo_dgrad(dy, q, scale), exact_dx, dtype, f"wo dgrad {fmt}", slack=2.0)


def test_shortlist_is_timed_once_and_stored(tmp_path, monkeypatch):
    monkeypatch.setenv("KOHAKUMOSS_KERNEL_CACHE", str(tmp_path))
    tuning._tables.clear()
    tuning.set_mode("table")
    tuning.reset()
    x, w, bias, dy, base = problem(512, 512, 512, torch.bfloat16, "mx")
    op = registry.resolve("fp8_linear", DEV, torch.bfloat16, recipe="mx")
    args = parts(base, DEV)
    before = tuning.TIMED.get("fp8_fwd", 0)
    a = op(x.to(DEV), *args, bias.to(DEV), "mx")
    b = op(x.to(DEV), *args, bias.to(DEV), "mx")
    assert tuning.TIMED.get("fp8_fwd", 0) == before + 1 and torch.equal(a, b)
    rows = [p for p in tmp_path.rglob("fp8_fwd.json")]
    assert len(rows) == 1 and "fwd_m512_n512_k512" in rows[0].read_text()
    tuning._tables.clear()


def test_text_encoder_linears_on_device():
    """A text-encoder-shaped MLP of plain nn.Linear modules (4096 -> 12288 -> 4096 scaled down) quantized
    in place on the card: weight-only int8 and fp8 through the weight-only kernels, mxfp8 through the
    fp8 op, per-group int8 through its own module; outputs close to the dense ones, state keys under
    `qweight`, and a kept fp32 linear fed 16-bit activations still runs."""
    from kohakumosstrainer_amd.quant import GroupQuantLinear, QuantLinear, quantize_text_linears

    def mlp():
        torch.manual_seed(1)
        m = nn.Sequential(nn.Linear(512, 1536), nn.GELU(), nn.Linear(1536, 512, bias=False)).to(DEV, torch.bfloat16)
        return m

    x = torch.randn(3, 50, 512, device=DEV, dtype=torch.bfloat16)
    want = mlp()(x).float()
    for precision, group, bound in (("int8", 0, 2e-2), ("fp8", 0, 6e-2), ("mxfp8", 0, 8e-2), ("int8", 128, 2e-2)):
        m = mlp()
        report = quantize_text_linears(m, precision, group, torch.bfloat16, recipe="mx")
        assert report["layers"] == 2 and report["skipped"] == 0 and report["quant_bytes"] < report["dense_bytes"]
        kind = GroupQuantLinear if group else QuantLinear
        assert isinstance(m[0], kind) and isinstance(m[2], kind)
        y = m(x)
        assert y.dtype == torch.bfloat16 and y.shape == want.shape
        rel = ((y.float() - want).norm() / want.norm()).item()
        assert rel < bound, (precision, group, rel)
        if not group:
            assert any(k.startswith("0.qweight.") for k in m.state_dict())
    from kohakumosstrainer_amd.model.linear import MossLinear as ML

    kept = ML(512, 256).to(DEV)  # fp32 parameters, 16-bit activations
    kept.init_weights(0.05)
    assert kept(x).dtype == torch.bfloat16


def test_modules_end_to_end_on_device():
    torch.manual_seed(0)
    model = nn.ModuleDict({"qkv": MossLinear(512, 1536, bias=True), "out": MossLinear(512, 512, bias=False)}).to(DEV, torch.bfloat16)
    for m in model.values():
        m.init_weights(0.05)
    x = torch.randn(4, 96, 512, device=DEV, dtype=torch.bfloat16)
    ref = {k: m(x).float() for k, m in model.items()}
    report = quantize_model(model, "mxfp8", dgrad=True)
    assert report["layers"] == 2
    for k, m in model.items():
        assert isinstance(m.base, ComputeWeight) and m.base.q.device.type == "cuda"
        y = m(x)
        assert y.dtype == torch.bfloat16
        rel = ((y.float() - ref[k]).norm() / ref[k].norm()).item()
        assert rel < 6e-2, (k, rel)
    # the device quantizer produced the same parts the host formats give
    w = torch.randn(512, 512) * 0.05
    qd, sd, auxd = quantize_pair(w.to(DEV, torch.bfloat16), "mx")
    qh, sh, auxh = quantize_pair(w.to(torch.bfloat16), "mx")
    assert torch.equal(qd.cpu().view(torch.uint8), qh.view(torch.uint8)) and torch.equal(sd.cpu(), sh) and torch.equal(auxd.cpu(), auxh)
    # int8 weight-only base on the same modules
    lin = MossLinear(512, 768).to(DEV, torch.bfloat16)
    lin.init_weights(0.05)
    want = lin(x).float()
    quantize_model(nn.ModuleDict({"l": lin}), "int8")
    assert isinstance(lin.base, QuantWeight)
    assert ((lin(x).float() - want).norm() / want.norm()).item() < 1e-2


def test_trainable_fp8_cache_refreshes_from_the_device_quantizers():
    torch.manual_seed(1)
    lin = MossLinear(512, 384, bias=True).to(DEV, torch.bfloat16)
    lin.init_weights(0.05)
    (got,) = attach_compute(nn.ModuleDict({"l": lin}), "mxfp8", default_filter(()), torch.bfloat16, dgrad=True)
    cache = lin.compute
    hq, hs = oracle_formats.quantize(lin.weight.detach().cpu(), "mx", "weight")
    assert torch.equal(cache.q.cpu().view(torch.uint8), hq.view(torch.uint8)) and torch.equal(cache.scale.cpu(), hs)
    tq, ts = oracle_formats.quantize(lin.weight.detach().cpu().t().contiguous(), "mx", "weight")
    assert torch.equal(cache.q_t.cpu().view(torch.uint8), tq.view(torch.uint8)) and torch.equal(cache.scale_t.cpu(), ts)
    x = torch.randn(256, 512, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    g = torch.randn(256, 384, device=DEV, dtype=torch.bfloat16)
    lin(x).backward(g)
    ref_w = (g.double().t() @ x.detach().double()).cpu()
    assert oracle_stats.rel_l2(lin.weight.grad.cpu(), ref_w) < 5e-3
    assert torch.equal(lin.bias.grad.cpu(), oracle_linear.bias_grad(g.cpu(), torch.bfloat16))
    exact_dx = exact_product(g.cpu(), tq, ts, None, "mx")
    assert oracle_stats.rel_l2(x.grad.cpu(), exact_dx) < 2e-3


def test_trainable_fp8_cache_block_recipe():
    """The trainable-weight op under the block recipe: both copies come from the device block
    quantizer (the W^T copy through the transposed view) and equal the host's bytes."""
    torch.manual_seed(2)
    lin = MossLinear(512, 384, bias=True).to(DEV, torch.bfloat16)
    lin.init_weights(0.05)
    attach_compute(nn.ModuleDict({"l": lin}), "fp8_compute", default_filter(()), torch.bfloat16, recipe="block", dgrad=True)
    cache = lin.compute
    assert cache.recipe == "block"
    hq, hs = oracle_formats.quantize(lin.weight.detach().cpu(), "block", "weight")
    assert torch.equal(cache.q.cpu().view(torch.uint8), hq.view(torch.uint8)) and torch.equal(cache.scale.cpu(), hs)
    tq, ts = oracle_formats.quantize(lin.weight.detach().cpu().t().contiguous(), "block", "weight")
    assert torch.equal(cache.q_t.cpu().view(torch.uint8), tq.view(torch.uint8)) and torch.equal(cache.scale_t.cpu(), ts)
    x = torch.randn(256, 512, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    g = torch.randn(256, 384, device=DEV, dtype=torch.bfloat16)
    y = lin(x)
    y.backward(g)
    exact_y = exact_product(x.detach().cpu(), hq, hs, lin.bias.detach().cpu(), "block")
    assert oracle_stats.rel_l2(y.detach().cpu(), exact_y) < 2e-3
    ref_w = (g.double().t() @ x.detach().double()).cpu()
    assert oracle_stats.rel_l2(lin.weight.grad.cpu(), ref_w) < 5e-3
    exact_dx = exact_product(g.cpu(), tq, ts, None, "block")
    assert oracle_stats.rel_l2(x.grad.cpu(), exact_dx) < 2e-3


def test_lora_training_step_over_frozen_mxfp8_base():
    """One adapter training step at the text-encoder shape with the benchmark's operand
    statistics: x ~N(0,1) [2048, 4096], frozen W ~N(0,0.02) [12288, 4096] as an MXFP8 base
    (forward, and the input gradient through the copy quantized along N, on the HIP kernels),
    rank-8 bypass A ~N(0,1/8) [8, 4096], B ~N(0,1e-3) [12288, 8], gamma = 1, added in bf16,
    incoming gradient ~N(0,1e-2); seeds 0 / 1 / 2 / 3 for x / W / dy / the factors. Output, input
    gradient and both factor gradients against the same step in fp64 from the stored codes (the
    closed form y = base(x) + (x A^T) B^T)."""
    m, k, n, r = 2048, 4096, 12288, 8
    g = torch.Generator()
    x = torch.randn(m, k, generator=g.manual_seed(0)).to(torch.bfloat16)
    w = (torch.randn(n, k, generator=g.manual_seed(1)) * 0.02).to(torch.bfloat16)
    dy = (torch.randn(m, n, generator=g.manual_seed(2)) * 1e-2).to(torch.bfloat16)
    g.manual_seed(3)
    down = (torch.randn(r, k, generator=g) / 8).to(torch.bfloat16)
    up = (torch.randn(n, r, generator=g) * 1e-3).to(torch.bfloat16)

    lin = MossLinear(k, n, bias=False).to(torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    lin = lin.to(DEV)
    quantize_model(nn.ModuleDict({"l": lin}), "mxfp8", dgrad=True)
    base = lin.base
    dn = down.to(DEV).requires_grad_(True)
    upd = up.to(DEV).requires_grad_(True)
    xd = x.to(DEV).requires_grad_(True)
    y = lin(xd) + (xd @ dn.t()) @ upd.t()
    y.backward(dy.to(DEV))

    q, s, q_t, s_t = (t.cpu() for t in (base.q, base.scale, base.q_t, base.scale_t))
    y_ref = exact_product(x, q, s, None, "mx") + (x.double() @ down.double().T) @ up.double().T
    assert oracle_stats.rel_l2(y.detach().cpu(), y_ref) < 4e-3
    # the eager step with the same parts: the 10x rule on the output and the input gradient
    eager_y = oracle_linear.lora_bypass(oracle_linear.fp8_forward(x, q, s, None, None, "mx"), x, down, up, 1.0)
    oracle_stats.assert_no_regression(y.detach().cpu(), eager_y, y_ref, name="lora fwd")
    dx_ref = exact_product(dy, q_t, s_t, None, "mx") + (dy.double() @ up.double()) @ down.double()
    assert oracle_stats.rel_l2(xd.grad.cpu(), dx_ref) < 4e-3
    up_ref = dy.double().t() @ (x.double() @ down.double().t())
    dn_ref = (dy.double() @ up.double()).t() @ x.double()
    assert oracle_stats.rel_l2(upd.grad.cpu(), up_ref) < 1e-2 and oracle_stats.rel_l2(dn.grad.cpu(), dn_ref) < 1e-2


@pytest.mark.parametrize("fmt", ("int8", "fp8"))
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("n,k", ((3072, 3072), (100, 136), (7, 40)))
def test_weight_quantizer_on_the_card_equals_the_oracle(fmt, dtype, n, k):
    """`weights.quantize` of a 16-bit weight on the GPU runs the per-row quantizer kernels: codes
    and scales bit for bit those of the oracle's frozen-base quantizer (reference
    `src/kohakumoss/quant/weights.py:31-43`), an all-zero row and a row with one huge entry included."""
    from kohakumosstrainer_amd.quant.weights import quantize

    g = torch.Generator().manual_seed(n + k)
    w = (torch.randn(n, k, generator=g) * 0.05).to(dtype)
    w[0] = 0
    w[1, 3] = 300.0
    q_want, s_want = oracle_linear.quantize_weight(w, fmt)
    q, s = quantize(w.cuda(), fmt)
    assert q.dtype == q_want.dtype and s.dtype == torch.float32
    assert torch.equal(s.cpu(), s_want)
    assert torch.equal(q.cpu().view(torch.uint8), q_want.view(torch.uint8))
