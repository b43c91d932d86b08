"""Module API on the host: quantized base storage, the nn.Linear replacements and what the
autograd graph keeps alive. Mirrors reference `tests/quant/test_quant.py:56-113`,
`tests/quant/test_eager_saved.py` and the packed-scale layout against its index formula."""

import pytest
import torch
from torch import nn

from kohakumosstrainer_amd.kernels.fp8 import formats
from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant import ComputeCache, ComputeWeight, QuantLinear, QuantWeight, attach_compute, default_filter, quantize, quantize_model, quantize_torch_linears
from kohakumosstrainer_amd.quant.compute import eligible, quantize_pair, recipe_of
from oracle import formats as oracle_formats
from oracle import linear as oracle_linear


def close(got, ref, bound=2e-2):
    rel = ((got - ref).norm() / ref.norm()).item()
    assert rel < bound, rel


def must_fail(check, what=""):
    try:
        check()
    except AssertionError:
        return
    raise AssertionError(f"check passed on the broken variant: {what}")


def test_package_formats_equal_the_oracle_bit_for_bit():
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(130, 256, generator=g) * torch.logspace(-4, 2, 130)[:, None]).to(torch.bfloat16)
    x[1] = 0
    for recipe, role in (("mx", "act"), ("tensor", "act"), ("row", "act"), ("block", "act"), ("block", "weight")):
        q, s = formats.quantize(x, recipe, role)
        rq, rs = oracle_formats.quantize(x, recipe, role)
        assert torch.equal(q.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(s, rs), recipe
        assert torch.equal(formats.dequantize(q, s, recipe, torch.bfloat16), oracle_formats.dequantize(rq, rs, recipe, torch.bfloat16))
    s = torch.randint(0, 255, (300, 96), dtype=torch.uint8)
    assert torch.equal(formats.swizzle_mx(s), oracle_formats.swizzle_mx(s))
    w = torch.randn(48, 40, generator=g)
    for fmt in ("int8", "fp8"):
        q, sc = quantize(w, fmt)
        rq, rsc = oracle_linear.quantize_weight(w, fmt)
        assert torch.equal(q.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(sc, rsc)


@pytest.mark.parametrize("rows,blocks", [(128, 4), (200, 12), (1, 4), (300, 96)])
def test_pack_mx_matches_index_formula(rows, blocks):
    s = torch.randint(1, 255, (rows, blocks), dtype=torch.uint8)
    flat = formats.pack_mx(s)
    groups = -(-rows // 128)
    assert flat.numel() == formats.packed_numel(rows, blocks * 32) == (blocks // 4) * groups * 512
    want = torch.zeros_like(flat)
    for r in range(rows):
        for b in range(blocks):
            want[((((b // 4) * groups + r // 128) * 16 + r % 16) * 4 + b % 4) * 8 + (r % 128) // 16] = s[r, b]
    assert torch.equal(flat, want)
    with pytest.raises(ValueError):
        formats.pack_mx(s[:, :3])


def test_quantize_model_replaces_and_forward_close():
    lin = MossLinear(512, 384, bias=True)
    lin.init_weights(0.05)
    x = torch.randn(7, 512)
    ref = lin(x)
    report = quantize_model(nn.ModuleDict({"lin": lin}), "int8")
    assert report["layers"] == 1 and report["quant_bytes"] < report["dense_bytes"] / 3
    assert isinstance(lin.base, QuantWeight) and lin.weight.numel() == 0
    close(lin(x), ref, 1e-2)
    lin.clear_base()
    assert lin.base is None and lin.is_plain


def test_quantize_model_mxfp8_parts_and_filter():
    model = nn.ModuleDict({"a": MossLinear(256, 384, bias=False), "keep": MossLinear(256, 256), "odd": MossLinear(320, 300), "tiny": MossLinear(64, 512)})
    for m in model.values():
        m.init_weights(0.05)
    x = torch.randn(5, 256)
    ref = model["a"](x)
    report = quantize_model(model, "mxfp8", accept=default_filter(("keep",)), dgrad=True)
    assert report["layers"] == 1 and report["skipped"] == 1, report
    base = model["a"].base
    assert isinstance(base, ComputeWeight) and base.recipe == "mx" and base.has_dgrad
    assert base.q.shape == (384, 256) and base.scale.shape == (384, 8) and base.scale.dtype == torch.uint8
    assert base.q_t.shape == (256, 384) and base.scale_t.shape == (256, 12)
    assert base.aux.numel() == formats.packed_numel(384, 256) and base.aux_t.numel() == formats.packed_numel(256, 384)
    assert model["keep"].base is None and model["odd"].base is None and model["tiny"].base is None
    close(model["a"](x), ref, 6e-2)
    assert recipe_of("mxfp8") == "mx" and recipe_of("fp8_compute", "tensor") == "tensor"
    assert eligible(384, 256) is None and eligible(200, 256) is not None


def test_quantize_torch_linears_on_plain_linears():
    holder = nn.ModuleDict({"a": nn.Linear(256, 256), "inner": nn.ModuleDict({"b": nn.Linear(256, 300, bias=False)}), "small": nn.Linear(100, 300)})
    x = torch.randn(3, 256)
    refs = {"a": holder["a"](x), "b": holder["inner"]["b"](x)}
    bias = holder["a"].bias.clone()
    assert quantize_torch_linears(holder, "int8", torch.float32) == 2
    assert type(holder["small"]) is nn.Linear
    got = {"a": holder["a"], "b": holder["inner"]["b"]}
    for name, layer in got.items():
        assert isinstance(layer, QuantLinear), name
        close(layer(x), refs[name])
    assert torch.equal(got["a"].bias, bias) and got["b"].bias is None
    must_fail(lambda: close(got["b"](x)[:, :256], refs["a"]), "another layer's output")


def test_only_quantized_parts_are_saved_for_backward():
    """No 16-bit weight copy may stay alive from forward to backward."""
    w = torch.randn(256, 256) * 0.05
    for base in (QuantWeight.from_weight(w, "int8"), ComputeWeight.from_weight(w, "mx", dgrad=True)):
        saved = []
        x = torch.randn(4, 256, requires_grad=True)
        with torch.autograd.graph.saved_tensors_hooks(lambda t: saved.append(t) or t, lambda t: t):
            y = base.linear(x, None)
        y.sum().backward()
        assert x.grad is not None and x.grad.shape == x.shape
        for t in saved:
            assert t.dtype in (torch.int8, torch.uint8, torch.float8_e4m3fn, torch.float32) and t.numel() < w.numel() * 2, (t.dtype, t.shape)
            if t.dtype == torch.float32:
                assert t.dim() == 1, "only the per-row scale may be fp32"


def test_compute_weight_stored_and_add_dgrad():
    w = torch.randn(256, 384) * 0.05
    q, s, aux = quantize_pair(w, "mx")
    base = ComputeWeight.from_stored("mx", q, s)
    assert not base.has_dgrad and torch.equal(base.aux, aux)
    base.add_dgrad()
    want_q, want_s, _ = quantize_pair(base.weight(torch.float32).t(), "mx")
    assert torch.equal(base.q_t.view(torch.uint8), want_q.view(torch.uint8)) and torch.equal(base.scale_t, want_s)
    assert set(base.tensors()) == {"q", "scale", "aux", "q_t", "scale_t", "aux_t"}
    x = torch.randn(6, 384, requires_grad=True)
    y = base.linear(x, torch.zeros(256))
    y.backward(torch.randn(6, 256))
    eager = oracle_linear.fp8_forward(x.detach(), q, s, None, torch.zeros(256), "mx")
    assert torch.equal(y.detach(), eager)
    with pytest.raises(ValueError):
        ComputeWeight("nope", {"q": q, "scale": s})


def test_compute_cache_train_op_gives_weight_gradient():
    lin = MossLinear(256, 384, bias=True)
    lin.init_weights(0.05)
    nn.init.normal_(lin.bias, std=0.1)
    (got,) = attach_compute(nn.ModuleDict({"l": lin}), "mxfp8", default_filter(()), torch.float32, dgrad=True)
    assert got is lin and isinstance(lin.compute, ComputeCache) and not lin.is_plain
    x = torch.randn(10, 256, requires_grad=True)
    y = lin(x)
    g = torch.randn(10, 384)
    y.backward(g)
    ref_w = g.double().t() @ x.detach().double()
    close(lin.weight.grad.double(), ref_w, 1e-5)
    close(lin.bias.grad.double(), g.double().sum(0), 1e-5)
    close(x.grad.double(), g.double() @ lin.weight.detach().double(), 8e-2)
    old = lin.compute.q.clone()
    with torch.no_grad():
        lin.weight.mul_(2.0)
    lin.compute.refresh(lin.weight)
    assert torch.equal(lin.compute.q.view(torch.uint8), old.view(torch.uint8)) and not torch.equal(lin.compute.scale, formats.quantize(lin.weight / 4, "mx")[1])
    lin.set_compute(None)
    assert lin.is_plain


def test_fp32_layer_takes_16bit_activations():
    """A layer kept in fp32 (a conditioning projection) runs in the activation's type: weight and
    bias are cast per call (reference `src/kohakumoss/model/linear.py:79-83`)."""
    for bias in (True, False):
        lin = MossLinear(64, 48, bias=bias)
        lin.init_weights(0.05)
        if bias:
            nn.init.normal_(lin.bias, std=0.1)
        x = torch.randn(5, 64).to(torch.bfloat16)
        y = lin(x)
        assert y.dtype == torch.bfloat16
        want = nn.functional.linear(x, lin.weight.to(torch.bfloat16), lin.bias.to(torch.bfloat16) if bias else None)
        assert torch.equal(y, want)
        assert lin.weight.dtype == torch.float32


def test_set_base_none_keeps_the_dense_weight():
    lin = MossLinear(256, 256, bias=False)
    lin.init_weights(0.05)
    dense = lin.weight.detach().clone()
    x = torch.randn(3, 256)
    ref = lin(x)
    lin.set_base(None)
    assert lin.base is None and lin.is_plain and torch.equal(lin.weight, dense)
    assert torch.equal(lin(x), ref)
    # attaching does not touch the parameter either: whoever attaches decides about it
    base = QuantWeight.from_weight(dense, "int8")
    lin.set_base(base)
    assert lin.base is base and not lin.is_plain and torch.equal(lin.weight, dense)
    close(lin(x), ref, 1e-2)
    lin.set_base(None)
    assert lin.base is None and "base" not in lin._modules and torch.equal(lin(x), ref)
    # a base that is no module (a streamed handle) attaches and detaches the same way
    class Handle:
        def linear(self, x, bias):
            return x[:, :1] * 0 + 7.0
    lin.set_base(Handle())
    assert float(lin(x)[0, 0]) == 7.0
    lin.clear_base()
    assert torch.equal(lin(x), ref)


def test_is_plain_sees_a_patched_forward_and_init_is_gaussian():
    lin = MossLinear(64, 64)
    assert lin.is_plain
    lin.forward = lambda x: x  # what an adapter library does to the instance
    assert not lin.is_plain
    del lin.forward
    assert lin.is_plain
    big = MossLinear(512, 512, bias=True)
    torch.manual_seed(3)
    big.init_weights(0.02)
    torch.manual_seed(3)
    want = torch.empty(512, 512).normal_(std=0.02)
    assert torch.equal(big.weight.detach(), want), "init_weights draws the weight with normal_ (same stream)"
    assert float(big.weight.detach().abs().max()) > 3 * 0.02, "an untruncated normal has tails beyond 3 sigma at this size"
    assert torch.count_nonzero(big.bias) == 0


def test_deleted_weight_leaves_a_typed_stand_in():
    lin = MossLinear(32, 16, dtype=torch.bfloat16)
    assert lin.weight_like is lin.weight
    del lin.weight
    held = lin.weight_like
    assert held.numel() == 0 and held.dtype == torch.bfloat16
    lin.to(torch.float16)
    assert lin.weight_like.dtype == torch.float16


def test_keep_filter_is_by_prefix_not_substring():
    accept = default_filter(("t_embedder", "final"), min_features=16)
    lin = MossLinear(64, 64)
    assert not accept("t_embedder", lin) and not accept("t_embedder.mlp.0", lin) and not accept("final.proj", lin)
    assert accept("blocks.0.t_embedder_proj", lin), "a name that only contains a kept key is quantized"
    assert accept("blocks.3.final", lin) and accept("t_embedder2.x", lin)
    assert not accept("x", MossLinear(8, 64))


def test_quantlinear_state_keys_use_qweight():
    """State of a QuantLinear must load on the other side: the base sits under `qweight`
    (reference `src/kohakumoss/quant/convert.py:78-79`)."""
    plain = nn.Linear(256, 256)
    ql = QuantLinear(plain, "int8", torch.float32)
    keys = set(ql.state_dict())
    assert {"qweight.q", "qweight.scale", "bias"} <= keys and not any(k.startswith("base.") for k in keys), keys
    other = QuantLinear(nn.Linear(256, 256), "int8", torch.float32)
    other.load_state_dict(ql.state_dict())
    x = torch.randn(2, 256)
    assert torch.equal(other(x), ql(x))
