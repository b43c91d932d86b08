"""The pre-quantized checkpoint layout (`quant.stored`, reference
`src/kohakumoss/quant/stored.py:16-94`): record and key names, a save / load round trip that
never materialises a 16-bit weight, and the errors. Host only (the eager backend)."""

import json

import pytest
import torch
from torch import nn

from kohakumosstrainer_amd.model.linear import MossLinear
from kohakumosstrainer_amd.quant import stored
from kohakumosstrainer_amd.quant.compute import ComputeWeight


class Tiny(nn.Module):
    def __init__(self):
        super().__init__()
        self.a = MossLinear(256, 128, bias=True)
        self.b = MossLinear(128, 256, bias=False)
        self.small = MossLinear(128, 8)
        self.norm = nn.LayerNorm(8)
        for lin in (self.a, self.b, self.small):
            lin.init_weights(0.05)   # MossLinear leaves its parameters unset until told
            if lin.bias is not None:
                nn.init.normal_(lin.bias, std=0.1)

    def forward(self, x):
        return self.norm(self.small(self.b(self.a(x))[..., :128]))


def quantized_model(recipe, seed=0):
    torch.manual_seed(seed)
    m = Tiny()
    for name in ("a", "b"):
        lin = getattr(m, name)
        lin.set_base(ComputeWeight.from_weight(lin.weight.detach(), recipe))
    return m


@pytest.mark.parametrize("recipe", ("mx", "row", "tensor", "block"))
def test_state_layout_and_record(recipe):
    m = quantized_model(recipe)
    keys = ["a.weight", "a.bias", "b.weight", "small.weight", "small.bias", "norm.weight", "norm.bias"]
    state, meta = stored.quantized_state(m, keys, torch.bfloat16)
    record = json.loads(meta[stored.FP8_KEY])
    assert record == {"recipe": recipe, "layers": ["a", "b"]}
    assert stored.stored_keys(record) == ({"a.weight", "b.weight"}, {"a.weight_scale", "b.weight_scale"})
    assert state["a.weight"].dtype == torch.float8_e4m3fn and state["a.weight"].shape == (128, 256)
    assert torch.equal(state["a.weight"].view(torch.uint8), m.a.base.q.view(torch.uint8))
    assert torch.equal(state["b.weight_scale"], m.b.base.scale)
    assert state["small.weight"].dtype == torch.bfloat16 and state["norm.bias"].dtype == torch.bfloat16
    assert set(state) == set(keys) | {"a.weight_scale", "b.weight_scale"}


def test_one_recipe_per_checkpoint_and_folded_models_refuse():
    m = quantized_model("mx")
    m.b.set_base(ComputeWeight.from_weight(torch.randn(256, 128), "row"))
    with pytest.raises(ValueError, match="one fp8 recipe"):
        stored.quantized_state(m, ["a.weight"], torch.bfloat16)
    m = quantized_model("mx")
    m.fold_scales = {"x": 1.0}
    with pytest.raises(ValueError, match="folded"):
        stored.quantized_state(m, ["a.weight"], torch.bfloat16)


@pytest.mark.parametrize("recipe", ("mx", "row", "block"))
def test_save_load_round_trip(tmp_path, recipe):
    m = quantized_model(recipe, seed=1)
    path = tmp_path / "model.safetensors"
    record = stored.save_quantized(m, path, torch.float32)
    assert stored.read_record(path) == record == {"recipe": recipe, "layers": ["a", "b"]}
    assert stored.read_record(tmp_path / "absent.safetensors") is None
    fresh = Tiny()
    n = stored.load_quantized(fresh, path, "cpu", torch.float32)
    assert n == 2
    for name in ("a", "b"):
        lin, src = getattr(fresh, name), getattr(m, name)
        assert isinstance(lin.base, ComputeWeight) and lin.base.recipe == recipe
        assert lin.weight.numel() == 0, "no dense copy of a stored layer is kept"
        assert torch.equal(lin.base.q.view(torch.uint8), src.base.q.view(torch.uint8))
        assert torch.equal(lin.base.scale, src.base.scale)
    assert torch.equal(fresh.small.weight, m.small.weight) and torch.equal(fresh.a.bias, m.a.bias)
    x = torch.randn(5, 256)
    assert torch.equal(fresh(x), m(x))


def test_plain_file_loads_without_a_record(tmp_path):
    from safetensors.torch import save_file

    torch.manual_seed(2)
    m = Tiny()
    path = tmp_path / "plain.safetensors"
    save_file({k: v.contiguous() for k, v in m.state_dict().items()}, str(path))
    assert stored.read_record(path) is None
    fresh = Tiny()
    assert stored.load_quantized(fresh, path, "cpu", torch.float32) == 0
    assert torch.equal(fresh.a.weight, m.a.weight)


ALL_KEYS = ["a.weight", "a.bias", "b.weight", "small.weight", "small.bias", "norm.weight", "norm.bias"]


def test_record_naming_absent_tensors_or_wrong_shapes_fails(tmp_path):
    from safetensors.torch import save_file

    m = quantized_model("row")
    state, meta = stored.quantized_state(m, ALL_KEYS, torch.float32)
    broken = dict(state)
    del broken["b.weight_scale"]
    save_file(broken, str(tmp_path / "lacks.safetensors"), metadata=meta)
    with pytest.raises(KeyError, match="record names"):
        stored.load_quantized(Tiny(), tmp_path / "lacks.safetensors", "cpu", torch.float32)
    wrong = dict(state)
    wrong["a.weight"] = wrong["a.weight"][:64].contiguous()
    save_file(wrong, str(tmp_path / "shape.safetensors"), metadata=meta)
    with pytest.raises(ValueError, match="stored codes"):
        stored.load_quantized(Tiny(), tmp_path / "shape.safetensors", "cpu", torch.float32)


def test_a_missing_or_misspelt_plain_tensor_is_an_error(tmp_path):
    """Nothing of the model may silently keep its initial value, and the file may hold nothing the
    model does not know."""
    from safetensors.torch import save_file

    m = quantized_model("mx")
    state, meta = stored.quantized_state(m, ALL_KEYS, torch.float32)
    short = {k: v for k, v in state.items() if k != "small.bias"}
    save_file(short, str(tmp_path / "short.safetensors"), metadata=meta)
    with pytest.raises(KeyError, match="small.bias"):
        stored.load_quantized(Tiny(), tmp_path / "short.safetensors", "cpu", torch.float32)
    extra = dict(state)
    extra["smal.bias"] = state["small.bias"].clone()
    save_file(extra, str(tmp_path / "extra.safetensors"), metadata=meta)
    with pytest.raises(KeyError, match="smal.bias"):
        stored.load_quantized(Tiny(), tmp_path / "extra.safetensors", "cpu", torch.float32)


@pytest.mark.parametrize("codes_as", ("e4m3", "bytes"))
def test_file_in_the_exporters_layout_loads(tmp_path, codes_as):
    """A file laid out as the reference's exporter writes it (`quantized_state` ->
    safetensors): codes under `<path>.weight` in float8_e4m3fn, scales under
    `<path>.weight_scale`, the record in the metadata. Files of an earlier version of this package
    (codes as bytes) load too. What `save_quantized` writes has the e4m3 dtype in the file."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    m = quantized_model("mx", seed=3)
    state, meta = stored.quantized_state(m, ALL_KEYS, torch.bfloat16)
    assert state["a.weight"].dtype == torch.float8_e4m3fn
    if codes_as == "bytes":
        state = {k: (v.view(torch.uint8) if v.dtype == torch.float8_e4m3fn else v) for k, v in state.items()}
    save_file(state, str(tmp_path / "ref.safetensors"), metadata=meta)
    fresh = Tiny()
    assert stored.load_quantized(fresh, tmp_path / "ref.safetensors", "cpu", torch.bfloat16) == 2
    assert torch.equal(fresh.a.base.q.view(torch.uint8), m.a.base.q.view(torch.uint8)) and fresh.a.base.q.dtype == torch.float8_e4m3fn
    assert torch.equal(fresh.b.base.scale, m.b.base.scale)
    stored.save_quantized(m, tmp_path / "ours.safetensors", torch.bfloat16)
    with safe_open(str(tmp_path / "ours.safetensors"), framework="pt") as f:
        assert f.get_tensor("a.weight").dtype == torch.float8_e4m3fn


def test_meta_initialised_model_loads_without_dense_copies(tmp_path):
    m = quantized_model("row", seed=4)
    stored.save_quantized(m, tmp_path / "m.safetensors", torch.float32)
    with torch.device("meta"):
        empty = Tiny.__new__(Tiny)
        nn.Module.__init__(empty)
        empty.a, empty.b, empty.small, empty.norm = MossLinear(256, 128, bias=True), MossLinear(128, 256, bias=False), MossLinear(128, 8), nn.LayerNorm(8)
    assert empty.a.weight.is_meta
    assert stored.load_quantized(empty, tmp_path / "m.safetensors", "cpu", torch.float32) == 2
    assert empty.a.weight.numel() == 0 and not any(p.is_meta for p in empty.parameters())
    x = torch.randn(3, 256)
    assert torch.equal(empty(x), m(x))


def test_streamed_slot_linear_holds_no_slot_tensor_in_the_graph():
    """A weight-streaming ring refills its slot between a layer's forward and backward. The
    streamed view must fetch the parts again for the input gradient: here the slot buffers are
    overwritten with another layer's codes right after the forward, and `fetch` copies the right
    layer back in when asked. Gradients equal those of the resident base."""
    from kohakumosstrainer_amd.quant.compute import ComputeWeight, StreamedParts

    g = torch.Generator().manual_seed(0)
    w_a, w_b = torch.randn(96, 128, generator=g) * 0.05, torch.randn(96, 128, generator=g) * 0.05
    layers = {"a": ComputeWeight.from_weight(w_a, "mx", dgrad=True), "b": ComputeWeight.from_weight(w_b, "mx", dgrad=True)}
    slot = {name: t.clone() for name, t in layers["a"].tensors().items()}
    fetched = []

    def fetch_a():
        fetched.append(len(fetched))
        for name, t in layers["a"].tensors().items():
            slot[name].copy_(t)
        return slot

    view = StreamedParts("mx", fetch_a, torch.float32, "cpu")
    x = torch.randn(10, 128, generator=g, requires_grad=True)
    bias = torch.randn(96, generator=g, requires_grad=True)
    y = view.linear(x, bias)
    for name, t in layers["b"].tensors().items():  # the ring moves on to another layer
        slot[name].copy_(t)
    y.backward(torch.ones_like(y))
    assert len(fetched) == 2, "one fetch per direction"
    x2 = x.detach().clone().requires_grad_()
    b2 = bias.detach().clone().requires_grad_()
    layers["a"].linear(x2, b2).backward(torch.ones_like(y))
    assert torch.equal(y.detach(), layers["a"].linear(x2, b2).detach())
    assert torch.equal(x.grad, x2.grad) and torch.equal(bias.grad, b2.grad)
    assert torch.equal(view.weight(torch.float32), layers["a"].weight(torch.float32))
