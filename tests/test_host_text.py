"""Text-encoder linear quantization on the host: the fate rules agree with what the converter
replaces, per-group codes against a definition-level restatement, bytes accounted as the state dict
has them. Mirrors reference `tests/encoders/text/test_streamed_load_parts.py:85-130`."""

import numpy as np
import pytest
import torch
from torch import nn

from kohakumosstrainer_amd.quant import GroupQuantLinear, QuantLinear, linear_fate, quantize_text_linears, quantizes
from kohakumosstrainer_amd.quant.text import dequantize_groups, quantize_groups


def must_fail(check, what=""):
    try:
        check()
    except AssertionError:
        return
    raise AssertionError(f"check passed on the broken variant: {what}")


def block() -> nn.Module:
    m = nn.Module()
    m.big = nn.Linear(512, 384)
    m.small = nn.Linear(64, 512)
    m.odd = nn.Linear(500, 512)
    m.inner = nn.Sequential(nn.Linear(256, 256, bias=False))
    return m


def assert_fates(fate, precision, group):
    m = block()
    named = {n: c for n, c in m.named_modules() if isinstance(c, nn.Linear)}
    said = {n for n, c in named.items() if fate(c, precision, group) == "quantize"}
    quantize_text_linears(m, precision, group, torch.float32)
    done = {n for n, c in m.named_modules() if n in named and type(c) is not nn.Linear}
    assert said == done, (said, done)
    assert quantizes(block(), precision, group) == bool(done)
    return done


@pytest.mark.parametrize("precision, group", [("int8", 0), ("int8", 128), ("fp8", 0), ("fp8", 64), ("mxfp8", 0)])
def test_linear_fate_is_what_the_converter_replaces(precision, group):
    done = assert_fates(linear_fate, precision, group)
    assert "small" not in done and "big" in done
    assert ("odd" in done) == (precision != "mxfp8" and group == 0), "500 columns: no multiple of a group, no multiple of 128"


def test_fate_check_fails_on_a_broken_fate():
    must_fail(lambda: assert_fates(lambda mod, p, g, mf=256: linear_fate(mod, p, 0, mf), "int8", 128), "group ignored")


def test_compute_precisions_skip_shapes_they_cannot_take():
    m = block()
    report = quantize_text_linears(m, "mxfp8", 0, torch.float32, recipe="mx")
    assert report["layers"] == 2 and report["skipped"] == 1, report  # big, inner.0; odd is skipped; small is left
    assert isinstance(m.big, QuantLinear) and type(m.odd) is nn.Linear and type(m.small) is nn.Linear
    assert linear_fate(m.odd, "mxfp8", 0) == "skip" and linear_fate(m.small, "mxfp8", 0) is None


def test_bytes_reported_are_the_state_dicts():
    m = block()
    before = sum(t.numel() * t.element_size() for t in m.state_dict().values())
    report = quantize_text_linears(m, "int8", 0, torch.float32)
    after = sum(t.numel() * t.element_size() for t in m.state_dict().values())
    assert report["layers"] == 3 and after - before == report["quant_bytes"] - report["dense_bytes"] != 0


@pytest.mark.parametrize("fmt", ("int8", "fp8"))
def test_group_codes_against_the_definition(fmt):
    g = torch.Generator().manual_seed(5)
    w = torch.randn(24, 256, generator=g) * torch.logspace(-3, 1, 24)[:, None]
    w[3, 64:128] = 0.0  # an all-zero group: floor scale, zero codes
    w[5, :5] = torch.tensor([127.0, 0.5, 1.5, -2.5, -127.0])
    group = 64
    q, s = quantize_groups(w, fmt, group)
    assert q.shape == (24, 256) and s.shape == (24, 4) and s.dtype == torch.float32
    limit = 127.0 if fmt == "int8" else 448.0
    for r in range(24):
        for b in range(4):
            run = w[r, b * group : (b + 1) * group].numpy().astype(np.float32)
            want_s = np.float32(max(np.abs(run).max(), np.float32(1e-12))) / np.float32(limit)
            assert s[r, b].item() == want_s, (r, b)
            ratio = run / want_s
            if fmt == "int8":
                want = np.clip(np.rint(ratio), -127, 127).astype(np.int8)
                assert np.array_equal(q[r, b * group : (b + 1) * group].numpy(), want), (r, b)
            else:
                want = torch.from_numpy(np.clip(ratio, -448, 448)).to(torch.float8_e4m3fn)
                assert torch.equal(q[r, b * group : (b + 1) * group].view(torch.uint8), want.view(torch.uint8)), (r, b)
    assert torch.count_nonzero(q[3, 64:128].float()) == 0
    back = dequantize_groups(q, s, torch.float32)
    step = s.repeat_interleave(group, dim=1) * (0.5 if fmt == "int8" else 32.0 / 2)  # half a code step / half the widest e4m3 step
    assert bool(((back - w).abs() <= step * 1.0001).all())
    with pytest.raises(ValueError):
        quantize_groups(w, fmt, 48)
    with pytest.raises(ValueError):
        quantize_groups(w, "int4", 64)


def test_group_linear_forward_and_dtype():
    lin = nn.Linear(256, 300)
    x = torch.randn(7, 256)
    ref = lin(x)
    gl = GroupQuantLinear(lin, "int8", 64)
    assert set(gl.state_dict()) == {"q", "scale", "bias"}
    rel = ((gl(x) - ref).norm() / ref.norm()).item()
    assert rel < 1e-2, rel
    y16 = gl(x.to(torch.bfloat16))
    assert y16.dtype == torch.bfloat16
    coarse = GroupQuantLinear(lin, "int8", 256)
    w = lin.weight.detach()
    assert (dequantize_groups(gl.q, gl.scale, torch.float32) - w).abs().mean() <= (dequantize_groups(coarse.q, coarse.scale, torch.float32) - w).abs().mean()
