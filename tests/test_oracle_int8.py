"""Pins of the int8 compute-linear oracle (`oracle/int8.py`), without a GPU: the reference's
known answers, a definition-level numpy restatement, exact agreement with an fp64 model of the
scheme where every quantization is exact, closeness to it elsewhere, and broken designs that
must fail (reference `tests/kernels/quant/test_int8_linear.py:41-148`)."""

import numpy as np
import pytest
import torch

from oracle import int8 as oi


def must_fail(check, what):
    try:
        check()
    except AssertionError:
        return
    raise AssertionError(f"check passed on the broken variant: {what}")


def rows64(x):
    """The scheme in fp64: per-row codes and scales."""
    s = x.abs().amax(1).clamp_min(1e-12) / 127.0
    return torch.round(x / s[:, None]).clamp(-127, 127), s


def model64(x, q, scale, bias):
    xq, xs = rows64(x.double())
    y = (xq @ q.double().T) * xs[:, None] * scale.double()[None, :]
    return y if bias is None else y + bias.double()


def dx64(g, q, scale, mode):
    if mode == "16bit":
        return g.double() @ (q.double() * scale.double()[:, None])
    gq, gs = rows64(g.double() * scale.double()[None, :])
    return (gq @ q.double()) * gs[:, None]


def weight(n, k, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.05
    scale = w.abs().amax(dim=1).clamp_min(1e-12) / 127.0
    return torch.round(w / scale[:, None]).clamp(-127, 127).to(torch.int8), scale.float(), g


def on_grid(m, k, g):
    """x = codes / 64 with a +-127 code in every row: scales are exactly 1/64 and every code is
    recovered without rounding."""
    codes = torch.randint(-126, 127, (m, k), generator=g).double()
    codes[torch.arange(m), torch.randint(0, k, (m,), generator=g)] = 127.0
    return (codes / 64.0).float()


def test_known_answers_half_even_clamp_and_floor():
    x = torch.tensor([[127.0, 0.5, 1.5, -2.5, -127.0], [0.0, 0.0, 0.0, 0.0, 0.0]])
    q, s = oi.quantize_rows(x)
    assert s[0].item() == 1.0 and s[1].item() == pytest.approx(1e-12 / 127.0)
    assert s[1].item() == float(np.float32(1e-12) / np.float32(127.0))
    assert q[0].tolist() == [127, 0, 2, -2, -127] and q[1].tolist() == [0] * 5
    assert q.dtype == torch.int8 and s.dtype == torch.float32


@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16, torch.float16))
def test_quantizer_matches_numpy_definition(dtype):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(37, 96, generator=g) * torch.logspace(-4, 3, 37)[:, None]).to(dtype)
    cs = torch.rand(96, generator=g) * 1e-2 + 1e-4
    for col in (None, cs):
        q, s = oi.quantize_rows(x, col)
        v = x.float().numpy()
        if col is not None:
            v = v * col.numpy()[None, :]          # fp32 product
        amax = np.maximum(np.abs(v).max(1), np.float32(1e-12))
        sn = (amax / np.float32(127.0)).astype(np.float32)
        qn = np.clip(np.rint(v / sn[:, None]), -127, 127).astype(np.int8)
        assert np.array_equal(s.numpy(), sn) and np.array_equal(q.numpy(), qn)

    amax = torch.rand(4096, generator=g) + 0.5
    assert np.array_equal(oi.row_scale(amax).numpy(), amax.numpy() / np.float32(127.0))

    def scalar_reciprocal():
        assert np.array_equal(oi.row_scale(amax).numpy(), (amax * (1.0 / 127.0)).numpy())

    must_fail(scalar_reciprocal, "scale through a reciprocal is not the correctly rounded division")


def test_int_mm_is_the_exact_integer_product():
    g = torch.Generator().manual_seed(4)
    a = torch.randint(-127, 128, (9, 300), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (300, 7), generator=g, dtype=torch.int8)
    want = torch.tensor([[sum(int(a[i, t]) * int(b[t, j]) for t in range(300)) for j in range(7)] for i in range(9)], dtype=torch.int32)
    assert torch.equal(oi.int_mm(a, b), want)
    big = torch.full((2, 8192), 127, dtype=torch.int8)
    assert oi.int_mm(big, (-big).t())[0, 0].item() == -8192 * 127 * 127


@pytest.mark.parametrize("mode", oi.DGRAD)
def test_forward_and_dgrad_equal_the_fp64_model_on_the_grid(mode):
    q, scale, g = weight(128, 256)
    bias = torch.randn(128, generator=g) * 0.1
    x = on_grid(33, 256, g)
    y = oi.forward(x, q, scale, bias)
    torch.testing.assert_close(y.double(), model64(x, q, scale, bias), rtol=1e-5, atol=1e-5)
    dy = torch.randn(33, 128, generator=g)
    torch.testing.assert_close(oi.dgrad(dy, q, scale, mode).double(), dx64(dy, q, scale, mode), rtol=1e-3, atol=1e-3)
    if mode == "int8":
        wrong = oi.dgrad(dy, q, torch.ones_like(scale), mode) * scale.mean()
        must_fail(lambda: torch.testing.assert_close(wrong.double(), dx64(dy, q, scale, mode), rtol=1e-3, atol=1e-3),
                  "weight scales not moved onto dy's columns")


def test_forward_off_the_grid_and_broken_designs():
    q, scale, g = weight(128, 256, seed=1)
    bias = torch.randn(128, generator=g) * 0.1
    x = torch.randn(33, 256, generator=g)
    ref = model64(x, q, scale, bias)

    def close(y):
        torch.testing.assert_close(y.double(), ref, rtol=1e-3, atol=1e-3)

    close(oi.forward(x, q, scale, bias))
    xq, xs = oi.quantize_rows(x)
    unscaled = (xq.double() @ q.double().T) * scale.double() + bias.double()
    dense = x.double() @ (q.double() * scale.double()[:, None]).T + bias.double()
    swapped = (xq.double() @ q.double().T) * xs.double().flip(0)[:, None] * scale.double() + bias.double()
    for what, wrong in (("activation scale dropped", unscaled), ("activation not quantized", dense), ("row scales in the wrong order", swapped)):
        must_fail(lambda w=wrong: close(w), what)


def test_argument_errors():
    with pytest.raises(ValueError):
        oi.quantize_rows(torch.zeros(4))
    with pytest.raises(ValueError):
        oi.dgrad(torch.zeros(2, 4), torch.zeros(4, 8, dtype=torch.int8), torch.ones(4), "fp4")


@pytest.mark.parametrize("group", (16, 64))
def test_rotated_forward_equals_the_fp64_model_on_the_grid(group):
    """x chosen so that x R is exactly codes / 64 with a 127 per row (R is its own inverse and
    the integers keep every butterfly exact): the rotated forward must equal the fp64 model of
    'rotate, quantize, multiply' and differ from the unrotated one."""
    from oracle import hadamard as oh

    q, scale, g = weight(128, 256, seed=5)
    bias = torch.randn(128, generator=g) * 0.1
    codes = on_grid(33, 256, g)
    h = oh.matrix(group).double()
    x = (codes.double().reshape(-1, group) @ h).reshape(codes.shape).float()
    assert torch.equal((x.double().reshape(-1, group) @ h).reshape(codes.shape).float(), codes)
    y = oi.forward(x, q, scale, bias, group)
    torch.testing.assert_close(y.double(), model64(codes, q, scale, bias), rtol=1e-5, atol=1e-5)
    must_fail(lambda: torch.testing.assert_close(oi.forward(x, q, scale, bias).double(), model64(codes, q, scale, bias), rtol=1e-3, atol=1e-3), "no rotation")
    dy = torch.randn(33, 128, generator=g)
    want = (dx64(dy, q, scale, "int8").reshape(-1, group) @ h).reshape(33, 256)
    torch.testing.assert_close(oi.dgrad(dy, q, scale, "int8", group).double(), want, rtol=1e-3, atol=1e-3)
