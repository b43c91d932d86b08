"""Pins of the rotation oracle (`oracle/hadamard.py`) without a GPU: an independent fp64
torch.kron construction, the algebra of H (symmetric, involutory, +-2^-j), the sign rule, exact
equality on integer inputs and must-fail variants (reference `tests/_util/hadamard_ref.py`,
`tests/kernels/quant/test_hadamard.py`)."""

import pytest
import torch

from oracle import hadamard as oh


def must_fail(check, what):
    try:
        check()
    except AssertionError:
        return
    raise AssertionError(f"check passed on the broken variant: {what}")


def h64(group, seed=oh.H4, normalise=True):
    base = torch.tensor(seed, dtype=torch.float64)
    h = base
    while h.shape[0] < group:
        h = torch.kron(h, base)
    return h / group**0.5 if normalise else h


def rot64(x, group, **kw):
    return (x.double().reshape(-1, group) @ h64(group, **kw)).reshape(x.shape)


@pytest.mark.parametrize("group", oh.GROUPS)
def test_matrix_algebra_and_sign_rule(group):
    h = oh.matrix(group).double()
    j = oh.stages(group)
    assert torch.equal(h, h64(group))
    assert torch.equal(h, h.T) and torch.equal(h @ h, torch.eye(group, dtype=torch.float64))
    assert torch.equal(h.abs(), torch.full_like(h, 2.0**-j))
    i = torch.arange(group)[:, None]
    k = torch.arange(group)[None, :]
    flips = sum(((i // 4**d) % 4 + (k // 4**d) % 4 == 3).int() for d in range(j))
    assert torch.equal(torch.sign(h), (1 - 2 * (flips % 2)).double())


@pytest.mark.parametrize("group", oh.GROUPS)
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16, torch.float16))
def test_exact_on_integer_inputs(group, dtype):
    """Small integers: every partial sum is an integer below 2^24 and the scaled result has few
    bits, so butterflies, matmul form and the fp64 construction agree exactly."""
    g = torch.Generator().manual_seed(group)
    x = (torch.randint(-3, 4, (6, 2 * group), generator=g).float() * group**0.5 / 2 ** oh.stages(group)).to(dtype)
    want = rot64(x, group)
    got = oh.butterflies(x, group)
    if dtype == torch.float32:
        assert torch.equal(got.double(), want)
    else:
        assert torch.equal(got, want.to(dtype))
    assert torch.equal(oh.rotate(x, group), got)
    assert torch.equal(oh.butterflies(got, group), x)  # its own inverse

    def transposed_digits():
        v = x.float().reshape(-1, group)
        j = oh.stages(group)
        idx = torch.arange(group)
        rev = sum(((idx // 4**d) % 4) * 4 ** (j - 1 - d) for d in range(j))
        assert torch.equal((oh.butterflies(v[:, rev], group)).double(), rot64(v, group).double())

    if group > 4:
        must_fail(transposed_digits, "digits in the wrong order")
    must_fail(lambda: torch.testing.assert_close(got.double(), rot64(x, group, seed=((1, 1), (1, -1)))), "Sylvester seed")
    must_fail(lambda: torch.testing.assert_close(got.double(), rot64(x, group, normalise=False)), "missing 1/sqrt(g)")


@pytest.mark.parametrize("group", (16, 256))
def test_close_on_random_inputs_and_argument_errors(group):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(9, 3 * group, generator=g)
    torch.testing.assert_close(oh.butterflies(x, group).double(), rot64(x, group), rtol=1e-5, atol=1e-5)
    xb = x.to(torch.bfloat16)
    torch.testing.assert_close(oh.butterflies(xb, group).double(), rot64(xb, group), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(oh.rotate(xb, group).double(), rot64(xb, group), rtol=1e-2, atol=1e-2)
    with pytest.raises(ValueError):
        oh.stages(8)
    with pytest.raises(ValueError):
        oh.butterflies(x[:, : group + 4], group)
