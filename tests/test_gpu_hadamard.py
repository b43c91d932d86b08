"""HIP group Hadamard rotation through the C ABI against the oracle's fp32 butterflies, bit for
bit (same operations in the same order), and against the fp64 Kronecker construction and the
reference's 16-bit matmul form by tolerance (reference `tests/kernels/quant/test_hadamard.py`)."""

import pytest
import torch

from kohakumosstrainer_amd import native
from oracle import hadamard as oh

pytestmark = pytest.mark.gpu
DTYPES = (torch.bfloat16, torch.float16)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("group", oh.GROUPS)
@pytest.mark.parametrize("rows", (1, 7, 64, 300))
def test_rotation_bits_equal_butterflies(dtype, group, rows):
    g = torch.Generator().manual_seed(group + rows)
    k = group * (3 if group >= 256 else 5)
    x = (torch.randn(rows, k, generator=g) * torch.logspace(-2, 2, rows)[:, None]).to(dtype)
    y = native.group_hadamard(x.cuda(), group).cpu()
    assert y.dtype == dtype and y.shape == x.shape
    assert torch.equal(y, oh.butterflies(x, group))
    h = oh.matrix(group).double()
    want = (x.double().reshape(-1, group) @ h).reshape(x.shape)
    torch.testing.assert_close(y.double(), want, rtol=2e-2, atol=1e-2 * x.double().abs().max().item())
    eager = oh.rotate(x, group)
    assert (y != eager).float().mean().item() < 0.02, "the matmul form differs in rare last-place roundings only"


def test_rotation_is_its_own_inverse_and_keeps_the_norm():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(512, 3072, generator=g).to(torch.bfloat16)
    y = native.group_hadamard(x.cuda(), 256)
    back = native.group_hadamard(y, 256).cpu()
    assert (back.float() - x.float()).norm() / x.float().norm() < 1e-2
    assert abs(y.float().norm().item() / x.float().norm().item() - 1) < 1e-3


def test_rotation_full_size_and_argument_errors():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(16384, 3072, generator=g).to(torch.bfloat16)
    y = native.group_hadamard(x.cuda(), 256).cpu()
    assert torch.equal(y[5000:5256], oh.butterflies(x[5000:5256], 256)) and torch.equal(y[-3:], oh.butterflies(x[-3:], 256))
    xs = torch.zeros(4, 96, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(native.KernelError):
        native.group_hadamard(xs, 8)
    with pytest.raises(native.KernelError):
        native.group_hadamard(xs, 64)  # 96 % 64
    with pytest.raises(ValueError):
        native.group_hadamard(xs.float(), 16)
    assert native.group_hadamard(xs[:0], 16).shape == (0, 96)
