"""Host side of the int8 compute linear without a GPU: the eager launchers against the oracle,
the op's autograd contract (only `q` and `scale` saved, bias gradient, leading dims), the
support check and the registry route. Mirrors reference
`tests/kernels/quant/test_int8_linear.py:84-148` on the CPU."""

import pytest
import torch

from kohakumosstrainer_amd.kernels import registry
from kohakumosstrainer_amd.kernels.int8 import formats as f8
from kohakumosstrainer_amd.kernels.int8 import op as int8_op
from oracle import int8 as oi


def problem(m, n, k, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.05
    scale = (w.abs().amax(dim=1).clamp_min(1e-12) / 127.0).float()
    q = torch.round(w / scale[:, None]).clamp(-127, 127).to(torch.int8)
    x = torch.randn(m, k, generator=g).to(dtype)
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    return x, q, scale, bias, dy


@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
def test_host_formats_equal_oracle(dtype):
    x, q, scale, bias, dy = problem(33, 64, 96, dtype)
    for col in (None, torch.rand(96) + 0.1):
        a, b = f8.quantize_rows(x, col)
        c, d = oi.quantize_rows(x, col)
        assert torch.equal(a, c) and torch.equal(b, d)
    assert torch.equal(f8.int_mm(a, q.t()), oi.int_mm(a, q.t()))
    cm = f8.col_major(q)
    assert torch.equal(cm, q) and cm.stride() == (1, q.shape[0])
    with pytest.raises(ValueError):
        f8.quantize_rows(x[0])


@pytest.mark.parametrize("mode", int8_op.DGRAD)
def test_eager_op_matches_oracle_and_autograd_contract(mode):
    x, q, scale, bias, dy = problem(17, 64, 128, torch.bfloat16, seed=1)
    op = registry.resolve("int8_linear", "cpu", torch.bfloat16, group=0, dgrad=mode)
    assert op.backend == "eager"
    xa = x.clone().requires_grad_(True)
    ba = bias.clone().requires_grad_(True)
    y = op(xa, q, scale, ba, 0, mode)
    assert torch.equal(y, oi.forward(x, q, scale, bias))
    node = y.grad_fn.next_functions[0][0]  # under the reshape of the leading dims
    saved = list(node.saved_tensors)
    assert len(saved) == 2 and saved[0].dtype == torch.int8 and saved[1].shape == (64,)
    y.backward(dy)
    assert torch.equal(xa.grad, oi.dgrad(dy, q, scale, mode))
    assert torch.equal(ba.grad, dy.float().sum(0).to(torch.bfloat16))
    y3 = op(x.reshape(1, 17, 128), q, scale, None, 0, mode)
    assert y3.shape == (1, 17, 64) and not y3.requires_grad
    assert torch.equal(y3[0], oi.forward(x, q, scale, None))


def test_support_check():
    registry.load_backends()
    assert registry.available("int8_linear", "cpu", torch.bfloat16, group=0, dgrad="int8")["eager"] is None
    assert registry.available("int8_linear", "cpu", torch.bfloat16, group=256, dgrad="int8")["eager"] is None
    assert "power of 4" in registry.available("int8_linear", "cpu", torch.bfloat16, group=8, dgrad="int8")["eager"]
    assert "not in" in registry.available("int8_linear", "cpu", torch.bfloat16, group=0, dgrad="fp4")["eager"]
    x, q, scale, bias, dy = problem(4, 8, 24)
    with pytest.raises(ValueError):
        int8_op.fwd_reference(x, q, scale, bias, 16)  # 24 % 16


@pytest.mark.parametrize("mode", int8_op.DGRAD)
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
def test_rotated_base_matches_oracle(mode, dtype):
    x, q, scale, bias, dy = problem(9, 32, 128, dtype, seed=2)
    op = registry.resolve("int8_linear", "cpu", dtype, group=64, dgrad=mode)
    xa = x.clone().requires_grad_(True)
    y = op(xa, q, scale, bias, 64, mode)
    assert torch.equal(y, oi.forward(x, q, scale, bias, 64))
    y.backward(dy)
    assert torch.equal(xa.grad, oi.dgrad(dy, q, scale, mode, 64))


def test_rotation_and_rotated_weight_only_on_the_host():
    from kohakumosstrainer_amd.kernels import hadamard
    from oracle import hadamard as oh
    from oracle import linear as ol

    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 2, 128, generator=g)
    for dt in (torch.float32, torch.bfloat16):
        xa = x.to(dt).detach().clone().requires_grad_(True)
        y = hadamard.group_hadamard(xa, 64)
        assert torch.equal(y, oh.rotate(x.to(dt), 64))
        y.backward(torch.ones_like(y))
        assert torch.equal(xa.grad, oh.rotate(torch.ones_like(y), 64))
    assert torch.equal(hadamard.hadamard_matrix(16), oh.matrix(16))
    with pytest.raises(ValueError):
        hadamard.group_hadamard(x, 48)
    xq, q, scale, bias, dy = problem(9, 32, 128, torch.bfloat16, seed=4)
    op = registry.resolve("quant_linear_rotated", "cpu", torch.bfloat16, fmt="int8", group=64)
    assert op.backend == "eager"
    xa = xq.clone().requires_grad_(True)
    y = op(xa, q, scale, bias, "int8", 64)
    assert torch.equal(y, ol.wo_forward(oh.rotate(xq, 64), q, scale, bias))
    y.backward(dy)
    assert torch.equal(xa.grad, oh.rotate(ol.wo_dgrad(dy, q, scale), 64))
