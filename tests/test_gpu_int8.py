"""int8 compute linear on the GPU through the C ABI and the registry: the HIP per-row quantizer
against the CPU oracle byte for byte, the op's forward and int8 input gradient against the
oracle bit for bit (the integer accumulation is exact and the epilogue rounds in the eager
path's order), the 16-bit input gradient by the weight-only tolerance. Mirrors reference
`tests/kernels/quant/test_int8_linear.py:163-260` (every backend against the eager reference and
fp64, both dgrad modes, bf16 and fp16, under torch.compile)."""

import pytest
import torch

from kohakumosstrainer_amd import native
from kohakumosstrainer_amd.kernels import registry, tuning
from oracle import int8 as oi
from oracle import stats as oracle_stats

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = (torch.bfloat16, torch.float16)


@pytest.fixture(autouse=True)
def untimed():
    tuning.set_mode("off")
    tuning.reset()
    yield
    tuning.set_mode("table")
    tuning.reset()


def activations(m, k, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) * torch.logspace(-3, 2, m)[:, None]
    if m > 2:
        x[1] = 0.0
        x[2, : min(k, 5)] = torch.tensor([127.0, 0.5, 1.5, -2.5, -127.0])[: min(k, 5)]
        x[2, min(k, 5):] = 0.0
    return x.to(dtype), g


def check_rows(x_cpu, col=None, view=lambda t: t):
    q, s = native.quant_rows_i8(view(x_cpu.cuda()), None if col is None else col.cuda())
    rq, rs = oi.quantize_rows(view(x_cpu), col)
    assert q.dtype == torch.int8 and s.dtype == torch.float32 and q.shape == rq.shape and q.is_contiguous()
    assert torch.equal(s.cpu().view(torch.int32), rs.view(torch.int32)), "scale bits"
    assert torch.equal(q.cpu(), rq), "codes"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k", [(300, 1024), (5, 7), (1, 1), (64, 200), (33, 4096), (9, 4104), (130, 8192)])
def test_quantizer_bytes_equal_oracle(dtype, m, k):
    x, g = activations(m, k, dtype, seed=m)
    col = torch.rand(k, generator=g) * 1e-2 + 1e-5
    check_rows(x)
    check_rows(x, col)
    check_rows(x, view=lambda t: t.t(), col=torch.rand(m, generator=g) + 0.1)
    if k >= 16:
        check_rows(x, view=lambda t: t[:, 8:], col=col[8:])
        check_rows(x, view=lambda t: t[:, 1 : k - 1])


def test_quantizer_half_even_known_answers_and_floor():
    x = torch.tensor([[127.0, 0.5, 1.5, -2.5, -127.0, 0.0, 0.0, 0.0], [0.0] * 8]).to(torch.bfloat16)
    q, s = native.quant_rows_i8(x.cuda())
    assert q.cpu()[0].tolist() == [127, 0, 2, -2, -127, 0, 0, 0] and q.cpu()[1].tolist() == [0] * 8
    assert s.cpu()[0].item() == 1.0 and s.cpu()[1].item() == oi.row_scale(torch.zeros(1)).item()


def test_quantizer_every_bf16_pattern_under_sampled_amax():
    g = torch.Generator().manual_seed(6)
    amax = torch.cat([torch.randint(1, 0x7F80, (120,), generator=g), torch.tensor([0, 1, 0x80, 0x7F7F])])
    pats = torch.arange(0x10000, dtype=torch.int32)
    keep = (pats & 0x7FFF)[None, :] <= amax[:, None].to(torch.int32)
    m = torch.where(keep, pats[None, :], torch.zeros((), dtype=torch.int32))
    x = (m - (m >= 0x8000).to(torch.int32) * 0x10000).to(torch.int16).view(torch.bfloat16)
    check_rows(x)


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_quantizer_vector_kernel_equals_the_dividing_kernel_on_every_pair(dtype):
    """Without column scales the vectorized kernel forms x / s from a rounded reciprocal and two
    fused corrections; the element-wise kernel (taken for a view that is not 16-byte aligned)
    divides. Every (amax, x) pair of finite 16-bit patterns with |x| <= amax must give the same
    byte and the same scale."""
    inf16 = 0x7F80 if dtype == torch.bfloat16 else 0x7C00
    pats = torch.arange(0x10000, dtype=torch.int32, device="cuda")
    chunk = 2048
    for a0 in range(0, inf16, chunk):
        amax = torch.arange(a0, min(a0 + chunk, inf16), device="cuda", dtype=torch.int32)
        keep = (pats & 0x7FFF)[None, :] <= amax[:, None]
        v = torch.where(keep, pats[None, :], torch.zeros((), dtype=torch.int32, device="cuda"))
        x = (v - (v >= 0x8000).to(torch.int32) * 0x10000).to(torch.int16).view(dtype)
        wide = torch.zeros(x.shape[0], x.shape[1] + 8, dtype=dtype, device="cuda")
        wide[:, 1:-7] = x
        q_fast, s_fast = native.quant_rows_i8(x)
        q_div, s_div = native.quant_rows_i8(wide[:, 1:-7])
        assert torch.equal(s_fast.view(torch.int32), s_div.view(torch.int32))
        assert torch.equal(q_fast, q_div), f"amax patterns {a0}..{a0 + chunk}"
        del x, wide, v, keep, q_fast, q_div


def test_quantizer_full_size():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(16384, 3072, generator=g)
    mask = torch.rand(16384, 3072, generator=g) < 1e-3
    x[mask] = (torch.randn(16384, 3072, generator=g) * 50)[mask]
    check_rows(x.to(torch.bfloat16))


def weight(n, k, g):
    w = torch.randn(n, k, generator=g) * 0.05
    scale = (w.abs().amax(dim=1).clamp_min(1e-12) / 127.0).float()
    return torch.round(w / scale[:, None]).clamp(-127, 127).to(torch.int8), scale


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(200, 256, 256), (513, 384, 1024), (5, 512, 768), (61, 2048, 4096)])
def test_int8_linear_forward_and_grads(dtype, m, n, k):
    g = torch.Generator().manual_seed(m)
    q, scale = weight(n, k, g)
    x = torch.randn(m, k, generator=g).to(dtype)
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    for mode in oi.DGRAD:
        op = registry.resolve("int8_linear", DEV, dtype, group=0, dgrad=mode)
        assert op.backend == "hip"
        xd = x.to(DEV).requires_grad_(True)
        bd = bias.to(DEV).requires_grad_(True)
        y = op(xd, q.to(DEV), scale.to(DEV), bd, 0, mode)
        y.backward(dy.to(DEV))
        assert torch.equal(y.detach().cpu(), oi.forward(x, q, scale, bias)), "forward bits"
        want_dx = oi.dgrad(dy, q, scale, mode)
        if mode == "int8":
            assert torch.equal(xd.grad.cpu(), want_dx), "int8 input gradient bits"
        else:
            exact = dy.double() @ (q.double() * scale.double()[:, None])
            oracle_stats.assert_no_regression(xd.grad.cpu(), want_dx, exact, name="16bit dgrad")
        assert torch.equal(bd.grad.cpu(), dy.float().sum(0).to(dtype))
    no_bias = registry.resolve("int8_linear", DEV, dtype, group=0, dgrad="int8")(x.to(DEV), q.to(DEV), scale.to(DEV), None, 0, "int8")
    assert torch.equal(no_bias.cpu(), oi.forward(x, q, scale, None)) and not no_bias.requires_grad


def test_int8_linear_leading_dims_compile_and_support():
    g = torch.Generator().manual_seed(2)
    q, scale = weight(256, 512, g)
    x = torch.randn(4, 32, 512, generator=g).to(torch.bfloat16)
    op = registry.resolve("int8_linear", DEV, torch.bfloat16, group=0, dgrad="int8")
    y = op(x.to(DEV), q.to(DEV), scale.to(DEV), None, 0, "int8")
    assert y.shape == (4, 32, 256)
    assert torch.equal(y.cpu().reshape(128, 256), oi.forward(x.reshape(128, 512), q, scale, None))
    compiled = torch.compile(lambda t: op(t, q.to(DEV), scale.to(DEV), None, 0, "int8"), fullgraph=True)
    assert torch.equal(compiled(x.to(DEV)), y)
    assert registry.available("int8_linear", DEV, torch.bfloat16, group=256, dgrad="int8")["hip"] is None
    assert "power of 4" in registry.available("int8_linear", DEV, torch.bfloat16, group=8, dgrad="int8")["hip"]
    assert "not in" in registry.available("int8_linear", DEV, torch.bfloat16, group=0, dgrad="fp4")["hip"]
    with pytest.raises(ValueError):
        op(x.to(DEV)[..., :320], q.to(DEV)[:, :320], scale.to(DEV), None, 0, "int8")  # K % 128


def test_quant_weight_module_runs_int8_compute():
    from kohakumosstrainer_amd.quant.weights import QuantWeight

    g = torch.Generator().manual_seed(8)
    w = torch.randn(384, 512, generator=g) * 0.05
    x = torch.randn(64, 512, generator=g).to(torch.bfloat16)
    from kohakumosstrainer_amd.quant.bind import rebind_quant, set_int8_compute

    base = QuantWeight.from_weight(w, "int8").to(DEV)
    assert set_int8_compute(base, "int8") == 1
    rebind_quant(base, DEV, torch.bfloat16)
    y = base.linear(x.to(DEV), None)
    assert torch.equal(y.cpu(), oi.forward(x, base.q.cpu(), base.scale.cpu(), None))
    with pytest.raises(ValueError):
        QuantWeight.from_weight(w, "fp8").__class__(base.q, base.scale, "fp8", int8_dgrad="int8")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("group", (64, 256))
def test_rotated_int8_linear(dtype, group):
    """A ConvRot base: x is rotated by the HIP butterfly kernel before the quantizer and dx after
    the GEMM. Against the oracle with the butterfly form of the rotation the result is equal bit
    for bit; against the reference's eager form (a 16-bit matmul with H, whose fp32 sums round
    in another order) and the fp64 model it is close."""
    from oracle import hadamard as oh

    m, n, k = 200, 384, 1024
    g = torch.Generator().manual_seed(group)
    q, scale = weight(n, k, g)
    x = torch.randn(m, k, generator=g).to(dtype)
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    for mode in oi.DGRAD:
        op = registry.resolve("int8_linear", DEV, dtype, group=group, dgrad=mode)
        assert op.backend == "hip"
        xd = x.to(DEV).requires_grad_(True)
        y = op(xd, q.to(DEV), scale.to(DEV), bias.to(DEV), group, mode)
        y.backward(dy.to(DEV))
        assert torch.equal(y.detach().cpu(), oi.forward(x, q, scale, bias, group, "butterflies"))
        eager = oi.forward(x, q, scale, bias, group)
        h = oh.matrix(group).double()
        xr = (x.double().reshape(-1, group) @ h).reshape(m, k)
        s64 = xr.abs().amax(1).clamp_min(1e-12) / 127.0
        exact = (torch.round(xr / s64[:, None]).clamp(-127, 127) @ q.double().T) * s64[:, None] * scale.double()[None, :] + bias.double()
        oracle_stats.assert_no_regression(y.detach().cpu(), eager, exact, name=f"rotated fwd g{group}")
        want_dx = oi.dgrad(dy, q, scale, mode, group, "butterflies")
        if mode == "int8":
            assert torch.equal(xd.grad.cpu(), want_dx)
        else:
            exact_dx = ((dy.double() @ (q.double() * scale.double()[:, None])).reshape(-1, group) @ h).reshape(m, k)
            oracle_stats.assert_no_regression(xd.grad.cpu(), oi.dgrad(dy, q, scale, mode, group), exact_dx, name="rotated 16bit dgrad")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("group", (4, 16, 64, 256, 1024))
def test_rotating_quantizer_equals_rotation_then_quantizer(dtype, group):
    """One kernel (rows rotated in LDS on their way to the quantizer) against the oracle's butterfly
    rotation followed by its row quantizer, byte for byte and scale bit for scale bit: whole and
    partial groups of four rows, a padded row stride, rows of the longest length the kernel holds, and
    the two-kernel route beyond it."""
    from oracle import hadamard as oh

    lib = native.load()
    for m, k in ((203, 1024), (4, 3072), (1, 4096), (64, 2048), (9, 8192)):
        if k % group:
            continue
        x, _ = activations(m, k, dtype, seed=group + m)
        want_q, want_s = oi.quantize_rows(oh.butterflies(x, group))
        q, s = native.quant_rows_i8_rotated(x.to(DEV), group)
        assert torch.equal(s.cpu().view(torch.int32), want_s.view(torch.int32)), (m, k, "scale bits")
        assert torch.equal(q.cpu(), want_q), (m, k, "codes")
        two_q, two_s = native.quant_rows_i8(native.group_hadamard(x.to(DEV), group))
        assert torch.equal(q, two_q) and torch.equal(s, two_s)
    # a view with a padded row stride goes through the one kernel too
    wide, _ = activations(37, 2048 + 64, dtype, seed=5)
    view = wide.to(DEV)[:, :2048]
    q, s = native.quant_rows_i8_rotated(view, group)
    want_q, want_s = oi.quantize_rows(oh.butterflies(wide[:, :2048].contiguous(), group))
    assert torch.equal(q.cpu(), want_q) and torch.equal(s.cpu().view(torch.int32), want_s.view(torch.int32))
    # what the kernel does not take is refused by the entry point (the wrapper routes around it)
    assert lib.km_quant_rows_i8_rotated(16, 4, 8192, 8192, native.KM_BF16, group, 16, 16, None) == native.KM_ERR_UNSUPPORTED
    assert lib.km_quant_rows_i8_rotated(16, 4, 1024, 1024, native.KM_BF16, 4, 16, 16, None) == native.KM_ERR_UNSUPPORTED
    assert lib.km_quant_rows_i8_rotated(None, 4, 1000, 1000, native.KM_BF16, 16, None, None, None) == native.KM_ERR_ARG


def test_int8_input_gradient_keeps_one_transposed_copy_per_code_tensor():
    from kohakumosstrainer_amd.kernels.backends.hip import int8 as hip_int8

    g = torch.Generator().manual_seed(11)
    q, scale = weight(256, 384, g)
    qd, sd = q.to(DEV), scale.to(DEV)
    dy = torch.randn(40, 256, generator=g).to(torch.bfloat16)
    first = hip_int8.dgrad(dy.to(DEV), qd, sd, 0, "int8")
    kept = hip_int8.transposed_codes(qd)
    assert kept.shape == (384, 256) and torch.equal(kept, qd.t())
    again = hip_int8.dgrad(dy.to(DEV), qd, sd, 0, "int8")
    assert hip_int8.transposed_codes(qd) is kept, "the copy is made once per code tensor"
    assert torch.equal(first, again) and torch.equal(first.cpu(), oi.dgrad(dy, q, scale, "int8"))
    # codes rewritten in place: the copy is made again
    qd.copy_(torch.roll(qd, 1, 0))
    rolled = hip_int8.dgrad(dy.to(DEV), qd, sd, 0, "int8")
    assert torch.equal(rolled.cpu(), oi.dgrad(dy, torch.roll(q, 1, 0), scale, "int8"))
    key = id(qd)
    del qd, kept
    import gc

    gc.collect()
    assert key not in hip_int8._TRANSPOSED, "the copy goes with its code tensor"


def test_rotated_weight_only_linear_and_module():
    from kohakumosstrainer_amd.quant.weights import QuantWeight
    from oracle import hadamard as oh
    from oracle import linear as ol

    g = torch.Generator().manual_seed(12)
    m, n, k, group = 130, 256, 768, 256
    q, scale = weight(n, k, g)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
    dy = torch.randn(m, n, generator=g).to(torch.bfloat16)
    op = registry.resolve("quant_linear_rotated", DEV, torch.bfloat16, fmt="int8", group=group)
    assert op.backend == "hip"
    xd = x.to(DEV).requires_grad_(True)
    y = op(xd, q.to(DEV), scale.to(DEV), bias.to(DEV), "int8", group)
    y.backward(dy.to(DEV))
    h = oh.matrix(group).double()
    w64 = q.double() * scale.double()[:, None]
    exact = (x.double().reshape(-1, group) @ h).reshape(m, k) @ w64.T + bias.double()
    eager = ol.wo_forward(oh.rotate(x, group), q, scale, bias)
    oracle_stats.assert_no_regression(y.detach().cpu(), eager, exact, name="rotated weight-only fwd")
    exact_dx = ((dy.double() @ w64).reshape(-1, group) @ h).reshape(m, k)
    oracle_stats.assert_no_regression(xd.grad.cpu(), oh.rotate(ol.wo_dgrad(dy, q, scale), group), exact_dx, name="rotated weight-only dgrad")
    base = QuantWeight(q, scale, "int8", rotation=group).to(DEV)
    base.bind(torch.bfloat16)
    assert torch.equal(base.linear(x.to(DEV), bias.to(DEV)), y.detach())
    torch.testing.assert_close(base.weight(torch.float32).cpu().double(), (w64.reshape(-1, group) @ h).reshape(n, k), rtol=1e-5, atol=1e-6)
