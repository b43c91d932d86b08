"""HIP int8 GEMM (int32 accumulation, fp32 row / column scales, bias) through the C ABI against
the exact integer product: the accumulation is exact and the epilogue rounds in the reference's
order, so outputs are compared bit for bit (reference `tests/kernels/quant/test_int8_linear.py`
compares its Triton GEMM with the eager path by tolerance; here equality holds)."""

import pytest
import torch

from kohakumosstrainer_amd import native

pytestmark = pytest.mark.gpu


def exact_epilogue(a, sa, b, sb, bias, dtype):
    """int8 codes -> exact integer product (fp64 holds it: |acc| <= K * 127^2 < 2^53), then the
    fp32 roundings in order: (acc * sa) * sb + bias, once to dtype."""
    acc = (a.double() @ b.double().T).to(torch.float32)  # exact below 2^24, rounded as int32 -> fp32 above
    y = acc * sa[:, None]
    if sb is not None:
        y = y * sb[None, :]
    if bias is not None:
        y = y + bias.float()
    return y.to(dtype)


def problem(m, n, k, seed, spread=127):
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-spread, spread + 1, (m, k), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    sa = torch.rand(m, generator=g) * 0.02 + 1e-3
    sb = torch.rand(n, generator=g) * 1e-3 + 1e-5
    return a, b, sa, sb, g


def n_configs():
    return len(native.configs(native.KERNEL_GEMM_FP8))


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("m,n,k", [(200, 384, 256), (1000, 512, 768), (1, 128, 128), (513, 200, 1152), (61, 136, 4096), (300, 256, 384)])
def test_i8_gemm_every_config_is_exact(dtype, m, n, k):
    a, b, sa, sb, g = problem(m, n, k, seed=m + n)
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    want = exact_epilogue(a, sa, b, sb, bias, dtype)
    want_plain = exact_epilogue(a, sa, b, None, None, dtype)
    for cfg in range(n_configs()):
        y = native.gemm_i8_rows(a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), bias.cuda(), dtype, cfg)
        assert torch.equal(y.cpu(), want), f"cfg{cfg} {m}x{n}x{k}"
        y = native.gemm_i8_rows(a.cuda(), sa.cuda(), b.cuda(), None, None, dtype, cfg)
        assert torch.equal(y.cpu(), want_plain), f"cfg{cfg} {m}x{n}x{k} no column scale"


def test_i8_gemm_one_hot_operands_pin_the_k_order():
    """A single +-1 per row of `a` picks one column of b^T: any K permutation that differs
    between the two operands, or a dropped half of a 128-byte step, shows."""
    k, n = 640, 128
    g = torch.Generator().manual_seed(9)
    b = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    a = torch.zeros(k, k, dtype=torch.int8)
    a[torch.arange(k), torch.arange(k)] = 1
    ones = torch.ones(k)
    y = native.gemm_i8_rows(a.cuda(), ones.cuda(), b.cuda(), None, None, torch.float16, 0)
    assert torch.equal(y.cpu(), b.t().to(torch.float16))


def test_i8_gemm_extreme_codes_do_not_overflow():
    """All codes -127 / +127 over K = 8192: |acc| = 8192 * 16129 = 1.3e8 < 2^31."""
    m, n, k = 128, 128, 8192
    a = torch.full((m, k), 127, dtype=torch.int8)
    b = torch.full((n, k), -127, dtype=torch.int8)
    b[::2] = 127
    sa = torch.full((m,), 2.0**-20)
    y = native.gemm_i8_rows(a.cuda(), sa.cuda(), b.cuda(), None, None, torch.bfloat16, 0)
    assert torch.equal(y.cpu(), exact_epilogue(a, sa, b, None, None, torch.bfloat16))


def test_i8_gemm_argument_errors():
    a = torch.zeros(64, 192, dtype=torch.int8, device="cuda")
    s = torch.ones(64, device="cuda")
    with pytest.raises(native.KernelError):
        native.gemm_i8_rows(a, s, a, s, None, torch.bfloat16, 0)  # K % 128
    a = torch.zeros(64, 256, dtype=torch.int8, device="cuda")
    with pytest.raises(native.KernelError):
        native.gemm_i8_rows(a, s, a, s, None, torch.bfloat16, 99)
    with pytest.raises(ValueError):
        native.gemm_i8_rows(a, s[:3], a, s, None, torch.bfloat16, 0)
    with pytest.raises(ValueError):
        native.gemm_i8_rows(a.float(), s, a, s, None, torch.bfloat16, 0)
    assert native.gemm_i8_rows(a[:0], s[:0], a, s, None, torch.bfloat16, 0).shape == (0, 64)


def test_i8_gemm_full_size_slice():
    """M=16384, K=3072, N=9216: a 128-row slice and the last rows against the exact product."""
    m, n, k = 16384, 9216, 3072
    g = torch.Generator().manual_seed(1)
    a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    sa = torch.rand(m, generator=g) * 0.02 + 1e-3
    sb = torch.rand(n, generator=g) * 1e-3 + 1e-5
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
    y = native.gemm_i8_rows(a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), bias.cuda(), torch.bfloat16, 0).cpu()
    for rows in (slice(4096, 4224), slice(m - 64, m)):
        assert torch.equal(y[rows], exact_epilogue(a[rows], sa[rows], b, sb, bias, torch.bfloat16))
