"""Operands at the edge of the 32-bit offsets the GEMM kernels compute with: just below the cap
the result is right (rows and columns whose byte offsets sit next to 2^31 / 2^30 included), at the
cap the entry point refuses before it touches a pointer. The kernels address a tile's operand rows
through a buffer descriptor based at the tile with 32-bit per-lane offsets; `km_gemm_*` caps
M*K and N*K at 2^31 - 1 bytes, the weight-only entry points cap N*K at 2^30 - 1 codes."""

import ctypes

import pytest
import torch

from kohakumosstrainer_amd import native
from oracle import formats


def finite_codes(shape, gen_seed, device):
    """Uniform e4m3 codes without the two NaN patterns, made on the device."""
    g = torch.Generator(device=device).manual_seed(gen_seed)
    mag = torch.randint(0, 0x7F, shape, generator=g, device=device, dtype=torch.uint8)
    sign = torch.randint(0, 2, shape, generator=g, device=device, dtype=torch.uint8) << 7
    return (mag | sign).view(torch.float8_e4m3fn)


@pytest.mark.gpu
def test_mx_gemm_with_an_activation_just_below_two_gib():
    k, n = 8192, 128
    m = (2**31 - 1) // k  # 262143 rows: M * K = 2^31 - 8192 bytes
    assert m * k <= 2**31 - 1 < (m + 1) * k
    dev = torch.device("cuda")
    a = finite_codes((m, k), 0, dev)
    g = torch.Generator(device=dev).manual_seed(1)
    a_scale = torch.randint(120, 128, (m, k // 32), generator=g, device=dev, dtype=torch.uint8)
    b = finite_codes((n, k), 2, dev)
    b_scale = torch.randint(120, 128, (n, k // 32), generator=g, device=dev, dtype=torch.uint8)
    bias = torch.randn(n, generator=g, device=dev).to(torch.bfloat16)
    for cfg in (0, 3):
        c = native.gemm_mx(a, a_scale, b, b_scale, bias, torch.bfloat16, cfg)
        assert c.shape == (m, n)
        for rows in (slice(0, 64), slice(m // 2 - 31, m // 2 + 33), slice(m - 300, m)):
            a64 = formats.dequantize(a[rows].cpu(), a_scale[rows].cpu(), "mx", torch.float64)
            b64 = formats.dequantize(b.cpu(), b_scale.cpu(), "mx", torch.float64)
            want = a64 @ b64.T + bias.cpu().double()
            got = c[rows].cpu().double()
            rel = ((got - want).norm() / want.norm()).item()
            assert rel <= 2e-3, f"cfg{cfg} rows {rows}: rel-L2 {rel:.3e}"


@pytest.mark.gpu
def test_weight_only_gemms_with_codes_just_below_one_gib():
    n, k, m = 131072, 8184, 64  # N * K = 2^30 - 1048576 codes; K % 8 == 0 keeps the tiled kernels
    assert n * k <= 2**30 - 1 < n * (k + 8)
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(3)
    q = torch.randint(-127, 128, (n, k), generator=g, device=dev, dtype=torch.int8)
    scale = torch.rand(n, generator=g, device=dev) * 1e-3 + 1e-4
    x = torch.randn(m, k, generator=g, device=dev).to(torch.bfloat16)
    dy = (torch.randn(m, n, generator=g, device=dev) * 0.1).to(torch.bfloat16)
    y = native.wo_gemm_fwd(x, q, scale, None, 0)
    for cols in (slice(0, 256), slice(n - 300, n)):
        want = (x.double() @ q[cols].double().T) * scale[cols].double()
        rel = ((y[:, cols].double() - want).norm() / want.norm()).item()
        assert rel <= 2e-3, f"forward columns {cols}: rel-L2 {rel:.3e}"
    # the input gradient reads q as stored: its row offsets n * K run up to the cap
    want = torch.zeros(m, k, device=dev, dtype=torch.float64)
    for lo in range(0, n, 8192):
        w = (q[lo : lo + 8192].float() * scale[lo : lo + 8192, None]).to(torch.bfloat16)
        want += dy[:, lo : lo + 8192].double() @ w.double()
    for cfg in (0, 3):
        dx = native.wo_gemm_dgrad(dy, q, scale, cfg)
        rel = ((dx.double() - want).norm() / want.norm()).item()
        assert rel <= 4e-3, f"dgrad cfg{cfg}: rel-L2 {rel:.3e}"
    # a one-hot gradient row reads back single rows of the rounded weight, the last one included
    probe = torch.zeros(8, n, device=dev, dtype=torch.bfloat16)
    picks = [0, 1, n // 2, n - 8191, n - 256, n - 17, n - 2, n - 1]
    for i, r in enumerate(picks):
        probe[i, r] = 1.0
    back = native.wo_gemm_dgrad(probe, q, scale, 0)
    rows = torch.tensor(picks, device=dev)
    assert torch.equal(back, (q[rows].float() * scale[rows, None]).to(torch.bfloat16))


@pytest.mark.gpu
def test_input_gradient_over_few_very_long_rows_of_codes():
    """Eight rows of 2^26 + 256 codes: 32 rows of such a q would pass 2^31 bytes, the stride by
    which the tiled kernels step through q, so the entry point must take another path. One-hot
    gradient rows read the rounded weight back, every element of every row."""
    n, k = 8, 2**26 + 256
    assert n * k <= 2**30 - 1 and 32 * k > 2**31 - 1
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(4)
    q = torch.randint(-127, 128, (n, k), generator=g, device=dev, dtype=torch.int8)
    scale = torch.rand(n, generator=g, device=dev) * 1e-3 + 1e-4
    probe = torch.eye(n, device=dev, dtype=torch.bfloat16)
    for cfg in (0, 2):
        back = native.wo_gemm_dgrad(probe, q, scale, cfg)
        for r in range(n):
            assert torch.equal(back[r], (q[r].float() * scale[r]).to(torch.bfloat16)), f"cfg{cfg} row {r}"
        del back


@pytest.mark.gpu
def test_input_gradient_with_a_contraction_too_long_for_tile_offsets():
    """dy[M, N] with N = 2^22: 256 rows of it are 2^31 bytes, one more than a tile's 32-bit offsets
    reach, so the entry point must not hand this shape to the tiled kernels. One-hot gradient rows
    (the last rows of what would be a 256-row tile and the rows after it included) read single
    rows of the rounded weight back exactly."""
    n, k, m = 2**22, 8, 260
    assert n > (2**31 - 1) // 512
    dev = torch.device("cuda")
    g = torch.Generator(device=dev).manual_seed(5)
    q = torch.randint(-127, 128, (n, k), generator=g, device=dev, dtype=torch.int8)
    scale = torch.rand(n, generator=g, device=dev) * 1e-3 + 1e-4
    dy = torch.zeros(m, n, device=dev, dtype=torch.bfloat16)
    picks = {0: 0, 1: n - 1, 127: n // 2 + 3, 254: 17, 255: n - 1, 256: n - 9, 259: n - 2}
    for r, c in picks.items():
        dy[r, c] = 1.0
    dx = native.wo_gemm_dgrad(dy, q, scale, 0)
    want = torch.zeros(m, k, device=dev, dtype=torch.bfloat16)
    for r, c in picks.items():
        want[r] = (q[c].float() * scale[c]).to(torch.bfloat16)
    assert torch.equal(dx, want)
    ws = native.wo_gemm_dgrad_workspace(dy, q, scale, 0)
    assert torch.equal(ws, want)


def _rc(fn, *args):
    rc = fn(*args)
    return rc, native.load().km_last_error().decode()


def test_operands_at_the_cap_are_refused_before_any_pointer_is_read():
    """No GPU needed: the size checks come first and the pointers are null."""
    lib = native.load()
    k = 8192
    m_over = (2**31 - 1) // k + 1
    null = None
    rc, why = _rc(lib.km_gemm_mx, null, null, null, null, null, null, m_over, 128, k, native.KM_BF16, native.SCALES_ROWMAJOR, 0, null)
    assert rc == native.KM_ERR_ARG and "too large" in why
    rc, why = _rc(lib.km_gemm_mx, null, null, null, null, null, null, 128, m_over, k, native.KM_BF16, native.SCALES_ROWMAJOR, 0, null)
    assert rc == native.KM_ERR_ARG and "too large" in why
    n, kk = 131072, 8192  # N * K = 2^30: one past the cap
    rc, why = _rc(lib.km_wo_gemm_fwd, null, null, null, null, null, 64, n, kk, native.KM_Q_INT8, native.KM_BF16, 0, null)
    assert rc == native.KM_ERR_ARG and "too large" in why
    rc, why = _rc(lib.km_wo_gemm_dgrad_w16, null, null, null, native.WSCALE_ROWS, 1, null, 64, n, kk, native.KM_Q_INT8, native.KM_BF16, 0, null)
    assert rc == native.KM_ERR_ARG and "too large" in why
    rc, why = _rc(lib.km_wo_gemm_dgrad, null, null, null, null, null, 64, n, kk, native.KM_Q_INT8, native.KM_BF16, 0, null)
    assert rc == native.KM_ERR_ARG and "too large" in why
