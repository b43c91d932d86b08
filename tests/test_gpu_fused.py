"""The one-launch MXFP8 linear for short M (`native.gemm_mx_fused`, the counterpart of the
reference's Triton `fused_mx_mm`, `backends/triton/fp8/fused.py:98-120`): it quantizes x inside the
GEMM. Checked against the fp64 product of the oracle's quantized operands with the reference's
pass rule (stated tolerance ||y - ref|| / ||ref|| <= 2e-3 for bf16, 4e-4 for fp16), against the
two-launch path (quantizer kernel + GEMM), and bit for bit where every partial sum is exact."""

import pytest
import torch

from kohakumosstrainer_amd import native
from kohakumosstrainer_amd.kernels import registry
from oracle import formats, linear
from oracle.stats import assert_no_regression, rel_l2

pytestmark = pytest.mark.gpu
REL_L2 = {torch.bfloat16: 2e-3, torch.float16: 4e-4}


def operands(m, n, k, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) * torch.logspace(-2, 2, m)[:, None]
    x[:, : k // 2] *= torch.logspace(-1, 1, k // 2)[None, :]
    if m > 2:
        x[1] = 0.0
    w = torch.randn(n, k, generator=g) * 0.05
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    return x.to(dtype), w, bias


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("m,n,k", [(1, 32, 128), (5, 96, 384), (16, 256, 1024), (17, 64, 640), (32, 192, 384), (20, 96, 256), (33, 128, 512), (48, 160, 256), (48, 192, 640), (64, 256, 3072), (100, 96, 896), (100, 128, 384)])
def test_fused_mx_against_fp64_and_the_two_launch_path(dtype, m, n, k):
    x, w, bias = operands(m, n, k, dtype, seed=m + n)
    xq, xs = formats.quantize(x, "mx")
    wq, ws = formats.quantize(w, "mx", "weight")
    truth = linear.exact64(xq, xs, "mx") @ linear.exact64(wq, ws, "mx").T + bias.double()
    eager = linear.fp8_forward(x, wq, ws, None, bias, "mx")
    wsp = native.pack_scales(ws.cuda())
    y = native.gemm_mx_fused(x.cuda(), wq.cuda(), wsp, bias.cuda())
    assert y.shape == (m, n) and y.dtype == dtype
    assert_no_regression(y.cpu(), eager, truth, f"fused mx {m}x{n}x{k}")
    assert rel_l2(y.cpu(), truth) <= REL_L2[dtype]
    gq, _, gsp = native.quant_mx(x.cuda(), natural=False, packed=True)
    two = native.gemm_mx(gq, gsp, wq.cuda(), wsp, bias.cuda(), dtype, 4, packed=True)
    assert rel_l2(y.cpu(), two.double().cpu()) <= 2 * REL_L2[dtype]
    y0 = native.gemm_mx_fused(x.cuda(), wq.cuda(), wsp, None)
    assert rel_l2(y0.cpu(), truth - bias.double()) <= REL_L2[dtype]
    # rows of x not densely packed
    wide = torch.zeros(m, k + 64, dtype=dtype, device="cuda")
    wide[:, :k] = x.cuda()
    assert torch.equal(native.gemm_mx_fused(wide[:, :k], wq.cuda(), wsp, bias.cuda()), y)


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_fused_mx_equals_the_two_launch_path_where_sums_are_exact(dtype):
    """Small integers in x, small-integer codes with unit scales in W: every product and partial
    sum is an integer below 2^24, so the order of the K split cannot matter and the fused kernel
    must give the bytes of quantizer + GEMM. A wrong exponent byte, a wrong lane pairing of the
    32-column blocks or a misplaced K half would change them."""
    exact_case_mx(dtype, 40, 96, 1024)
    exact_case_mx(dtype, 30, 128, 512)    # two row tiles, 64-column workgroups


def exact_case_mx(dtype, m, n, k):
    g = torch.Generator().manual_seed(3)
    x = torch.randint(-6, 7, (m, k), generator=g).float()
    x[:, ::64] *= 32                                   # blocks of one row with different exponents
    x[3] = 0
    x[5, 100:132] = 0
    w = torch.randint(-8, 9, (n, k), generator=g).float()
    wq = w.to(torch.float8_e4m3fn)
    ws = torch.full((n, k // 32), 127, dtype=torch.uint8)
    ws[:, 3] = 129
    wsp = native.pack_scales(ws.cuda())
    xd = x.to(dtype).cuda()
    gq, gs, gsp = native.quant_mx(xd, packed=True)
    two = native.gemm_mx(gq, gsp, wq.cuda(), wsp, None, dtype, 4, packed=True)
    fused = native.gemm_mx_fused(xd, wq.cuda(), wsp, None)
    assert torch.equal(fused, two)
    truth = linear.exact64(gq.cpu(), gs.cpu(), "mx") @ linear.exact64(wq, ws, "mx").T
    assert torch.equal(fused.double().cpu(), truth.to(dtype).double())


def test_fused_mx_nan_and_inf_inputs_follow_the_quantizer():
    m, n, k = 16, 64, 256
    x, w, _ = operands(m, n, k, torch.bfloat16, seed=9)
    x[2, 7] = float("nan")
    x[4, 40] = float("inf")
    wq, ws = formats.quantize(w, "mx", "weight")
    wsp = native.pack_scales(ws.cuda())
    fused = native.gemm_mx_fused(x.cuda(), wq.cuda(), wsp, None)
    gq, _, gsp = native.quant_mx(x.cuda(), natural=False, packed=True)
    two = native.gemm_mx(gq, gsp, wq.cuda(), wsp, None, torch.bfloat16, 4, packed=True)
    assert torch.equal(torch.isnan(fused), torch.isnan(two))
    keep = ~torch.isnan(two)
    assert rel_l2(fused[keep].double().cpu(), two[keep].double().cpu()) <= 4e-3


def test_fused_mx_argument_errors_and_planner_candidate():
    x = torch.zeros(4, 256, device="cuda", dtype=torch.bfloat16)
    wq = torch.zeros(48, 256, device="cuda").to(torch.float8_e4m3fn)
    with pytest.raises(ValueError):
        native.gemm_mx_fused(x, wq, torch.zeros(native.packed_scale_bytes(48, 256), dtype=torch.uint8, device="cuda"), None)  # N % 32
    wq = torch.zeros(64, 256, device="cuda").to(torch.float8_e4m3fn)
    with pytest.raises(ValueError):
        native.gemm_mx_fused(x, wq, torch.zeros(7, dtype=torch.uint8, device="cuda"), None)
    y = native.gemm_mx_fused(x[:0], wq, torch.zeros(native.packed_scale_bytes(64, 256), dtype=torch.uint8, device="cuda"), None)
    assert y.shape == (0, 64)
    from kohakumosstrainer_amd.kernels.backends.hip import fp8_linear

    registry.load_backends()
    assert fp8_linear.candidates("mx", 16, 256, 256)[0]["gemm"] == "fused"
    assert fp8_linear.candidates("mx", 32, 256, 256)[-1]["gemm"] == "fused"
    assert not any(c["gemm"] == "fused" for c in fp8_linear.candidates("mx", 4096, 256, 256))
    assert not any(c["gemm"] == "fused" for c in fp8_linear.candidates("mx", 16, 48, 256))
    assert fp8_linear.candidates("row", 16, 256, 256)[-1]["gemm"] == "fused"
    assert not any(c["gemm"] == "fused" for c in fp8_linear.candidates("row", 32, 256, 256))
    assert fp8_linear.candidates("block", 16, 256, 256)[0]["gemm"] == "fused"
    assert not any(c["gemm"] == "fused" for c in fp8_linear.candidates("tensor", 16, 256, 256))


# ---- per-row recipe ---------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("m,n,k", [(1, 32, 128), (5, 96, 384), (16, 256, 1024), (17, 64, 640), (32, 192, 384), (20, 96, 256), (33, 128, 512), (48, 160, 256), (48, 192, 640), (64, 256, 3072), (100, 96, 896), (100, 128, 384)])
def test_fused_row_against_fp64_and_the_two_launch_path(dtype, m, n, k):
    x, w, bias = operands(m, n, k, dtype, seed=m + n + 1)
    xq, xs = formats.quantize(x, "row")
    wq, ws = formats.quantize(w, "row", "weight")
    truth = linear.exact64(xq, xs, "row") @ linear.exact64(wq, ws, "row").T + bias.double()
    eager = linear.fp8_forward(x, wq, ws, None, bias, "row")
    y = native.gemm_fp8_rows_fused(x.cuda(), wq.cuda(), ws.cuda(), bias.cuda())
    assert y.shape == (m, n) and y.dtype == dtype
    assert_no_regression(y.cpu(), eager, truth, f"fused row {m}x{n}x{k}")
    assert rel_l2(y.cpu(), truth) <= REL_L2[dtype]
    gq, gs = native.quant_rows(x.cuda())
    two = native.gemm_fp8_rows(gq, gs, wq.cuda(), ws.cuda(), bias.cuda(), dtype, 4)
    assert rel_l2(y.cpu(), two.double().cpu()) <= 2 * REL_L2[dtype]
    y0 = native.gemm_fp8_rows_fused(x.cuda(), wq.cuda(), ws.cuda(), None)
    assert rel_l2(y0.cpu(), truth - bias.double()) <= REL_L2[dtype]
    wide = torch.zeros(m, k + 64, dtype=dtype, device="cuda")
    wide[:, :k] = x.cuda()
    assert torch.equal(native.gemm_fp8_rows_fused(wide[:, :k], wq.cuda(), ws.cuda(), bias.cuda()), y)


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_fused_row_equals_the_two_launch_path_where_sums_are_exact(dtype):
    """Rows whose abs-max is 448 * 2^e have the scale 2^e exactly; with small-integer multiples of
    it in x and small-integer codes in W every partial sum is exact, so the fused kernel must give
    the bytes of quantizer + GEMM whatever the K split. The row maximum sits in a different K step
    (wavefront) for every row: a prologue that missed a wavefront's share would change the scale."""
    exact_case_row(dtype, 40, 96, 1024)
    exact_case_row(dtype, 30, 128, 512)   # two row tiles, 64-column workgroups


def exact_case_row(dtype, m, n, k):
    g = torch.Generator().manual_seed(5)
    x = torch.randint(-6, 7, (m, k), generator=g).float()
    for r in range(m):
        x[r] *= 2.0 ** (r % 7 - 3)
        x[r, (r * 131) % k] = 448.0 * 2.0 ** (r % 7 - 3) / 64   # amax = 7 * 2^e: s = 2^(e-6) exactly
    x[3] = 0
    w = torch.randint(-8, 9, (n, k), generator=g).float()
    wq = w.to(torch.float8_e4m3fn)
    ws = (torch.ones(n) * 0.5).float()
    xd = x.to(dtype).cuda()
    assert torch.equal(xd.float().cpu(), x)
    gq, gs = native.quant_rows(xd)
    two = native.gemm_fp8_rows(gq, gs, wq.cuda(), ws.cuda(), None, dtype, 4)
    fused = native.gemm_fp8_rows_fused(xd, wq.cuda(), ws.cuda(), None)
    assert torch.equal(fused, two)


def test_fused_row_nonfinite_rows_follow_the_quantizer():
    m, n, k = 16, 64, 256
    x, w, _ = operands(m, n, k, torch.bfloat16, seed=9)
    x[2, 7] = float("nan")
    x[4, 200] = float("inf")
    wq, ws = formats.quantize(w, "row", "weight")
    fused = native.gemm_fp8_rows_fused(x.cuda(), wq.cuda(), ws.cuda(), None)
    gq, gs = native.quant_rows(x.cuda())
    two = native.gemm_fp8_rows(gq, gs, wq.cuda(), ws.cuda(), None, torch.bfloat16, 4)
    assert torch.equal(torch.isnan(fused), torch.isnan(two))
    keep = ~torch.isnan(two)
    assert rel_l2(fused[keep].double().cpu(), two[keep].double().cpu()) <= 4e-3


# ---- block recipe ------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("m,n,k", [(1, 32, 128), (5, 96, 384), (16, 256, 1024), (17, 64, 640), (32, 192, 384), (20, 160, 256), (33, 128, 512), (48, 192, 640), (64, 256, 3072), (100, 96, 896)])
def test_fused_block_against_fp64_and_the_two_launch_path(dtype, m, n, k):
    x, w, bias = operands(m, n, k, dtype, seed=m + n + 2)
    w[: n // 2, : k // 2] *= 16.0   # weight blocks with different scales
    xq, xs = formats.quantize(x, "block", "act")
    wq, ws = formats.quantize(w, "block", "weight")
    truth = linear.exact64(xq, xs, "block") @ linear.exact64(wq, ws, "block").T + bias.double()
    eager = linear.fp8_forward(x, wq, ws, None, bias, "block")
    y = native.gemm_fp8_blocks_fused(x.cuda(), wq.cuda(), ws.cuda(), bias.cuda())
    assert y.shape == (m, n) and y.dtype == dtype
    assert_no_regression(y.cpu(), eager, truth, f"fused block {m}x{n}x{k}")
    assert rel_l2(y.cpu(), truth) <= REL_L2[dtype]
    gq, gs = native.quant_blocks(x.cuda(), "act")
    two = native.gemm_fp8_blocks(gq, gs, wq.cuda(), ws.cuda(), bias.cuda(), dtype, 1)
    assert rel_l2(y.cpu(), two.double().cpu()) <= 2 * REL_L2[dtype]
    y0 = native.gemm_fp8_blocks_fused(x.cuda(), wq.cuda(), ws.cuda(), None)
    assert rel_l2(y0.cpu(), truth - bias.double()) <= REL_L2[dtype]


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_fused_block_equals_the_two_launch_path_where_sums_are_exact(dtype):
    """Every 128-column block of a row has the abs-max 7 * 2^e (scale 2^(e-6) exactly), x holds
    small-integer multiples of 2^e and W small-integer codes with power-of-two block scales: all
    partial sums are exact, so the one-launch kernel must give the bytes of quantizer + GEMM."""
    for m, n, k in ((40, 96, 1024), (30, 128, 512)):
        g = torch.Generator().manual_seed(7)
        x = torch.randint(-6, 7, (m, k), generator=g).float()
        for r in range(m):
            for kb in range(k // 128):
                e = (r + 2 * kb) % 3 - 1
                x[r, kb * 128 : kb * 128 + 128] *= 2.0**e
                x[r, kb * 128 + (r * 37 + kb) % 128] = 7 * 2.0**e
        x[3] = 0
        wq = torch.randint(-4, 5, (n, k), generator=g).float().to(torch.float8_e4m3fn)
        ws = 2.0 ** torch.randint(-1, 2, (-(-n // 128), k // 128), generator=g).float()
        # promoted terms are multiples of 1/4 below 2^14 and there are at most 8 of them: exact in fp32
        xd = x.to(dtype).cuda()
        assert torch.equal(xd.float().cpu(), x)
        gq, gs = native.quant_blocks(xd, "act")
        two = native.gemm_fp8_blocks(gq, gs, wq.cuda(), ws.cuda(), None, dtype, 1)
        fused = native.gemm_fp8_blocks_fused(xd, wq.cuda(), ws.cuda(), None)
        assert torch.equal(fused, two), (m, n, k)


# ---- through the registered op ------------------------------------------------------------------


@pytest.mark.parametrize("recipe", ("mx", "row", "block"))
def test_short_m_through_the_registered_op(recipe, tmp_path, monkeypatch):
    """`fp8_linear` at 8 rows: with timing off the planner binds its first candidate (mx and block: the
    one-launch kernel); with the table on it times the one-launch kernel among the tile
    configurations and stores a winner. Either way the result obeys the GEMM tolerance."""
    from kohakumosstrainer_amd.kernels import tuning
    from kohakumosstrainer_amd.kernels.backends.hip import fp8_linear
    from kohakumosstrainer_amd.quant.compute import ComputeWeight

    registry.load_backends()
    m, n, k = 8, 256, 512
    x, w, bias = operands(m, n, k, torch.bfloat16, seed=21)
    xq, xs = formats.quantize(x, recipe)
    wq, ws = formats.quantize(w.to(torch.bfloat16), recipe, "weight")
    truth = linear.exact64(xq, xs, recipe) @ linear.exact64(wq, ws, recipe).T + bias.double()
    monkeypatch.setenv("KOHAKUMOSS_KERNEL_CACHE", str(tmp_path))
    try:
        for mode in ("off", "table"):
            tuning._tables.clear()
            tuning.set_mode(mode)
            tuning.reset()
            cw = ComputeWeight.from_weight(w.to(torch.bfloat16).cuda(), recipe)
            cw.bind(torch.bfloat16, torch.device("cuda"))
            y = cw.linear(x.cuda(), bias.cuda())
            assert rel_l2(y.cpu(), truth) <= REL_L2[torch.bfloat16], (recipe, mode)
            chosen = fp8_linear._select("fwd", x.cuda(), cw.q, cw.scale, cw.aux, bias.cuda(), recipe, False)
            if mode == "off":
                assert chosen["gemm"] == ("hip" if recipe == "row" else "fused")
            else:
                rows = list(tmp_path.rglob("fp8_fwd.json"))
                assert len(rows) == 1 and "fused" in rows[0].read_text(), "the one-launch kernel was among the timed candidates"
    finally:
        tuning._tables.clear()
        tuning.set_mode("table")
        tuning.reset()
