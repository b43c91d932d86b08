"""The `block` fp8 recipe on the GPU through the C ABI: quantizers (`native.quant_blocks`, one
fp32 scale per row and 128 columns for activations, per 128 x 128 block for weights) against the
CPU oracle bit for bit, and the promoting GEMM (`native.gemm_fp8_blocks`) against the fp64
product of the exactly dequantized operands, next to the oracle's eager result, with the
reference's pass rule (`tests/kernels/quant/test_fp8.py:61-82,117-148`).
Stated tolerance for bf16 outputs: ||y - ref|| / ||ref|| <= 2e-3 (fp16: 4e-4)."""

import pytest
import torch

from kohakumosstrainer_amd import native
from kohakumosstrainer_amd.kernels import registry
from oracle import formats, linear
from oracle.stats import assert_no_regression, rel_l2, stats

pytestmark = pytest.mark.gpu
DTYPES = (torch.bfloat16, torch.float16)
REL_L2 = {torch.bfloat16: 2e-3, torch.float16: 4e-4}


def u8(t):
    return t.view(torch.uint8)


def operand(m, k, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) * torch.logspace(-3, 2, m)[:, None]
    x[:, : k // 2] *= torch.logspace(-2, 1, k // 2)[None, :]
    if m > 2:
        x[1] = 0.0
    return x.to(dtype)


def check(x_cpu, role, view=lambda t: t):
    q, s = native.quant_blocks(view(x_cpu.cuda()), role)
    rq, rs = formats.quantize(view(x_cpu), "block", role)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert q.shape == rq.shape and s.shape == rs.shape and q.is_contiguous() and s.is_contiguous()
    assert torch.equal(s.cpu().view(torch.int32), rs.view(torch.int32)), f"{role}: scale bits"
    assert torch.equal(u8(q).cpu(), u8(rq)), f"{role}: code bytes"
    if role == "act":
        # the K-major copy of the scales the GEMM reads: same numbers, transposed; alone or with the natural ones
        q2, s2, st = native.quant_blocks(view(x_cpu.cuda()), role, kmajor=True)
        q3, none, st3 = native.quant_blocks(view(x_cpu.cuda()), role, natural=False, kmajor=True)
        assert none is None and st.shape == (rs.shape[1], rs.shape[0]) and st.is_contiguous()
        assert torch.equal(st.view(torch.int32), s.t().view(torch.int32)) and torch.equal(st3.view(torch.int32), st.view(torch.int32))
        assert torch.equal(u8(q2), u8(q)) and torch.equal(u8(q3), u8(q)) and torch.equal(s2.view(torch.int32), s.view(torch.int32))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("role", ("act", "weight"))
@pytest.mark.parametrize("m,k", [(300, 1024), (1, 128), (7, 384), (128, 128), (129, 256), (1000, 384), (33, 4096), (256, 3072)])
def test_block_quantizer_bytes_equal_oracle(dtype, role, m, k):
    """Dense operands (vector kernels), rows not densely packed, a view that is not 16-byte
    aligned (element-wise kernel) and ragged row counts (weight blocks padded with zeros)."""
    x = operand(m, k, dtype, seed=21)
    check(x, role)
    if k >= 256:
        check(x, role, view=lambda t: t[:, 128:])       # unit stride, row pitch > cols
        wide = torch.zeros(m, k + 8, dtype=dtype)
        wide[:, 1 : k + 1] = x
        check(wide, role, view=lambda t: t[:, 1 : k + 1])  # misaligned: the dividing kernel


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("role", ("act", "weight"))
@pytest.mark.parametrize("n,k", [(256, 384), (384, 128), (200, 256), (256, 200), (128, 72)])
def test_block_quantizer_transposed_view(dtype, role, n, k):
    """`quantize(w.t(), "block", role)` of the input-gradient weight copy: the operand is [K, N]
    with unit stride down its rows; N must be a multiple of 128 only as its column count. A weight
    whose K is a multiple of 128 too is quantized in memory order and transposed; any other
    (K = 200, 72) takes the element-wise kernel."""
    w = operand(n, k, dtype, seed=5)
    if n % 128:
        with pytest.raises(ValueError):
            native.quant_blocks(w.cuda().t(), role)
        return
    check(w, role, view=lambda t: t.t())
    if role == "weight" and k % 128 == 0:
        q, s = native.quant_blocks(w.cuda(), "weight")
        qt, st = native.quant_blocks(w.cuda().t(), "weight")
        assert torch.equal(u8(qt), u8(q).t()) and torch.equal(st, s.t()), "blocks of the transpose are the transposed blocks"


def test_block_quantizer_zero_tiny_inf_and_nan_blocks():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(256, 256, generator=g)
    x[0] = 0.0
    x[1] = 1e-20                                   # below the 1e-12 amax floor
    x[2, 5] = float("inf")
    x[2, 130] = float("-inf")
    x[3, 7] = float("nan")
    x[4, ::2] = -0.0
    x[5] *= 1e30
    x[6] *= 1e-30
    x[130:140, 128:] = 0.0
    x[200, 200] = float("nan")
    x = x.to(torch.bfloat16)
    for role in ("act", "weight"):
        q, s = native.quant_blocks(x.cuda(), role)
        rq, rs = formats.quantize(x, "block", role)
        assert torch.equal(torch.isnan(s.cpu()), torch.isnan(rs)), role
        keep = ~torch.isnan(rs)
        assert torch.equal(s.cpu()[keep].view(torch.int32), rs[keep].view(torch.int32)), role
        assert torch.equal(u8(q).cpu(), u8(rq)), role
        # the misaligned view takes the dividing kernel: same bytes
        wide = torch.zeros(256, 264, dtype=torch.bfloat16, device="cuda")
        wide[:, 1:257] = x.cuda()
        q2, s2 = native.quant_blocks(wide[:, 1:257], role)
        assert torch.equal(u8(q2), u8(q)) and torch.equal(s2.view(torch.int32), s.view(torch.int32)), role
    floor = torch.tensor(1e-12).div(torch.tensor(448.0)).item()
    assert native.quant_blocks(x.cuda(), "act")[1][0, 0].item() == floor


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_quantizer_every_input_pattern_under_sampled_amax(dtype):
    """A block's 128 columns hold 16-bit patterns below a sampled amax pattern: every finite
    pattern of the dtype appears under 64 different block maxima, in both roles."""
    inf16 = 0x7F80 if dtype == torch.bfloat16 else 0x7C00
    g = torch.Generator().manual_seed(7)
    amax = torch.cat([torch.randint(1, inf16, (58,), generator=g), torch.tensor([0, 1, 0x80, inf16 - 1, inf16 // 2, inf16 // 2 + 1])])
    pats = torch.arange(0x10000, dtype=torch.int32)
    keep = (pats & 0x7FFF)[None, :] <= amax[:, None].to(torch.int32)
    m = torch.where(keep, pats[None, :], torch.zeros((), dtype=torch.int32))
    x = (m - (m >= 0x8000).to(torch.int32) * 0x10000).to(torch.int16).view(dtype)  # [64, 65536]
    check(x, "act")
    # the same blocks as 128 x 128 tiles of one amax each: tile (i, j) = 128 patterns x 128 rows
    tiles = x.view(64, 4, 128, 128).permute(0, 2, 1, 3).reshape(64 * 128, 512).contiguous()
    check(tiles, "weight")


def test_block_quantizer_full_size_operands():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(16384, 3072, generator=g)
    mask = torch.rand(x.shape, generator=g) < 1e-3
    x = torch.where(mask, torch.randn(x.shape, generator=g) * 50, x).to(torch.bfloat16)
    check(x, "act")
    w = (torch.randn(9216, 3072, generator=g) * 0.02).to(torch.bfloat16)
    check(w, "weight")
    check(w, "weight", view=lambda t: t.t())


def test_block_argument_errors():
    x = torch.zeros(4, 256, device="cuda")
    with pytest.raises(ValueError):
        native.quant_blocks(x, "act")  # fp32 input
    with pytest.raises(ValueError):
        native.quant_blocks(x.bfloat16()[:, :200], "act")
    with pytest.raises(ValueError):
        native.quant_blocks(x.bfloat16(), "bias")
    with pytest.raises(ValueError):
        native.quant_blocks(x.bfloat16(), "weight", kmajor=True)
    q, s = native.quant_blocks(x.bfloat16()[:0], "weight")
    assert q.shape == (0, 256) and s.shape == (0, 2)
    a = torch.zeros(8, 256, device="cuda").to(torch.float8_e4m3fn)
    with pytest.raises(ValueError):
        native.gemm_fp8_blocks(a, torch.ones(8, 2, device="cuda"), a, torch.ones(8, 2, device="cuda"), None, torch.bfloat16)


# ---- GEMM ---------------------------------------------------------------------------------


def gemm_operands(m, n, k, dtype, seed=0, spread=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    if spread:
        x = x * torch.logspace(-3, 2, m)[:, None]
        x[:, k // 2 :] *= 8.0   # K blocks of one row with different scales
    w = torch.randn(n, k, generator=g) * 0.05
    w[: n // 2, : k // 2] *= 16.0   # weight blocks with different scales
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    return x.to(dtype), w, bias


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,n,k", [(200, 384, 256), (1, 256, 512), (1000, 512, 384), (513, 200, 1024), (256, 256, 128), (130, 136, 640), (384, 128, 896)])
def test_block_gemm_against_fp64(dtype, m, n, k):
    x, w, bias = gemm_operands(m, n, k, dtype)
    xq, xs = formats.quantize(x, "block", "act")
    wq, ws = formats.quantize(w, "block", "weight")
    truth = linear.exact64(xq, xs, "block") @ linear.exact64(wq, ws, "block").T + bias.double()
    eager = linear.fp8_forward(x, wq, ws, None, bias, "block")
    n_cfg = len(native.configs(native.KERNEL_GEMM_BLOCKS))
    assert n_cfg >= 2
    for cfg in range(n_cfg):
        y = native.gemm_fp8_blocks(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), bias.cuda(), dtype, cfg)
        assert y.shape == (m, n) and y.dtype == dtype
        assert_no_regression(y.cpu(), eager, truth, f"block cfg{cfg} {m}x{n}x{k}")
        assert rel_l2(y.cpu(), truth) <= REL_L2[dtype]
        y0 = native.gemm_fp8_blocks(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), None, dtype, cfg)
        assert rel_l2(y0.cpu(), truth - bias.double()) <= REL_L2[dtype]
        yk = native.gemm_fp8_blocks(xq.cuda(), xs.t().contiguous().cuda(), wq.cuda(), ws.cuda(), bias.cuda(), dtype, cfg, kmajor=True)
        assert torch.equal(yk, y), "K-major activation scales"
        if cfg:
            assert torch.equal(y, first), "tile configurations add the same blocks in the same order"
        first = y


@pytest.mark.parametrize("m,n,k,dtype", [(4400, 4500, 256, torch.bfloat16), (4400, 4500, 384, torch.bfloat16), (8192, 2304, 512, torch.bfloat16),
                                         (4400, 4500, 256, torch.float16)])
def test_block_gemm_walks_more_tiles_than_compute_units(m, n, k, dtype):
    """More 256 x 256 tiles than the device has compute units: the large-tile configuration then walks
    several tiles per work-group (even numbers of K steps) and fetches a tile's first slabs during
    the tile before. Ragged last rows and columns; every configuration gives the same bytes."""
    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn(m, k, generator=g) * torch.logspace(-2, 2, m)[:, None]).to(dtype).cuda()
    w = (torch.randn(n, k, generator=g) * 0.05).to(dtype).cuda()
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype).cuda()
    wq, ws = native.quant_blocks(w, "weight")
    xq, xs, xs_t = native.quant_blocks(x, "act", natural=True, kmajor=True)
    cfgs = native.configs(native.KERNEL_GEMM_BLOCKS)
    assert any(c["bm"] * c["bn"] == 256 * 256 for c in cfgs) and (m // 256) * (n // 256) > 256
    outs = [native.gemm_fp8_blocks(xq, xs_t, wq, ws, bias, dtype, c["id"], kmajor=True) for c in cfgs]
    torch.cuda.synchronize()
    for c, y in zip(cfgs[1:], outs[1:]):
        assert torch.equal(y, outs[0]), f"configuration {c}"
    # and the same through the natural scale layout, twice in a row (nothing left over between launches)
    for c in cfgs:
        for _ in range(2):
            assert torch.equal(native.gemm_fp8_blocks(xq, xs, wq, ws, bias, dtype, c["id"]), outs[0]), f"configuration {c}"
    # rows against the 64-bit product of the dequantized operands
    rows = torch.tensor([0, 255, 256, 2047, m - 1])
    a64 = xq[rows.cuda()].float().double() * xs[rows.cuda()].double().repeat_interleave(128, dim=1)
    w64 = wq.float().double() * ws.double().repeat_interleave(128, dim=0)[:n].repeat_interleave(128, dim=1)
    truth = a64 @ w64.T + bias.double()
    assert rel_l2(outs[0][rows.cuda()].cpu(), truth.cpu()) <= REL_L2[dtype]


def test_block_gemm_uses_every_scale():
    """One scale changed by a factor of 2 (activation: one row and K block; weight: one 128 x 128
    block) must change exactly the outputs it covers, by the partial product of that block."""
    m, n, k = 256, 384, 512
    x, w, _ = gemm_operands(m, n, k, torch.bfloat16, seed=2, spread=False)
    xq, xs = native.quant_blocks(x.cuda(), "act")
    wq, ws = native.quant_blocks(w.cuda().bfloat16(), "weight")
    base = native.gemm_fp8_blocks(xq, xs, wq, ws, None, torch.float16).float()
    xs2 = xs.clone()
    xs2[77, 2] *= 2
    moved = (native.gemm_fp8_blocks(xq, xs2, wq, ws, None, torch.float16).float() != base).nonzero()
    assert set(moved[:, 0].tolist()) == {77}
    ws2 = ws.clone()
    ws2[1, 3] *= 2
    moved = (native.gemm_fp8_blocks(xq, xs, wq, ws2, None, torch.float16).float() != base).nonzero()
    assert moved[:, 1].min() >= 128 and moved[:, 1].max() < 256 and moved.shape[0] > 0.9 * m * 128


def test_block_gemm_deep_k_accumulates_in_fp32():
    """M,N,K = 2048,512,8192 (reference `tests/kernels/quant/test_fp8_accumulation.py:83-90`). Each
    128-deep block product comes from the matrix instruction, which sums groups of 8 products with
    13 fraction bits (`oracle/mfma_model.py`), and is promoted into an fp32 running sum. Checked
    against that model with no fitted slack: on a 32 x 128 slice the fp16 and bf16 outputs equal the
    correctly rounded model except within the adders' bound of a rounding boundary; over the whole
    output abs_mean / rel_mean are no worse than the eager result's moved by the mean cut measured
    on the slice; a running sum rounded to bf16 at every promotion must fail."""
    import numpy as np

    from oracle import mfma_model
    from tests._mfma_check import check_against_model, no_worse_than_eager

    m, n, k = 2048, 512, 8192
    g = torch.Generator().manual_seed(0)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g) * 0.02
    xq, xs = formats.quantize(x, "block", "act")
    wq, ws = formats.quantize(w, "block", "weight")
    a64, b64 = linear.exact64(xq, xs, "block"), linear.exact64(wq, ws, "block")
    truth = a64 @ b64.T
    eager_y = linear.fp8_forward(x, wq, ws, None, None, "block")

    rows, cols = slice(700, 732), slice(0, 128)
    unit = lambda r: np.full((r, k // 32), 127, np.uint8)
    parts = mfma_model.step_partials(xq.view(torch.uint8).numpy()[rows], unit(32), wq.view(torch.uint8).numpy()[cols], unit(128))
    parts = parts * xs.double().numpy()[rows].T[:, :, None] * ws.double().numpy()[0][:, None, None]  # s[m, kb] * sb[n/128 = 0, kb]
    model = parts.sum(0)
    reach = mfma_model.running_abs_max(parts)
    bound = mfma_model.float_add_bound(reach, k) + (k // 128) * 2.0**-23 * reach  # + one fp32 multiply-add per block
    cut = np.abs(model - truth[rows, cols].numpy()).mean()
    assert 0 < cut < 1e-4

    def no_worse(y, what="block"):
        report = no_worse_than_eager(y, eager_y, truth, float(cut), what)
        print(f"deep K {what}: abs_mean {report['abs_mean']:.3e} <= {report['abs_allowed']:.3e}, rel_mean {report['rel_mean']:.3e} <= {report['rel_allowed']:.3e}")

    for cfg in range(len(native.configs(native.KERNEL_GEMM_BLOCKS))):
        ybf = native.gemm_fp8_blocks(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), None, torch.bfloat16, cfg).cpu()
        y16 = native.gemm_fp8_blocks(xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), None, torch.float16, cfg).cpu()
        check_against_model(y16[rows, cols], ybf[rows, cols], model, bound, f"block cfg{cfg}")
        no_worse(ybf)
    lossy = torch.zeros(m, n, dtype=torch.bfloat16)
    for kb in range(k // 128):
        sl = slice(kb * 128, (kb + 1) * 128)
        lossy = (lossy.double() + a64[:, sl] @ b64[:, sl].T).to(torch.bfloat16)
    try:
        no_worse(lossy)
    except AssertionError:
        return
    raise AssertionError("a bf16 running sum passed the accumulation check")


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_recipe_through_the_registered_op(dtype):
    """`fp8_linear` resolved on the GPU with recipe="block": forward and both input gradients
    (fp8 through the W^T copy, 16-bit without it) and the bias gradient."""
    from kohakumosstrainer_amd.quant.compute import ComputeWeight

    registry.load_backends()
    m, n, k = 300, 384, 256
    x, w, bias = gemm_operands(m, n, k, dtype, seed=4, spread=False)
    for with_dgrad in (True, False):
        cw = ComputeWeight.from_weight(w.cuda().to(dtype), "block", dgrad=with_dgrad)
        cw.bind(dtype, torch.device("cuda"))
        rq, rs = formats.quantize(w.to(dtype), "block", "weight")
        assert torch.equal(u8(cw.q).cpu(), u8(rq)) and torch.equal(cw.scale.cpu(), rs)
        xg = x.cuda().requires_grad_(True)
        bg = bias.cuda().requires_grad_(True)
        y = cw.linear(xg, bg)
        xq, xs = formats.quantize(x, "block", "act")
        truth = linear.exact64(xq, xs, "block") @ linear.exact64(rq, rs, "block").T + bias.double()
        assert rel_l2(y.detach().cpu(), truth) <= REL_L2[dtype]
        gdy = torch.Generator().manual_seed(9)
        dy = (torch.randn(m, n, generator=gdy) * 0.1).to(dtype)
        y.backward(dy.cuda())
        w64 = linear.exact64(rq, rs, "block")
        if with_dgrad:
            dq, ds = formats.quantize(dy, "block", "act")
            tq, ts = formats.quantize(w.to(dtype).t(), "block", "weight")
            assert torch.equal(u8(cw.q_t).cpu(), u8(tq)) and torch.equal(cw.scale_t.cpu(), ts)
            dx_truth = linear.exact64(dq, ds, "block") @ linear.exact64(tq, ts, "block").T
        else:
            dx_truth = dy.double() @ w64
        assert rel_l2(xg.grad.cpu(), dx_truth) <= 2 * REL_L2[dtype]
        assert rel_l2(bg.grad.cpu(), dy.double().sum(0)) <= REL_L2[dtype]
