"""The large-tile GEMM configurations run with as many work-groups as the card holds at once; a
work-group walks several tiles, and the last K steps of one tile already fetch the first slabs and
scales of the next. Shapes here have more tiles than the card has compute units, ragged edges in
both directions and an odd, an even and a single K step, so that every kind of transition occurs:
interior -> interior, interior -> edge, a padded last step, the last tile of a work-group.

Checked per recipe: every tile configuration against configuration 4 (small tiles, one work-group
per tile) bit for bit over the whole output, and configuration 0 against the fp64 product of the
exactly dequantized operands on a sample of rows (stated tolerance for bf16 outputs:
||y - ref|| / ||ref|| <= 2e-3, as in test_gpu_gemm_fp8.py)."""

import pytest
import torch

from kohakumosstrainer_amd import native
from oracle import formats, linear
from oracle.stats import rel_l2

pytestmark = pytest.mark.gpu
REL_L2_BF16 = 2e-3
ONE_TILE_PER_GROUP = 4  # 64 x 128 tiles: never persistent
SHAPES = [(20000, 4200, 384), (33000, 2100, 256), (70000, 264, 128), (70000, 132, 128)]  # the last: no tile takes the vector epilogue (N % 8 != 0)


def operands(m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(m, k, generator=g) * torch.logspace(-2, 1, m)[:, None]).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g) * 0.05 * torch.logspace(-1, 1, n)[:, None]
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
    return x, w, bias


def sample_rows(m):
    return torch.cat([torch.arange(0, m, 211), torch.arange(max(m - 300, 0), m)]).unique()


def every_config_equal(run, kernel=None):
    """Configurations on the 16 x 16 x 128 MFMA add the same products in the same order whatever the
    tile: equal bit for bit. The 32 x 32 x 64 MFMA splits a K step in two: equal to rounding."""
    ref = run(ONE_TILE_PER_GROUP)
    for row in native.configs(kernel if kernel is not None else native.KERNEL_GEMM_MX):
        cfg = row["id"]
        if cfg == ONE_TILE_PER_GROUP:
            continue
        y = run(cfg)
        if row.get("mfma", 16) == 16:
            assert torch.equal(y, ref), f"configuration {cfg} differs from configuration {ONE_TILE_PER_GROUP} in {(y != ref).sum().item()} elements"
        else:
            assert rel_l2(y.float().cpu(), ref.double().cpu()) <= REL_L2_BF16, f"configuration {cfg}"
    return run(0)


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_mx_gemm_walks_tiles(m, n, k):
    x, w, bias = operands(m, n, k, seed=11)
    xq, xs = formats.quantize(x, "mx")
    wq, ws = formats.quantize(w, "mx", "weight")
    dx, dxs, dw, dws, db = xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), bias.cuda()
    y = every_config_equal(lambda cfg: native.gemm_mx(dx, dxs, dw, dws, db, torch.bfloat16, cfg))
    xsp, wsp = native.pack_scales(dxs), native.pack_scales(dws)
    yp = every_config_equal(lambda cfg: native.gemm_mx(dx, xsp, dw, wsp, db, torch.bfloat16, cfg, packed=True))
    assert torch.equal(yp, y), "packed against natural scales"
    rows = sample_rows(m)
    truth = linear.exact64(xq[rows], xs[rows], "mx") @ linear.exact64(wq, ws, "mx").T + bias.double()
    assert rel_l2(y[rows.cuda()].cpu(), truth) <= REL_L2_BF16
    nb = native.gemm_mx(dx, xsp, dw, wsp, None, torch.bfloat16, 0, packed=True)
    assert rel_l2(nb[rows.cuda()].cpu(), truth - bias.double()) <= REL_L2_BF16


@pytest.mark.parametrize("m,n,k", SHAPES[:2])
def test_row_and_tensor_gemm_walk_tiles(m, n, k):
    x, w, bias = operands(m, n, k, seed=12)
    rows = sample_rows(m)
    for recipe, gemm in (("row", native.gemm_fp8_rows), ("tensor", native.gemm_fp8_tensor)):
        xq, xs = formats.quantize(x, recipe)
        wq, ws = formats.quantize(w, recipe, "weight")
        dx, dxs, dw, dws, db = xq.cuda(), xs.cuda(), wq.cuda(), ws.cuda(), bias.cuda()
        y = every_config_equal(lambda cfg: gemm(dx, dxs, dw, dws, db, torch.bfloat16, cfg))
        xs_rows = xs[rows] if recipe == "row" else xs
        truth = linear.exact64(xq[rows], xs_rows, recipe) @ linear.exact64(wq, ws, recipe).T + bias.double()
        assert rel_l2(y[rows.cuda()].cpu(), truth) <= REL_L2_BF16, recipe


@pytest.mark.parametrize("m,n,k", SHAPES[:2])
def test_int8_gemm_walks_tiles(m, n, k):
    """int8 codes, int32 accumulation: the result is exact up to the last rounding, so the sample
    is compared with the oracle's arithmetic bit for bit."""
    g = torch.Generator().manual_seed(13)
    a = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    sa = torch.rand(m, generator=g) * 0.01 + 1e-4
    sb = torch.rand(n, generator=g) * 0.01 + 1e-4
    bias = (torch.randn(n, generator=g) * 0.1).to(torch.bfloat16)
    da, dsa, db_, dsb, dbias = a.cuda(), sa.cuda(), b.cuda(), sb.cuda(), bias.cuda()
    y = every_config_equal(lambda cfg: native.gemm_i8_rows(da, dsa, db_, dsb, dbias, torch.bfloat16, cfg), native.KERNEL_GEMM_FP8)
    rows = sample_rows(m)
    acc = (a[rows].double() @ b.double().T).float()  # exact: |sum| < 2^24 * 2^7
    want = (((acc * sa[rows, None]) * sb[None, :]) + bias.float()).to(torch.bfloat16)
    assert torch.equal(y[rows.cuda()].cpu(), want)


def test_resident_launch_under_graph_capture():
    """The first launch of a configuration asks the runtime how many work-groups the card holds;
    that query and the launch itself must work while a stream is being captured, and every replay
    must give the eager result (inputs refilled between replays, eager work in between)."""
    m, n, k = 4096, 4352, 256  # 16 x 17 = 272 tiles of 256 x 256: more than the card's compute units
    g = torch.Generator().manual_seed(21)
    dev = torch.device("cuda:0")
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16).to(dev)
    wq, _, wsp = native.quant_mx(w, natural=False, packed=True)
    static_x = x.clone()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        for cfg in (2, 0):  # warm both paths outside the capture as a training loop would
            xq, _, xsp = native.quant_mx(static_x, natural=False, packed=True)
            native.gemm_mx(xq, xsp, wq, wsp, None, torch.bfloat16, cfg, packed=True)
    torch.cuda.current_stream().wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        xq, _, xsp = native.quant_mx(static_x, natural=False, packed=True)
        y_graph = native.gemm_mx(xq, xsp, wq, wsp, None, torch.bfloat16, 0, packed=True)
    for i in range(3):
        fresh = torch.randn(m, k, generator=g).to(torch.bfloat16).to(dev) * (i + 1)
        static_x.copy_(fresh)
        graph.replay()
        xq, _, xsp = native.quant_mx(fresh, natural=False, packed=True)
        eager = native.gemm_mx(xq, xsp, wq, wsp, None, torch.bfloat16, 0, packed=True)
        torch.cuda.synchronize()
        assert torch.equal(y_graph, eager), f"replay {i}"
