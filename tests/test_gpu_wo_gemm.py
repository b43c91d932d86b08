"""HIP weight-only dequant-GEMMs through the C ABI against the fp64 product with the exact
dequantized weight, next to the oracle's eager result (dequantize, then a 16-bit matmul),
with the reference's pass rule. Mirrors reference `tests/kernels/quant/test_quant.py`
(off-tile shapes, int8 and fp8 codes, both 16-bit dtypes, bias on and off, the
wrong-scale-axis negative control)."""

import pytest
import torch

from kohakumosstrainer_amd import native
from oracle import linear
from oracle.stats import assert_no_regression, rel_l2

pytestmark = pytest.mark.gpu
SHAPES = ((200, 150, 136), (1, 96, 64), (513, 384, 1000), (300, 256, 512), (1024, 512, 256), (512, 320, 768))


def must_fail(check, what=""):
    try:
        check()
    except AssertionError:
        return
    raise AssertionError(f"check passed on the broken variant: {what}")


def case(m, n, k, fmt, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(n, k, generator=g) * 0.05
    q, scale = linear.quantize_weight(w, fmt)
    x = torch.randn(m, k, generator=g).to(dtype)
    bias = (torch.randn(n, generator=g) * 0.1).to(dtype)
    dy = torch.randn(m, n, generator=g).to(dtype)
    return x, q, scale, bias, dy


def n_configs():
    return len(native.configs(native.KERNEL_WO_FWD))


@pytest.mark.parametrize("fmt", ("int8", "fp8"))
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("with_bias", (False, True))
def test_forward_and_dgrad(fmt, dtype, m, n, k, with_bias):
    x, q, scale, bias, dy = case(m, n, k, fmt, dtype)
    b = bias if with_bias else None
    w64 = linear.wo_exact64(q, scale)
    truth = x.double() @ w64.T + (b.double() if with_bias else 0)
    eager = linear.wo_forward(x, q, scale, b)
    tol = 2e-3 if dtype == torch.bfloat16 else 4e-4
    for cfg in range(n_configs()):
        y = native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), None if b is None else b.cuda(), cfg)
        assert y.shape == (m, n) and y.dtype == dtype
        assert_no_regression(y.cpu(), eager, truth, f"wo fwd {fmt} cfg{cfg} {m}x{n}x{k}")
        assert rel_l2(y.cpu(), truth) <= tol
    truth_dx = dy.double() @ w64
    eager_dx = linear.wo_dgrad(dy, q, scale)
    first = None
    for cfg in range(n_configs()):
        dx = native.wo_gemm_dgrad(dy.cuda(), q.cuda(), scale.cuda(), cfg)
        assert dx.shape == (m, k) and dx.dtype == dtype
        assert_no_regression(dx.cpu(), eager_dx, truth_dx, f"wo dgrad {fmt} cfg{cfg} {m}x{n}x{k}")
        # every tile shape sums a row's products in the same order
        first = dx if first is None else first
        assert torch.equal(dx, first), f"cfg{cfg} differs from cfg0"
    if n % 8 == 0:
        # the entry point that transposes the codes into a workspace first feeds the MFMA the same operands
        assert torch.equal(native.wo_gemm_dgrad_workspace(dy.cuda(), q.cuda(), scale.cuda(), 0), first)


def fp8_base(n, k, recipe, seed=0):
    """(q, scale) of a frozen fp8 compute base quantized by the oracle, plus its exact fp64 value."""
    from oracle import formats

    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
    q, scale = formats.quantize(w, recipe, "weight")
    w64 = formats.dequantize(q, scale, recipe, torch.float64)
    return q, scale, w64


@pytest.mark.parametrize("recipe", ("tensor", "row", "mx", "block"))
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("m,n,k", ((200, 256, 384), (64, 128, 128), (513, 1024, 640), (300, 384, 1152)))
def test_input_gradient_of_an_fp8_base_without_a_transposed_copy(recipe, dtype, m, n, k):
    """dx = dy @ dequantize(q, scale) over the codes as stored, for every scale layout of the fp8
    compute recipes (reference `backends/triton/fp8/linear.py:152-153`): against the fp64 product
    with the exactly dequantized weight, next to the oracle's eager result (10x rule), every tile
    shape; the widened weight itself is read back through identity rows, bit for bit."""
    from oracle import formats

    q, scale, w64 = fp8_base(n, k, recipe)
    g = torch.Generator().manual_seed(5)
    dy = torch.randn(m, n, generator=g).to(dtype)
    truth = dy.double() @ w64
    eager = linear.fp8_dgrad(dy, q, scale, None, None, None, recipe)
    first = None
    for cfg in range(n_configs()):
        dx = native.wo_gemm_dgrad(dy.cuda(), q.cuda(), scale.cuda(), cfg, recipe)
        assert dx.shape == (m, k) and dx.dtype == dtype
        assert_no_regression(dx.cpu(), eager, truth, f"w16 dgrad {recipe} cfg{cfg} {m}x{n}x{k}")
        # every tile shape (and lane layout) sums a row's products in the same order
        first = dx if first is None else first
        assert torch.equal(dx, first), f"{recipe} cfg{cfg} differs from cfg0"
    eye = torch.eye(n, dtype=dtype)[:256]
    back = native.wo_gemm_dgrad(eye.cuda(), q.cuda(), scale.cuda(), 0, recipe).cpu()
    assert torch.equal(back, formats.dequantize(q, scale, recipe, dtype)[:256])


@pytest.mark.parametrize("fmt", ("int8", "fp8"))
def test_two_tile_shapes_in_one_call(fmt):
    """The configuration with `tail` covers whole rounds of the card with 256 x 256 tiles and the
    remaining tile columns with half-size tiles (128 x 256 forward, 256 x 128 for the gradient) in a
    second launch. 17 x 17 large tiles are more
    than the card's compute units and not a multiple of them, rows and columns are ragged, and the
    columns of the second launch start in the middle of the output: every element must equal the
    one-shape configuration's bit for bit, forward (bias and scale follow the column window) and
    input gradient."""
    mixed = [c["id"] for c in native.configs(native.KERNEL_WO_FWD) if c.get("tail", 0)]
    assert mixed, "no configuration with a tail"
    m, wide, deep = 4100, 4200, 264
    x, q, scale, bias, _ = case(m, wide, deep, fmt, torch.bfloat16, seed=3)  # forward: 4200 output columns
    y0 = native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), bias.cuda(), 0)
    _, q2, scale2, _, dy = case(m, deep, wide, fmt, torch.bfloat16, seed=4)  # gradient: 4200 input features
    dx0 = native.wo_gemm_dgrad(dy.cuda(), q2.cuda(), scale2.cuda(), 0)
    assert rel_l2(y0.cpu(), x.double() @ linear.wo_exact64(q, scale).T + bias.double()) <= 2e-3
    # the gradient multiplies by the weight rounded to 16 bits: judged next to the eager result
    assert_no_regression(dx0.cpu(), linear.wo_dgrad(dy, q2, scale2), dy.double() @ linear.wo_exact64(q2, scale2), f"wo dgrad {fmt} 17 x 17 tiles")
    for cfg in mixed:
        assert torch.equal(native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), bias.cuda(), cfg), y0)
        assert torch.equal(native.wo_gemm_dgrad(dy.cuda(), q2.cuda(), scale2.cuda(), cfg), dx0)


def test_two_tile_shapes_when_the_large_tiles_cover_everything():
    """256 x 2 large tiles are whole rounds of a card with 256 (or 128, 64 ...) compute units, and the
    last tile column is only 128 wide: the window of the half-size tiles starts past the last
    128-column tile and must come out empty, not negative."""
    mixed = [c["id"] for c in native.configs(native.KERNEL_WO_FWD) if c.get("tail", 0)][0]
    m, n, k = 65536, 64, 384
    _, q, scale, _, dy = case(m, n, k, "fp8", torch.bfloat16, seed=8)
    dx0 = native.wo_gemm_dgrad(dy.cuda(), q.cuda(), scale.cuda(), 0)
    assert torch.equal(native.wo_gemm_dgrad(dy.cuda(), q.cuda(), scale.cuda(), mixed), dx0)
    x, q, scale, bias, _ = case(m, k, n, "fp8", torch.bfloat16, seed=9)
    y0 = native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), bias.cuda(), 0)
    assert torch.equal(native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), bias.cuda(), mixed), y0)


def test_two_tile_shapes_under_graph_capture():
    """Both launches of the two-shape configuration, and its question to the runtime about the
    number of compute units, inside a captured stream: every replay equals the eager result (inputs
    refilled between replays, eager work in between)."""
    mixed = [c["id"] for c in native.configs(native.KERNEL_WO_FWD) if c.get("tail", 0)][0]
    m, n, k = 4100, 264, 4200
    _, q, scale, _, dy = case(m, n, k, "fp8", torch.bfloat16, seed=6)
    dq, dscale, static_dy = q.cuda(), scale.cuda(), dy.cuda()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        native.wo_gemm_dgrad(static_dy, dq, dscale, 0)  # the library is loaded; the mixed configuration may be new to it
    torch.cuda.current_stream().wait_stream(stream)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        dx_graph = native.wo_gemm_dgrad(static_dy, dq, dscale, mixed)
    g = torch.Generator().manual_seed(7)
    for i in range(3):
        fresh = (torch.randn(m, n, generator=g) * (i + 1)).to(torch.bfloat16).cuda()
        static_dy.copy_(fresh)
        graph.replay()
        eager = native.wo_gemm_dgrad(fresh, dq, dscale, 0)
        torch.cuda.synchronize()
        assert torch.equal(dx_graph, eager), f"replay {i}"


@pytest.mark.parametrize("fmt,recipe", (("int8", "row"), ("fp8", "row"), ("fp8", "mx")))
@pytest.mark.parametrize("m,n,k", ((37, 100, 50), (130, 96, 66), (16, 64, 1), (5, 0, 64)))
def test_input_gradient_shapes_off_the_vector_path(fmt, recipe, m, n, k):
    """N not a multiple of 8, K not a multiple of 4, an empty contraction, a misaligned operand: the
    one-thread-per-element kernel, judged by the same rule."""
    from oracle import formats

    g = torch.Generator().manual_seed(11)
    if recipe == "mx":
        n, k = max(n, 32), 64 if k < 32 else 96
        w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
        q, scale = formats.quantize(w, "mx", "weight")
        w64 = formats.dequantize(q, scale, "mx", torch.float64)
        dy = torch.randn(m, n, generator=g).to(torch.bfloat16)
        eager = linear.fp8_dgrad(dy, q, scale, None, None, None, "mx")
        # a view one element into a buffer: the pointer is not 16-byte aligned
        shifted = torch.empty(m * n + 1, dtype=torch.bfloat16, device="cuda")[1:].view(m, n).copy_(dy)
        dx = native.wo_gemm_dgrad(shifted, q.cuda(), scale.cuda(), 0, "mx")
    else:
        w = torch.randn(n, k, generator=g) * 0.05
        q, scale = linear.quantize_weight(w, fmt) if n else (torch.zeros(0, k, dtype=torch.int8 if fmt == "int8" else torch.float8_e4m3fn), torch.zeros(0))
        w64 = linear.wo_exact64(q, scale)
        dy = torch.randn(m, n, generator=g).to(torch.bfloat16)
        eager = linear.wo_dgrad(dy, q, scale)
        dx = native.wo_gemm_dgrad(dy.cuda(), q.cuda(), scale.cuda(), 0, "row")
    assert dx.shape == (m, k)
    if n == 0:
        assert not dx.any(), "an empty contraction gives zeros"
        return
    assert_no_regression(dx.cpu(), eager, dy.double() @ w64, f"scalar dgrad {fmt} {recipe} {m}x{n}x{k}")


def test_leaving_the_tiled_kernels_is_announced_once_per_shape():
    """A ragged problem is served, correctly, by the one-thread-per-element kernel; the binding says so
    once per direction and shape instead of leaving a silent cliff for the tuner to time."""
    import warnings

    x, q, scale, bias, dy = case(24, 40, 36, "int8", torch.bfloat16, seed=3)  # K % 8 != 0
    native._SLOW_SEEN.clear()
    with pytest.warns(native.SlowPathWarning, match="forward M=24 N=40 K=36"):
        native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), None)
    with warnings.catch_warnings():
        warnings.simplefilter("error", native.SlowPathWarning)
        native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), None)  # the second call is silent
        x2, q2, s2, _, dy2 = case(24, 64, 128, "int8", torch.bfloat16, seed=4)
        native.wo_gemm_fwd(x2.cuda(), q2.cuda(), s2.cuda(), None)  # a shape the tiles take: no warning
        native.wo_gemm_dgrad(dy2.cuda(), q2.cuda(), s2.cuda())
    x3, q3, s3, _, dy3 = case(24, 36, 64, "int8", torch.bfloat16, seed=5)  # N % 8 != 0
    with pytest.warns(native.SlowPathWarning, match="input gradient M=24 N=36 K=64"):
        native.wo_gemm_dgrad(dy3.cuda(), q3.cuda(), s3.cuda())


def test_int8_forward_is_exact_product_for_small_integers():
    """Integer activations and codes with unit scales: every product and partial sum is an
    integer below 2^24, so the kernel must reproduce the fp64 product exactly after the one
    bf16 rounding."""
    g = torch.Generator().manual_seed(3)
    m, n, k = 130, 192, 320
    x = torch.randint(-4, 5, (m, k), generator=g).to(torch.bfloat16)
    q = torch.randint(-127, 128, (n, k), generator=g).to(torch.int8)
    scale = torch.ones(n)
    y = native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), None, 0).cpu()
    want = (x.double() @ q.double().T).to(torch.bfloat16)
    assert torch.equal(y, want)


@pytest.mark.parametrize("fmt", ("int8", "fp8"))
def test_error_check_rejects_wrong_scale_axis(fmt):
    m, n, k = 64, 96, 96
    x, q, scale, _, _ = case(m, n, k, fmt, torch.bfloat16)
    eager = linear.wo_forward(x, q, scale, None)
    truth = x.double() @ linear.wo_exact64(q, scale).T
    good = native.wo_gemm_fwd(x.cuda(), q.cuda(), scale.cuda(), None, 0).cpu()
    assert_no_regression(good, eager, truth, "good")
    scale_in = scale[torch.arange(k) % n]
    broken = (x.float() @ (q.float() * scale_in[None, :]).T).to(torch.bfloat16)
    must_fail(lambda: assert_no_regression(broken, eager, truth, "broken"), "scale along the input axis")
    rolled = native.wo_gemm_fwd(x.cuda(), q.cuda(), (scale * torch.where(torch.arange(n) % 2 == 0, 1.0, 64.0)).roll(1).cuda(), None, 0).cpu()
    must_fail(lambda: assert_no_regression(rolled, eager, truth, "rolled"), "scales on the wrong rows")


def test_int8_weight_only_frozen_base_shape():
    """x bf16 [4096, 3072], W int8 [3072, 3072] uniform in [-127, 127], scale |N(0,0.02)|/127 + 1e-6,
    fp32 bias ~N(0,0.01): a 256-row slice against the fp64 product, and the whole output
    against the slice-wise property that rows are independent (permutation equivariance)."""
    g = torch.Generator().manual_seed(0)
    m, k, n = 4096, 3072, 3072
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    q = torch.randint(-127, 128, (n, k), generator=g).to(torch.int8)
    scale = torch.randn(n, generator=g).abs() * 0.02 / 127 + 1e-6
    bias = torch.randn(n, generator=g) * 0.01
    xg, qg, sg, bg = x.cuda(), q.cuda(), scale.cuda(), bias.to(torch.bfloat16).cuda()
    y = native.wo_gemm_fwd(xg, qg, sg, bg, 0)
    rows = torch.arange(1000, 1256)
    truth = x[rows].double() @ linear.wo_exact64(q, scale).T + bias.to(torch.bfloat16).double()
    eager = linear.wo_forward(x[rows], q, scale, bias)
    assert_no_regression(y[rows].cpu(), eager, truth, "int8 frozen base")
    assert rel_l2(y[rows].cpu(), truth) <= 2e-3
    perm = torch.randperm(m, generator=g).cuda()
    assert torch.equal(native.wo_gemm_fwd(xg[perm].contiguous(), qg, sg, bg, 0), y[perm])
    # every tile shape (the 192-column one fills the card exactly at this shape) adds a row's
    # products in the same order
    dy = torch.randn(m, n, generator=g).to(torch.bfloat16).cuda()
    dx = native.wo_gemm_dgrad(dy, qg, sg, 0)
    for cfg in range(1, n_configs()):
        assert torch.equal(native.wo_gemm_fwd(xg, qg, sg, bg, cfg), y), f"forward cfg{cfg}"
        assert torch.equal(native.wo_gemm_dgrad(dy, qg, sg, cfg), dx), f"input gradient cfg{cfg}"


def test_fp8_weight_only_per_tensor_scale_mlp_up_projection():
    """The DiT MLP up-projection shape: x bf16 [8192, 3072] ~N(0,1) (eight packed samples; only
    the token count matters to the linear), W bf16 ~N(0,0.02) [12288, 3072] quantized with ONE
    scale s = amax / 448 (tensor / tensor division) and handed to the op as that value broadcast
    to the 12288 rows, bf16 bias. Forward and input gradient: a 256-row slice against the fp64
    product with the exactly dequantized weight next to the oracle's eager result (10x rule,
    rel-L2 <= 2e-3 forward, 4e-3 for the gradient whose scale lies on the contraction axis), and
    the whole output against row-permutation equivariance."""
    from oracle import formats

    m, k, n = 8192, 3072, 12288
    g = torch.Generator().manual_seed(0)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    g.manual_seed(1)
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(n, generator=g) * 0.01).to(torch.bfloat16)
    g.manual_seed(2)
    dy = (torch.randn(m, n, generator=g) * 0.01).to(torch.bfloat16)
    q, s = formats.quantize(w, "tensor", "weight")
    assert s.numel() == 1 and s.item() == (w.float().abs().amax() / torch.tensor(448.0)).item()
    scale = s.reshape(1).expand(n).contiguous()
    xg, qg, sg, bg, dyg = x.cuda(), q.cuda(), scale.cuda(), bias.cuda(), dy.cuda()
    w64 = linear.wo_exact64(q, scale)
    rows = torch.arange(3000, 3256)
    perm = torch.randperm(m, generator=g).cuda()

    y = native.wo_gemm_fwd(xg, qg, sg, bg, 0)
    truth = x[rows].double() @ w64.T + bias.double()
    assert_no_regression(y[rows].cpu(), linear.wo_forward(x[rows], q, scale, bias), truth, "e4m3 per-tensor fwd")
    assert rel_l2(y[rows].cpu(), truth) <= 2e-3
    assert torch.equal(native.wo_gemm_fwd(xg[perm].contiguous(), qg, sg, bg, 0), y[perm])

    dx = native.wo_gemm_dgrad(dyg, qg, sg, 0)
    truth_dx = dy[rows].double() @ w64
    assert_no_regression(dx[rows].cpu(), linear.wo_dgrad(dy[rows], q, scale), truth_dx, "e4m3 per-tensor dgrad")
    assert rel_l2(dx[rows].cpu(), truth_dx) <= 4e-3
    assert torch.equal(native.wo_gemm_dgrad(dyg[perm].contiguous(), qg, sg, 0), dx[perm])
    for cfg in range(1, n_configs()):
        assert torch.equal(native.wo_gemm_fwd(xg, qg, sg, bg, cfg), y), f"forward cfg{cfg}"
        assert torch.equal(native.wo_gemm_dgrad(dyg, qg, sg, cfg), dx), f"input gradient cfg{cfg}"


def test_argument_errors():
    x = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    q = torch.zeros(16, 64, dtype=torch.int8, device="cuda")
    s = torch.ones(16, device="cuda")
    with pytest.raises(ValueError):
        native.wo_gemm_fwd(x, q.float(), s, None)
    with pytest.raises(ValueError):
        native.wo_gemm_fwd(x, q[:, :32], s, None)
    with pytest.raises(ValueError):
        native.wo_gemm_fwd(x, q, s[:3], None)
    with pytest.raises(native.KernelError):
        native.wo_gemm_fwd(x, q, s, None, 99)
    assert native.wo_gemm_fwd(x[:0], q, s, None).shape == (0, 16)


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_every_e4m3_code_widens_exactly(dtype):
    """Identity activations read the widened weight back: forward must return every finite
    e4m3 code's exact value (all are representable in bf16 and f16), dgrad the once-rounded
    scaled value. (The two NaN codes are left out: a NaN weight poisons every sum it is in.)"""
    codes = torch.arange(256, dtype=torch.uint8)
    codes[0x7F] = 0
    codes[0xFF] = 0x80
    q = torch.cat([codes.repeat(2, 1), codes.flip(0).repeat(2, 1)], 0).contiguous().view(torch.float8_e4m3fn)  # [N=4, K=256]
    scale = torch.tensor([1.0, 0.37, 3.0, 1e-3])
    eye = torch.eye(256, dtype=dtype)
    y = native.wo_gemm_fwd(eye.cuda(), q.cuda(), torch.ones(4).cuda(), None, 0).cpu()  # [256, 4] = W^T
    assert torch.equal(y.float(), q.float().t())
    dx = native.wo_gemm_dgrad(torch.eye(4, dtype=dtype).cuda(), q.cuda(), scale.cuda(), 0).cpu()  # [4, 256] = round(W * s)
    assert torch.equal(dx, (q.float() * scale[:, None]).to(dtype))
