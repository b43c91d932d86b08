"""HIP quantizers against the CPU oracle, bit for bit, through the C ABI
(`native.quant_mx` / `native.quant_tensor` / `native.quant_rows`). Mirrors reference
`tests/kernels/quant/test_fp8.py:61-82` (bytes equal the eager reference, strided input)
and adds the column-wise (transposed) case, an exhaustive bf16 sweep and the full-size
`[16384, 3072]` operand with outliers."""

import pytest
import torch

from kohakumosstrainer_amd import native
from oracle import formats

pytestmark = pytest.mark.gpu
DTYPES = (torch.bfloat16, torch.float16)


def u8(t):
    return t.view(torch.uint8)


def activations(m, k, dtype, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) * torch.logspace(-3, 2, m)[:, None]
    if m > 2:
        x[1] = 0.0
        x[2, : min(k, 32)] = torch.linspace(-1.75, 1.75, 32)[: min(k, 32)]
    if m > 3 and k >= 64:
        x[3, 32:64] = torch.linspace(-1.75, 1.75, 32) * (1 + 2.0**-7)
    return x.to(dtype)


def packed_reference(scale: torch.Tensor) -> torch.Tensor:
    """The MFMA-packed copy of natural scales [rows, blocks] by its index formula: byte
    (r, b) -> ((((b//4)*ceil(rows/128) + r//128)*16 + r%16)*4 + b%4)*8 + (r%128)//16."""
    rows, blocks = scale.shape
    groups = -(-rows // 128)
    out = torch.zeros((blocks // 4) * groups * 512, dtype=torch.uint8)
    r = torch.arange(rows)[:, None].expand(rows, blocks)
    b = torch.arange(blocks)[None, :].expand(rows, blocks)
    off = ((((b // 4) * groups + r // 128) * 16 + r % 16) * 4 + b % 4) * 8 + (r % 128) // 16
    out[off.reshape(-1)] = scale.reshape(-1)
    return out


def check_mx(x_cpu: torch.Tensor, view=lambda t: t):
    """Quantize `view(x)` on the GPU and with the oracle; bytes must be equal."""
    xg = view(x_cpu.cuda())
    q, s = native.quant_mx(xg)
    rq, rs = formats.quantize(view(x_cpu), "mx", "act")
    if xg.shape[1] % 128 == 0:
        q2, s2, sp = native.quant_mx(xg, packed=True)
        assert torch.equal(u8(q2), u8(q)) and torch.equal(s2, s)
        assert torch.equal(sp.cpu(), packed_reference(rs)), "packed scale bytes"
        _, none, sp3 = native.quant_mx(xg, natural=False, packed=True)
        assert none is None and torch.equal(sp3, sp)
        assert torch.equal(native.pack_scales(s), sp)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.uint8
    assert q.shape == rq.shape and s.shape == rs.shape
    assert q.is_contiguous() and s.is_contiguous()
    assert torch.equal(s.cpu(), rs), "scale bytes"
    assert torch.equal(u8(q).cpu(), u8(rq)), "code bytes"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k", [(300, 1024), (1, 32), (7, 96), (1000, 384), (33, 4096)])
def test_mx_rows_bytes_equal_oracle(dtype, m, k):
    check_mx(activations(m, k, dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k", [(256, 64), (320, 200), (32, 8), (1024, 384), (96, 1000), (4096, 72)])
def test_mx_cols_bytes_equal_oracle(dtype, m, k):
    """Column-wise quantization: the operand is the transposed view of an [m, k] tensor."""
    check_mx(activations(m, k, dtype, seed=3), view=lambda t: t.t())


@pytest.mark.parametrize("dtype", DTYPES)
def test_mx_strided_and_unaligned_views(dtype):
    base = activations(130, 640, dtype, seed=5)
    check_mx(base, view=lambda t: t[:, 64:576])  # row stride > K
    check_mx(base, view=lambda t: t[3:, 32:96])  # aligned offset start
    check_mx(base, view=lambda t: t[:, 1:65])  # 2-byte aligned only: generic kernel
    check_mx(base, view=lambda t: t[::2, ::2][:, :160])  # both strides non-unit
    check_mx(base, view=lambda t: t.t().contiguous().t())  # column-major storage
    check_mx(base, view=lambda t: t[:96, :33].t())  # transposed, odd leading dimension


def test_mx_every_finite_bf16_pattern():
    x = torch.arange(65536, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16)
    x = x[torch.isfinite(x.float())]
    x = x[: (x.numel() // 32) * 32]
    for seed in range(4):
        perm = torch.randperm(x.numel(), generator=torch.Generator().manual_seed(seed))
        check_mx(x[perm].view(-1, 32 * (1 + seed % 2)))
        check_mx(x[perm].view(32, -1), view=lambda t: t.t())


def test_mx_zero_block_byte_and_sign_of_zero():
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    x[0, 0] = -0.0
    x[1, :32] = torch.tensor([-1e-38, 1e-38] * 16, dtype=torch.bfloat16)
    q, s = native.quant_mx(x.cuda())
    assert s[0].tolist() == [19, 19] and s[2].tolist() == [19, 19]
    assert u8(q)[0, 0].item() == 0x80 and u8(q)[0, 1].item() == 0
    check_mx(x)


def test_mx_nan_and_inf_elements():
    x = activations(8, 128, torch.bfloat16)
    x[0, 5] = float("inf")
    x[4, 70] = float("nan")
    q, s = native.quant_mx(x.cuda())
    rq, rs = formats.quantize(x, "mx")
    assert torch.equal(s.cpu(), rs) and torch.equal(u8(q).cpu(), u8(rq))


def test_mx_argument_errors():
    with pytest.raises(ValueError):
        native.quant_mx(torch.zeros(4, 48, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        native.quant_mx(torch.zeros(64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(ValueError):
        native.quant_mx(torch.zeros(4, 64, dtype=torch.float32, device="cuda"))
    with pytest.raises(ValueError):
        native.quant_mx(torch.zeros(4, 64, dtype=torch.bfloat16))
    q, s = native.quant_mx(torch.zeros(0, 64, dtype=torch.bfloat16, device="cuda"))
    assert q.shape == (0, 64) and s.shape == (0, 2)


def outlier_operand(m=16384, k=3072):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(m, k, generator=g)
    mask = torch.rand(m, k, generator=g) < 1e-3
    x[mask] = (torch.randn(m, k, generator=g) * 50)[mask]
    return x.to(torch.bfloat16)


def test_mx_full_size_rows_and_cols_with_outliers():
    """bf16 [16384, 3072] ~N(0,1) with 0.1 % entries +-N(0,50): row-wise and column-wise."""
    x = outlier_operand()
    check_mx(x)
    check_mx(x, view=lambda t: t.t())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k", [(300, 1024), (5, 7), (1, 1), (64, 200)])
def test_tensor_recipe_bytes_equal_oracle(dtype, m, k):
    x = activations(m, k, dtype, seed=7)
    q, s = native.quant_tensor(x.cuda())
    rq, rs = formats.quantize(x, "tensor")
    assert s.dtype == torch.float32 and s.shape == (1,)
    assert torch.equal(s.cpu(), rs)
    assert torch.equal(u8(q).cpu(), u8(rq))
    q2, s2 = native.quant_tensor(x.cuda().t())
    rq2, rs2 = formats.quantize(x.t(), "tensor")
    assert torch.equal(s2.cpu(), rs2) and torch.equal(u8(q2).cpu(), u8(rq2))


def test_tensor_recipe_all_zero_and_weight_like():
    z = torch.zeros(16, 64, dtype=torch.bfloat16)
    q, s = native.quant_tensor(z.cuda())
    rq, rs = formats.quantize(z, "tensor")
    assert torch.equal(s.cpu(), rs) and torch.equal(u8(q).cpu(), u8(rq))
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(1024, 768, generator=g) * 0.02).to(torch.bfloat16)
    q, s = native.quant_tensor(w.cuda())
    rq, rs = formats.quantize(w, "tensor")
    assert torch.equal(s.cpu(), rs) and torch.equal(u8(q).cpu(), u8(rq))


def check_rows(x_cpu: torch.Tensor, view=lambda t: t):
    q, s = native.quant_rows(view(x_cpu.cuda()))
    rq, rs = formats.quantize(view(x_cpu), "row")
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32 and s.shape == (rq.shape[0],)
    assert q.shape == rq.shape and q.is_contiguous()
    assert torch.equal(s.cpu().view(torch.int32), rs.view(torch.int32)), "scale bits"
    assert torch.equal(u8(q).cpu(), u8(rq)), "code bytes"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("m,k", [(300, 1024), (5, 7), (1, 1), (64, 200), (33, 4096), (9, 4104), (130, 8192), (3, 12288), (256, 384), (48, 200), (1040, 136)])
def test_row_recipe_bytes_equal_oracle(dtype, m, k):
    """Reference `tests/kernels/quant/test_fp8.py:61-82` for the row recipe: rows kept in
    registers (K <= 4096), rows read twice (K > 4096), ragged K (element-wise kernel) and the
    transposed view `quantize(w.t(), "row")` of the input-gradient weight copy."""
    x = activations(m, k, dtype, seed=11)
    check_rows(x)
    check_rows(x, view=lambda t: t.t())
    if k >= 16:
        check_rows(x, view=lambda t: t[:, 8:])          # unit stride, rows not densely packed
        check_rows(x, view=lambda t: t[:, 1 : k - 1])   # not 16-byte aligned


def test_row_recipe_power_of_two_scales_hit_rounding_ties():
    """With amax = 448 * 2^e the scale is 2^e and x / s is exact, so bf16 inputs (8 significand
    bits) land on e4m3 ties (4 significand bits), in its subnormal range and on the clamp."""
    bits = torch.arange(0x3000, 0x4400, dtype=torch.int32)  # every bf16 pattern in [2^-31, 512)
    vals = (bits << 16).view(torch.float32)
    rows = []
    for e in (-20, -3, 0, 5, 40):
        r = vals * 2.0**e
        r = torch.where(r.abs() > 448 * 2.0**e, torch.zeros(()), r)
        r[0] = 448 * 2.0**e
        rows += [r, -r]
    x = torch.stack(rows).to(torch.bfloat16)
    assert torch.equal(x.float(), torch.stack(rows))
    check_rows(x)                                   # 5120 columns: the re-reading kernel
    check_rows(x[:, :4096].contiguous())            # rows held in registers
    check_rows(x.to(torch.float16)[4:8])


def test_row_recipe_zero_tiny_inf_and_nan_rows():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(8, 256, generator=g)
    x[0] = 0.0
    x[1] = 1e-20                                   # below the 1e-12 amax floor
    x[2, 5] = float("inf")
    x[2, 6] = float("-inf")
    x[3, 7] = float("nan")
    x[4, ::2] = -0.0
    x[5] *= 1e30
    x[6] *= 1e-30
    x = x.to(torch.bfloat16)
    q, s = native.quant_rows(x.cuda())
    rq, rs = formats.quantize(x, "row")
    assert torch.equal(torch.isnan(s.cpu()), torch.isnan(rs))
    keep = ~torch.isnan(rs)
    assert torch.equal(s.cpu()[keep].view(torch.int32), rs[keep].view(torch.int32))
    assert torch.equal(u8(q).cpu(), u8(rq))
    assert s.cpu()[0].item() == rs[0].item() == torch.tensor(1e-12).div(torch.tensor(448.0)).item()
    # the same rows as columns of a [256, 8] matrix: the transposing kernels
    xt = x.t().contiguous()
    q2, s2 = native.quant_rows(xt.cuda().t())
    assert torch.equal(u8(q2), u8(q)) and torch.equal(s2.view(torch.int32), s.view(torch.int32))


def pattern_rows(amax_patterns: torch.Tensor, dtype) -> torch.Tensor:
    """Row i holds every 16-bit pattern of `dtype` whose magnitude is at most amax_patterns[i]
    (the others are zero), so its amax is exactly that pattern: [len, 65536]."""
    pats = torch.arange(0x10000, dtype=torch.int32, device=amax_patterns.device)
    keep = (pats & 0x7FFF)[None, :] <= amax_patterns[:, None].to(torch.int32)
    m = torch.where(keep, pats[None, :], torch.zeros((), dtype=torch.int32, device=pats.device))
    return (m - (m >= 0x8000).to(torch.int32) * 0x10000).to(torch.int16).view(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_row_recipe_every_input_pattern_under_sampled_amax(dtype):
    inf16 = 0x7F80 if dtype == torch.bfloat16 else 0x7C00
    g = torch.Generator().manual_seed(5)
    amax = torch.cat([torch.randint(1, inf16, (250,), generator=g), torch.tensor([0, 1, 0x80, inf16 - 1, inf16 // 2, inf16 // 2 + 1])])
    check_rows(pattern_rows(amax, dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_row_recipe_vector_kernels_equal_the_dividing_kernel_on_every_pair(dtype):
    """The vectorized kernels form x / s from a rounded reciprocal and two fused corrections;
    the element-wise kernel (taken for a view that is not 16-byte aligned) divides. Every
    (amax, x) pair of finite 16-bit patterns with |x| <= amax must give the same byte."""
    inf16 = 0x7F80 if dtype == torch.bfloat16 else 0x7C00
    chunk = 2048
    for a0 in range(0, inf16, chunk):
        amax = torch.arange(a0, min(a0 + chunk, inf16), device="cuda")
        x = pattern_rows(amax, dtype)
        wide = torch.zeros(x.shape[0], x.shape[1] + 8, dtype=dtype, device="cuda")
        wide[:, 1:-7] = x
        q_fast, s_fast = native.quant_rows(x)
        q_div, s_div = native.quant_rows(wide[:, 1:-7])
        assert torch.equal(s_fast.view(torch.int32), s_div.view(torch.int32))
        assert torch.equal(u8(q_fast), u8(q_div)), f"amax patterns {a0}..{a0 + chunk}"
        del x, wide, q_fast, q_div


def test_row_recipe_full_size_activation():
    x = outlier_operand()
    check_rows(x)
    check_rows(x, view=lambda t: t.t())


def test_row_recipe_argument_errors():
    x = torch.zeros(4, 8, device="cuda")
    with pytest.raises(ValueError):
        native.quant_rows(x)  # fp32 input
    with pytest.raises(ValueError):
        native.quant_rows(x.bfloat16()[0])
    q, s = native.quant_rows(x.bfloat16()[:0])
    assert q.shape == (0, 8) and s.shape == (0,)


def test_mx_committed_vectors_rows_and_cols():
    """The committed known-answer bytes (definition-level, independent of the oracle): the
    row-wise kernel on the vectors as they are, the column-wise kernel on their transpose."""
    from pathlib import Path

    import numpy as np

    d = np.load(Path(__file__).parent / "golden" / "mx_vectors.npz")
    x = torch.from_numpy(d["x_bits"].astype(np.int32)).to(torch.uint16).view(torch.bfloat16)
    want_q, want_s = torch.from_numpy(d["codes"]), torch.from_numpy(d["scales"])
    q, s = native.quant_mx(x.cuda())
    assert torch.equal(u8(q).cpu(), want_q) and torch.equal(s.cpu(), want_s)
    xt = x.t().contiguous().cuda()  # [128, R]: quantizing xt.t() runs the transposing kernel
    q2, s2 = native.quant_mx(xt.t())
    assert torch.equal(u8(q2).cpu(), want_q) and torch.equal(s2.cpu(), want_s)
