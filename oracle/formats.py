"""Oracle (test infrastructure): fp8 compute formats on the CPU with torch.

Restates the reference's eager quantizer / dequantizer,
`src/kohakumoss_kernels/fp8/formats.py:44-136`. An operand is 2-D `[rows, K]`, K the
contraction axis, codes are `float8_e4m3fn` (largest finite 448):

    tensor  one fp32 scale [1]
    row     one fp32 scale per row [rows]
    block   fp32 per row and 128 columns (activations) / per 128x128 block (weights)
    mx      one E8M0 byte per row and 32 columns [rows, K/32]

fp32 scales are `max(amax, 1e-12) / 448` as a correctly rounded fp32 division and the
codes round `x / s` once. The mx exponent is read from the bits of the fp32 block amax
`m * 2^E`: `e = E - 8`, one more when `m > 1.75` (448 = 1.75 * 2^8), never below -127,
stored with bias 127; codes round `x * 2^-e` once. An all-zero block therefore stores
the byte of the amax floor 1e-30, which is 19.
"""

import torch
from torch import Tensor

E4M3 = torch.float8_e4m3fn
E4M3_MAX = 448.0
MX_BLOCK = 32
BLOCK = 128
RECIPES = ("tensor", "row", "block", "mx")
ROLES = ("act", "weight")
AMAX_FLOOR = 1e-12
MX_AMAX_FLOOR = 1e-30
E8M0_BIAS = 127


def validate(x: Tensor, recipe: str, role: str) -> None:
    """Argument errors of `quantize` (reference `formats.py:33-41`): ValueError."""
    if recipe not in RECIPES:
        raise ValueError(f"fp8 recipe {recipe!r} not in {RECIPES}")
    if role not in ROLES:
        raise ValueError(f"fp8 role {role!r} not in {ROLES}")
    if x.dim() != 2:
        raise ValueError(f"fp8 operand must be 2-D, got {tuple(x.shape)}")
    group = {"block": BLOCK, "mx": MX_BLOCK}.get(recipe, 1)
    if x.shape[1] % group:
        raise ValueError(f"fp8 {recipe}: K={x.shape[1]} is not a multiple of {group}")


def fp32_scale(amax: Tensor) -> Tensor:
    """`max(amax, 1e-12) / 448`, both operands tensors so the division is the correctly
    rounded one (reference `formats.py:48-52`)."""
    a = amax.to(torch.float32).clamp_min(AMAX_FLOOR)
    return a / torch.full_like(a, E4M3_MAX)


def round_e4m3(v: Tensor, s: Tensor) -> Tensor:
    """`v / s` clamped to the e4m3 range and rounded once (reference `formats.py:44-45`)."""
    return torch.clamp(v / s, -E4M3_MAX, E4M3_MAX).to(E4M3)


def mx_biased_exponent(amax: Tensor) -> Tensor:
    """int32 `e + 127` of the power-of-two block scale `2^e` from the bits of the fp32
    amax (reference `formats.py:55-61`)."""
    word = amax.to(torch.float32).clamp_min(MX_AMAX_FLOOR).view(torch.int32)
    exponent = (word >> 23) & 0xFF
    round_up = ((word & 0x007FFFFF) > 0x00600000).to(torch.int32)
    return (exponent - 8 + round_up).clamp_min(0)


def pow2_from_biased(biased: Tensor, sign: int = 1) -> Tensor:
    """Exact fp32 `2^(sign * (biased - 127))` built from exponent bits (reference
    `formats.py:64-67`); `biased` in [0, 254]."""
    e = biased.to(torch.int32) - E8M0_BIAS
    return ((E8M0_BIAS + sign * e) << 23).view(torch.float32)


def quantize(x: Tensor, recipe: str, role: str = "act") -> tuple[Tensor, Tensor]:
    """`(q e4m3 [rows, K], scale)` of a 2-D operand (reference `formats.py:70-100`).
    `role` only matters for `block`."""
    validate(x, recipe, role)
    v = x.detach().to(torch.float32).contiguous()
    rows, k = v.shape
    if recipe == "tensor":
        s = fp32_scale(v.abs().amax().reshape(1))
        return round_e4m3(v, s), s
    if recipe == "row":
        s = fp32_scale(v.abs().amax(dim=1))
        return round_e4m3(v, s[:, None]), s
    if recipe == "mx":
        blocks = v.view(rows, k // MX_BLOCK, MX_BLOCK)
        biased = mx_biased_exponent(blocks.abs().amax(dim=-1))
        inverse = pow2_from_biased(biased, -1)
        q = (blocks * inverse[..., None]).clamp_(-E4M3_MAX, E4M3_MAX).to(E4M3)
        return q.view(rows, k), biased.to(torch.uint8)
    if role == "act":
        blocks = v.view(rows, k // BLOCK, BLOCK)
        s = fp32_scale(blocks.abs().amax(dim=-1))
        return round_e4m3(blocks, s[..., None]).view(rows, k), s
    padded = torch.nn.functional.pad(v, (0, 0, 0, -rows % BLOCK))
    blocks = padded.view(-1, BLOCK, k // BLOCK, BLOCK)
    s = fp32_scale(blocks.abs().amax(dim=(1, 3)))
    q = round_e4m3(blocks, s[:, None, :, None]).view(-1, k)[:rows]
    return q, s


def dequantize(q: Tensor, scale: Tensor, recipe: str, dtype: torch.dtype) -> Tensor:
    """`q * scale` in fp32, rounded once to `dtype` (reference `formats.py:103-125`)."""
    rows, k = q.shape
    v = q.to(torch.float32)
    if recipe == "tensor":
        out = v * scale.to(torch.float32).reshape(())
    elif recipe == "row":
        out = v * scale.to(torch.float32)[:, None]
    elif recipe == "mx":
        blocks = v.view(rows, k // MX_BLOCK, MX_BLOCK)
        out = (blocks * pow2_from_biased(scale)[..., None]).view(rows, k)
    elif recipe == "block" and scale.shape[0] == rows:
        blocks = v.view(rows, k // BLOCK, BLOCK)
        out = (blocks * scale.to(torch.float32)[..., None]).view(rows, k)
    elif recipe == "block":
        padded = torch.nn.functional.pad(v, (0, 0, 0, -rows % BLOCK))
        blocks = padded.view(-1, BLOCK, k // BLOCK, BLOCK)
        out = (blocks * scale.to(torch.float32)[:, None, :, None]).view(-1, k)[:rows]
    else:
        raise ValueError(f"fp8 recipe {recipe!r} not in {RECIPES}")
    return out.to(dtype)


def swizzle_mx(scale: Tensor) -> Tensor:
    """`[rows, K/32]` E8M0 bytes -> the flat 128-row x 4-column tile layout of a vendor
    block-scaled GEMM, zero padded (reference `formats.py:128-136`): byte (r, c) lands at
    `(r//128)*ct*512 + (c//4)*512 + (r%32)*16 + ((r%128)//32)*4 + c%4`, ct = ceil(cols/4).
    """
    rows, cols = scale.shape
    row_tiles, col_tiles = -(-rows // 128), -(-cols // 4)
    padded = scale.new_zeros(row_tiles * 128, col_tiles * 4)
    padded[:rows, :cols] = scale
    tiles = padded.view(row_tiles, 4, 32, col_tiles, 4)  # [rt, r//32, r%32, ct, c%4]
    return tiles.permute(0, 3, 2, 1, 4).reshape(-1).contiguous()
