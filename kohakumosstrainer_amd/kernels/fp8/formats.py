"""fp8 compute formats: quantizer and dequantizer of every recipe.

An operand is 2-D `[rows, K]` with K the contraction axis; codes are e4m3fn (max 448).

    tensor  one fp32 scale [1]
    row     one fp32 scale per row [rows]
    block   activations: fp32 per row and 128 columns; weights: fp32 per 128x128 block
    mx      OCP MX: one E8M0 byte per 32 columns [rows, K/32]

Interface and arithmetic follow reference `src/kohakumoss_kernels/fp8/formats.py:70-136`.
`quantize` runs the hand-written HIP quantizers for device tensors of the recipes the GPU
path serves (mx, tensor, row; bf16 / fp16 input) and plain torch ops otherwise (host tensors,
the block recipe, fp32 input): both produce the same bytes. `pack_mx` builds the
MFMA-packed scale copy the HIP GEMM reads (the role `swizzle_mx` plays for a vendor GEMM).
"""

import torch
from torch import Tensor

E4M3 = torch.float8_e4m3fn
E4M3_MAX = 448.0
MX_BLOCK = 32
BLOCK = 128
RECIPES = ("tensor", "row", "block", "mx")
ROLES = ("act", "weight")
_HIP_DTYPES = (torch.bfloat16, torch.float16)


def _check(x: Tensor, recipe: str, role: str) -> None:
    if recipe not in RECIPES:
        raise ValueError(f"fp8 recipe {recipe!r} not in {RECIPES}")
    if role not in ROLES:
        raise ValueError(f"fp8 role {role!r} not in {ROLES}")
    if x.dim() != 2:
        raise ValueError(f"fp8 operand must be 2-D, got {tuple(x.shape)}")
    step = {"block": BLOCK, "mx": MX_BLOCK}.get(recipe, 1)
    if x.shape[1] % step:
        raise ValueError(f"fp8 {recipe}: K={x.shape[1]} is not a multiple of {step}")


def _scale_of(amax: Tensor) -> Tensor:
    # tensor / tensor: the correctly rounded fp32 division
    a = amax.float().clamp_min(1e-12)
    return a / torch.full_like(a, E4M3_MAX)


def _codes(v: Tensor, s: Tensor) -> Tensor:
    return (v / s).clamp_(-E4M3_MAX, E4M3_MAX).to(E4M3)


def mx_biased_exponent(amax: Tensor) -> Tensor:
    """int32 e + 127 of the block scale 2^e: from amax = m 2^E, e = E - 8, one more when
    m > 1.75 (448 = 1.75 * 2^8); the amax floor 1e-30 gives an all-zero block byte 19."""
    bits = amax.float().clamp_min(1e-30).view(torch.int32)
    return ((bits >> 23) & 0xFF) - 8 + ((bits & 0x7FFFFF) > 0x600000).to(torch.int32)


def pow2_from_biased(biased: Tensor, sign: int = 1) -> Tensor:
    """Exact fp32 2^(sign * (biased - 127))."""
    return ((127 + sign * (biased.to(torch.int32) - 127)) << 23).view(torch.float32)


def _quantize_torch(x: Tensor, recipe: str, role: str) -> tuple[Tensor, Tensor]:
    v = x.detach().float().contiguous()
    rows, k = v.shape
    if recipe == "tensor":
        s = _scale_of(v.abs().amax().reshape(1))
        return _codes(v, s), s
    if recipe == "row":
        s = _scale_of(v.abs().amax(1))
        return _codes(v, s[:, None]), s
    if recipe == "mx":
        g = v.view(rows, k // MX_BLOCK, MX_BLOCK)
        biased = mx_biased_exponent(g.abs().amax(-1))
        q = (g * pow2_from_biased(biased, -1)[..., None]).clamp_(-E4M3_MAX, E4M3_MAX).to(E4M3)
        return q.view(rows, k), biased.to(torch.uint8)
    if role == "act":
        g = v.view(rows, k // BLOCK, BLOCK)
        s = _scale_of(g.abs().amax(-1))
        return _codes(g, s[..., None]).view(rows, k), s
    g = torch.nn.functional.pad(v, (0, 0, 0, -rows % BLOCK)).view(-1, BLOCK, k // BLOCK, BLOCK)
    s = _scale_of(g.abs().amax((1, 3)))
    return _codes(g, s[:, None, :, None]).view(-1, k)[:rows], s


def quantize(x: Tensor, recipe: str, role: str = "act") -> tuple[Tensor, Tensor]:
    """`(q e4m3 [rows, K], scale)` of a 2-D operand under `recipe`; `role` matters only for
    `block` (weights scale 128x128 blocks)."""
    _check(x, recipe, role)
    if x.device.type == "cuda" and x.dtype in _HIP_DTYPES and x.numel():
        from kohakumosstrainer_amd import native

        x = x.detach()
        if recipe == "block":
            return native.quant_blocks(x, role)
        return {"mx": native.quant_mx, "tensor": native.quant_tensor, "row": native.quant_rows}[recipe](x)
    return _quantize_torch(x, recipe, role)


def dequantize(q: Tensor, scale: Tensor, recipe: str, dtype: torch.dtype) -> Tensor:
    """`q * scale` in fp32, rounded once to `dtype` (a block scale with fewer rows than `q` is
    a 128x128 weight-block scale)."""
    rows, k = q.shape
    v = q.float()
    if recipe == "tensor":
        out = v * scale.float().reshape(())
    elif recipe == "row":
        out = v * scale.float()[:, None]
    elif recipe == "mx":
        out = (v.view(rows, k // MX_BLOCK, MX_BLOCK) * pow2_from_biased(scale)[..., None]).view(rows, k)
    elif recipe == "block" and scale.shape[0] == rows:
        out = (v.view(rows, k // BLOCK, BLOCK) * scale.float()[..., None]).view(rows, k)
    elif recipe == "block":
        g = torch.nn.functional.pad(v, (0, 0, 0, -rows % BLOCK)).view(-1, BLOCK, k // BLOCK, BLOCK)
        out = (g * scale.float()[:, None, :, None]).view(-1, k)[:rows]
    else:
        raise ValueError(f"fp8 recipe {recipe!r} not in {RECIPES}")
    return out.to(dtype)


def swizzle_mx(scale: Tensor) -> Tensor:
    """`[rows, K/32]` uint8 -> the flat 128x4-tile SWIZZLE_32_4_4 layout of a vendor block-scaled
    GEMM, zero padded: byte (r, c) at (r//128)*ct*512 + (c//4)*512 + (r%32)*16 + ((r%128)//32)*4 + c%4."""
    rows, cols = scale.shape
    rt, ct = -(-rows // 128), -(-cols // 4)
    padded = scale.new_zeros(rt * 128, ct * 4)
    padded[:rows, :cols] = scale
    return padded.view(rt, 4, 32, ct, 4).permute(0, 3, 2, 1, 4).reshape(-1).contiguous()


def packed_numel(rows: int, k: int) -> int:
    """Bytes of the MFMA-packed scale copy of a `[rows, k]` mx operand (k % 128 == 0)."""
    return (k // 128) * (-(-rows // 128)) * 512


def pack_mx(scale: Tensor) -> Tensor:
    """`[rows, K/32]` uint8 (K % 128 == 0) -> the MFMA-packed copy the gfx950 GEMM reads: per K
    step of 128 and group of 128 rows, 512 bytes ordered [row%16][block%4][row%128//16], i.e.
    byte (r, b) at ((((b//4)*ceil(rows/128) + r//128)*16 + r%16)*4 + b%4)*8 + (r%128)//16; rows
    past the end are zero padding."""
    rows, blocks = scale.shape
    if blocks % 4:
        raise ValueError(f"packed mx scales need K % 128 == 0, got K={blocks * 32}")
    if scale.device.type == "cuda" and rows:
        from kohakumosstrainer_amd import native

        return native.pack_scales(scale)
    groups = -(-rows // 128)
    padded = scale.new_zeros(groups * 128, blocks)
    padded[:rows] = scale
    # [group, tile, r16, step, b4] -> [step, group, r16, b4, tile]
    return padded.view(groups, 8, 16, blocks // 4, 4).permute(3, 0, 2, 4, 1).reshape(-1).contiguous()
