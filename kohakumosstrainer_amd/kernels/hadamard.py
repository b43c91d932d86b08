"""Group Hadamard rotation (ConvRot): `x . blockdiag(H_g)` along the last axis, `g = 4^j`.

`H_g` is the j-fold Kronecker power of the 4 x 4 matrix with ones everywhere but -1 on the
anti-diagonal, scaled by `2^-j`: symmetric, its own inverse, every entry `+-2^-j` (exact in
fp16 and bf16). So the rotation is its own backward: `d/dx (x R) = dy R`.

On a gfx950 device 16-bit tensors go to the HIP butterfly kernel (`km_group_hadamard`);
elsewhere 16-bit inputs multiply by `H_g` in their own dtype and other dtypes run the fp32
butterflies (both as reference `src/kohakumoss_kernels/hadamard.py:31-101`).
"""

from __future__ import annotations

from functools import lru_cache

import torch
from torch import Tensor

GROUPS = (4, 16, 64, 256, 1024)
HALF = (torch.float16, torch.bfloat16)
_SEED = ((1.0, 1.0, 1.0, -1.0), (1.0, 1.0, -1.0, 1.0), (1.0, -1.0, 1.0, 1.0), (-1.0, 1.0, 1.0, 1.0))


def stages(group: int) -> int:
    """`j` with `group == 4^j`, j >= 1; ValueError for anything else."""
    g, j = int(group), 0
    while g >= 4 and g % 4 == 0:
        g, j = g // 4, j + 1
    if g != 1 or j == 0:
        raise ValueError(f"Hadamard group {group} is not a power of 4 >= 4")
    return j


def check_group(x: Tensor, group: int) -> int:
    j = stages(group)
    if x.shape[-1] % group:
        raise ValueError(f"last dim {x.shape[-1]} is not a multiple of group {group}")
    return j


@lru_cache(maxsize=None)
def _matrix(group: int, dtype: torch.dtype, device: str) -> Tensor:
    seed = torch.tensor(_SEED)
    h = seed
    for _ in range(stages(group) - 1):
        h = torch.kron(h, seed)
    return (h / float(2 ** stages(group))).to(device=device, dtype=dtype)


def hadamard_matrix(group: int, dtype: torch.dtype = torch.float32, device="cpu") -> Tensor:
    """`H_group` (a fresh copy the caller may modify)."""
    return _matrix(int(group), dtype, str(torch.device(device))).clone()


def _butterflies(x: Tensor, group: int) -> Tensor:
    """fp32 stages of 4-point butterflies, most significant base-4 digit of the index first:
    with t = ((x0 + x1) + x2) + x3 the outputs are t - 2 x3, t - 2 x2, t - 2 x1, t - 2 x0."""
    j = check_group(x, group)
    v = x.to(torch.float32)
    outer = v.numel() // group
    for stage in range(j):
        inner = group // 4 ** (stage + 1)
        quad = v.reshape(outer * 4**stage, 4, inner)
        total = ((quad[:, 0] + quad[:, 1]) + quad[:, 2]) + quad[:, 3]
        v = torch.stack([total - 2.0 * quad[:, 3 - i] for i in range(4)], dim=1)
    return (v.reshape(x.shape) * (0.5**j)).to(x.dtype)


def group_hadamard_eager(x: Tensor, group: int) -> Tensor:
    check_group(x, group)
    if x.dtype in HALF:
        h = _matrix(int(group), x.dtype, str(x.device))
        return (x.reshape(-1, group) @ h).reshape(x.shape)
    return _butterflies(x, group)


def rotate_2d(x: Tensor, group: int) -> Tensor:
    """Rotation without autograd: the HIP kernel for 16-bit device tensors on gfx950, the eager
    forms otherwise."""
    check_group(x, group)
    if x.is_cuda and x.dtype in HALF:
        from kohakumosstrainer_amd.kernels.arch import arch_of

        if arch_of(x.device).name == "gfx950":
            from kohakumosstrainer_amd import native

            return native.group_hadamard(x.reshape(-1, x.shape[-1]), group).reshape(x.shape)
    return group_hadamard_eager(x, group)


_LIB = torch.library.Library("kohakumoss_amd", "FRAGMENT")
_LIB.define("group_hadamard(Tensor x, int group) -> Tensor")
torch.library.impl("kohakumoss_amd::group_hadamard", "CompositeExplicitAutograd", lib=_LIB)(lambda x, group: rotate_2d(x, group))
torch.library.register_fake("kohakumoss_amd::group_hadamard", lib=_LIB)(lambda x, group: torch.empty_like(x))


def _setup(ctx, inputs, output):
    ctx.group = inputs[1]


def _backward(ctx, grad):
    return torch.ops.kohakumoss_amd.group_hadamard(grad.contiguous(), ctx.group), None


torch.library.register_autograd("kohakumoss_amd::group_hadamard", _backward, setup_context=_setup, lib=_LIB)


def group_hadamard(x: Tensor, group: int) -> Tensor:
    """Differentiable `x . blockdiag(H_group)`; traces as one op under torch.compile."""
    check_group(x, group)
    return torch.ops.kohakumoss_amd.group_hadamard(x.contiguous(), int(group))
