"""Regular-Hadamard rotation over groups of the last dim (ConvRot).

H_g is the normalised Kronecker power of H4 = [[1,1,1,-1],[1,1,-1,1],[1,-1,1,1],[-1,1,1,1]] for
g = 4^j: symmetric and involutory, entries +-2^-j (exact in fp16 / bf16). `group_hadamard(x, g)`
is x times blockdiag(H_g) over the last dim, its own inverse and its own adjoint (so its
backward is the rotation of the incoming gradient). On a GPU, bf16 / fp16 tensors go through the
hand-written HIP butterfly kernel; everything else through torch ops. Interface follows
reference `src/kohakumoss_kernels/hadamard.py:31-101` and the `group_hadamard` op of
`backends/triton/hadamard.py:108-152`.
"""

from functools import cache

import torch
from torch import Tensor

H4 = ((1, 1, 1, -1), (1, 1, -1, 1), (1, -1, 1, 1), (-1, 1, 1, 1))
GROUPS = (4, 16, 64, 256, 1024)
HALF = (torch.float16, torch.bfloat16)


def stages(group: int) -> int:
    """j of g = 4^j; ValueError unless `group` is a power of 4 of at least 4."""
    j, g = 0, int(group)
    while g > 1 and g % 4 == 0:
        g //= 4
        j += 1
    if g != 1 or j == 0:
        raise ValueError(f"Hadamard group {group} is not a power of 4 >= 4")
    return j


def check_group(x: Tensor, group: int) -> int:
    """The stage count of `group`; ValueError when it does not divide x's last dim."""
    j = stages(group)
    if x.shape[-1] % group:
        raise ValueError(f"last dim {x.shape[-1]} is not a multiple of group {group}")
    return j


@cache
def _matrix(group: int, dtype: torch.dtype, device: torch.device) -> Tensor:
    seed = torch.tensor(H4, dtype=torch.float32)
    h = seed
    for _ in range(stages(group) - 1):
        h = torch.kron(h, seed)
    return (h / float(group) ** 0.5).to(device=device, dtype=dtype)


def hadamard_matrix(group: int, dtype: torch.dtype = torch.float32, device="cpu") -> Tensor:
    """H_group [group, group] in `dtype` on `device` (cached; do not modify)."""
    return _matrix(int(group), dtype, torch.device(device))


def _butterflies(x: Tensor, group: int, j: int) -> Tensor:
    """j fp32 4-point stages, most significant base-4 digit first: y_k = sum(x) - 2 x_(3-k),
    the sum taken in index order."""
    v = x.float()
    rows = v.numel() // group
    for a in range(j):
        x0, x1, x2, x3 = v.reshape(rows * 4**a, 4, group // 4 ** (a + 1)).unbind(1)
        total = ((x0 + x1) + x2) + x3
        v = torch.stack([total - 2.0 * x3, total - 2.0 * x2, total - 2.0 * x1, total - 2.0 * x0], 1)
    return (v.reshape(x.shape) * 2.0**-j).to(x.dtype)


def group_hadamard_eager(x: Tensor, group: int) -> Tensor:
    """x [..., K] -> x . blockdiag(H_group) in x's dtype with torch ops: a 16-bit matmul with H
    (fp32 accumulation) for fp16 / bf16, fp32 butterflies for any other dtype."""
    j = check_group(x, group)
    if x.dtype in HALF:
        return (x.reshape(-1, group) @ hadamard_matrix(group, x.dtype, x.device)).reshape(x.shape)
    return _butterflies(x, group, j)


def rotate_2d(x: Tensor, group: int) -> Tensor:
    """[R, K] -> [R, K] rotated, no autograd: the HIP kernel for 16-bit device tensors, torch ops
    otherwise."""
    check_group(x, group)
    if x.device.type == "cuda" and x.dtype in HALF:
        from kohakumosstrainer_amd import native

        return native.group_hadamard(x, group)
    with torch.no_grad():
        return group_hadamard_eager(x, group)


@torch.library.custom_op("kohakumoss_amd::group_hadamard", mutates_args=())
def _op(x: Tensor, group: int) -> Tensor:
    return rotate_2d(x, group)


@_op.register_fake
def _(x, group):
    return torch.empty_like(x)


def _setup(ctx, inputs, output):
    ctx.group = inputs[1]


_op.register_autograd(lambda ctx, g: (_op(g.contiguous(), ctx.group), None), setup_context=_setup)


def group_hadamard(x: Tensor, group: int) -> Tensor:
    """x [..., K] -> x . blockdiag(H_group), differentiable (the backward is the same rotation)."""
    shape = x.shape
    return _op(x.reshape(-1, shape[-1]).contiguous(), int(group)).view(shape)
