"""Oracle (test infrastructure): the group Hadamard rotation (ConvRot) on the CPU with torch.

H_g is the normalised Kronecker power of H4 = [[1,1,1,-1],[1,1,-1,1],[1,-1,1,1],[-1,1,1,1]] for
g = 4^j: symmetric, its own inverse, entries +-2^-j. Restates reference
`src/kohakumoss_kernels/hadamard.py`: `stages` :31-40, the matrix :49-56, the fp32 butterflies
:71-82 (what the reference's GPU kernel computes, `backends/triton/hadamard.py:28-49`) and the
16-bit eager form, a matmul with H in the input's dtype :85-101.

Pinned by `tests/test_oracle_hadamard.py`: an independent fp64 torch.kron construction
(reference `tests/_util/hadamard_ref.py:8-24`), symmetry and H H = I, exact equality with it on
integer inputs (every sum is exact there) in every group size, the sign rule "flip where the
base-4 digits of row and column add to 3", closeness on random inputs; a transposed digit
order, a Sylvester seed and a missing scale must fail. No function here is "parity unpinned".
"""

import torch
from torch import Tensor

H4 = ((1, 1, 1, -1), (1, 1, -1, 1), (1, -1, 1, 1), (-1, 1, 1, 1))
GROUPS = (4, 16, 64, 256, 1024)


def stages(group: int) -> int:
    """j of group = 4^j; ValueError unless group is a power of 4 of at least 4."""
    j, g = 0, int(group)
    while g > 1 and g % 4 == 0:
        g //= 4
        j += 1
    if g != 1 or j == 0:
        raise ValueError(f"Hadamard group {group} is not a power of 4 >= 4")
    return j


def check_group(x: Tensor, group: int) -> int:
    j = stages(group)
    if x.shape[-1] % group:
        raise ValueError(f"last dim {x.shape[-1]} is not a multiple of group {group}")
    return j


def matrix(group: int, dtype: torch.dtype = torch.float32) -> Tensor:
    """H_group: the j-fold Kronecker power of H4 times 2^-j."""
    j = stages(group)
    seed = torch.tensor(H4, dtype=torch.float32)
    h = seed
    for _ in range(j - 1):
        h = torch.kron(h, seed)
    return (h * 2.0**-j).to(dtype)


def butterflies(x: Tensor, group: int) -> Tensor:
    """x . blockdiag(H_group) by j fp32 stages of 4-point butterflies, the most significant
    base-4 digit of the index first: y_k = ((x0 + x1) + x2) + x3 - 2 x_(3-k); then 2^-j and one
    rounding to x's dtype."""
    j = check_group(x, group)
    v = x.to(torch.float32)
    rows = v.numel() // group
    for a in range(j):
        x0, x1, x2, x3 = v.reshape(rows * 4**a, 4, group // 4 ** (a + 1)).unbind(1)
        total = ((x0 + x1) + x2) + x3
        v = torch.stack([total - 2.0 * x3, total - 2.0 * x2, total - 2.0 * x1, total - 2.0 * x0], 1)
    return (v.reshape(x.shape) * 2.0**-j).to(x.dtype)


def rotate(x: Tensor, group: int) -> Tensor:
    """The reference's eager rotation: 16-bit inputs multiply by H in their own dtype (fp32
    accumulation inside the matmul), anything else goes through the butterflies."""
    check_group(x, group)
    if x.dtype in (torch.float16, torch.bfloat16):
        return (x.reshape(-1, group) @ matrix(group, x.dtype)).reshape(x.shape)
    return butterflies(x, group)
