"""Binding quantized linears to their compute device and dtype after a placement (reference
`src/kohakumoss/quant/bind.py:14-40`; W4A8 and embedding bases are outside this path)."""

import torch
from torch import nn

from kohakumosstrainer_amd.quant.compute import ComputeWeight
from kohakumosstrainer_amd.quant.weights import QuantWeight


def rebind_quant(module: nn.Module, device, dtype, autograd: bool = True) -> None:
    """Bind every quantized base to (device, dtype); `autograd=False` binds fp8-compute bases
    of a model that never runs backward to the gradient-free op."""
    for m in module.modules():
        if isinstance(m, ComputeWeight):
            m.bind(dtype, device, autograd=autograd)
        elif isinstance(m, QuantWeight):
            m.bind(dtype, device)


def set_int8_compute(module: nn.Module, dgrad: str) -> int:
    """Select int8 compute (the `int8_linear` op with input-gradient mode `dgrad`) on every int8
    base inside `module`; it takes effect at their next `bind`. Returns how many were switched."""
    switched = [m for m in module.modules() if isinstance(m, QuantWeight) and m.fmt == "int8"]
    for m in switched:
        m.int8_dgrad = dgrad
    return len(switched)


def work_device(device) -> torch.device:
    """Where weights are quantized: the compute device when it is a GPU."""
    device = torch.device(device)
    return device if device.type == "cuda" else torch.device("cpu")
