"""Binding quantized linears to their compute device and dtype after a placement (reference
`src/kohakumoss/quant/bind.py:14-40`)."""

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


def work_device(device) -> torch.device:
    """Where weights are quantized: the compute device when it is a GPU."""
    device = torch.device(device)
    return device if device.type == "cuda" else torch.device("cpu")
