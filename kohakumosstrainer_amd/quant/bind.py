"""Re-binding the quantized bases of a model after it moved or changed dtype, and switching int8
bases to the int8 compute linear. Replaces reference `src/kohakumoss/quant/bind.py`."""

from __future__ import annotations

import torch
from torch import nn

from kohakumosstrainer_amd.quant.compute import ComputeWeight
from kohakumosstrainer_amd.quant.weights import QuantWeight


def work_device(device) -> torch.device:
    """Where quantization work runs for a model headed to `device`: that device when it is a GPU
    that is there, else the host."""
    device = torch.device(device)
    return device if device.type == "cuda" and torch.cuda.is_available() else torch.device("cpu")


def rebind_quant(module: nn.Module, device, dtype, autograd: bool = True) -> None:
    """Bind every quantized base under `module` for `(device, dtype)`: each resolves its op once
    here instead of on its first call."""
    for child in module.modules():
        if isinstance(child, ComputeWeight):
            child.bind(dtype, device, autograd=autograd)
        elif isinstance(child, QuantWeight):
            child.bind(dtype, device)


def set_int8_compute(module: nn.Module, dgrad: str) -> int:
    """Route every int8 weight-only base under `module` through the int8 compute linear with the
    given input-gradient mode; returns how many were switched."""
    switched = 0
    for child in module.modules():
        if isinstance(child, QuantWeight) and child.fmt == "int8":
            child.int8_dgrad, child._call = dgrad, None
            switched += 1
    return switched
