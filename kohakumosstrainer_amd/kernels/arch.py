"""Arch table: a torch device -> the `Arch` entry dispatch and support checks key on.

The reference's table (`src/kohakumoss_kernels/hardware/arch.py:7-53`) is the CUDA sm ladder
plus XPU and CPU; a ROCm device would fall onto `sm90` there through
`torch.cuda.get_device_capability`. Here a ROCm device is identified by its gfx name:
`gfx950` (MI350X / MI355X, CDNA4) is the entry the HIP backend serves; any other AMD GPU gets
an entry of kind "hip" that no backend claims.
"""

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Arch:
    """One arch-table entry. `name` is `gfx950`, another gfx name, or `cpu`; `sm` is kept for
    interface parity with the CUDA ladder (95 for gfx950, which is what ROCm reports)."""

    name: str
    sm: int
    kind: str
    has_bf16: bool
    has_fp8: bool
    tensor_core_fp16: bool
    has_mx: bool = False

    @property
    def is_gpu(self) -> bool:
        return self.kind == "hip"


CPU = Arch("cpu", 0, "cpu", True, False, False)
GFX950 = Arch("gfx950", 95, "hip", True, True, True, has_mx=True)
_BY_NAME = {"gfx950": GFX950}
_FORCED: list[Arch] = []


def _gfx_name(device: torch.device) -> str:
    props = torch.cuda.get_device_properties(device)
    return str(getattr(props, "gcnArchName", "") or "").split(":")[0]


def arch_of(device: torch.device | str) -> Arch:
    """Arch-table entry of `device`."""
    if _FORCED:
        return _FORCED[-1]
    device = torch.device(device)
    if device.type != "cuda":
        return CPU
    name = _gfx_name(device) if torch.version.hip else ""
    if name in _BY_NAME:
        return _BY_NAME[name]
    major, minor = torch.cuda.get_device_capability(device)
    return Arch(name or f"sm{major}{minor}", major * 10 + minor, "hip" if torch.version.hip else "cuda", True, False, True)


class forced_arch:
    """Context manager: `arch_of` answers `arch` inside (tests of the dispatch on a host
    without the device)."""

    def __init__(self, arch: Arch):
        self.arch = arch

    def __enter__(self):
        _FORCED.append(self.arch)
        return self.arch

    def __exit__(self, *exc):
        _FORCED.pop()
