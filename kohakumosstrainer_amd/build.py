"""Build libkm_kernels.so (the HIP kernels + C ABI) for gfx950 with hipcc.

    python -m kohakumosstrainer_amd.build

The library is built in-tree (`kohakumosstrainer_amd/_lib/libkm_kernels.so`) so that it
travels with the source tree to a GPU machine; nothing is compiled at import time.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OUT_DIR = PKG / "_lib"
LIB = OUT_DIR / "libkm_kernels.so"
HOST_LIB = OUT_DIR / "libkm_hostcheck.so"
SOURCES = ("km_api.hip", "km_quant.hip", "km_gemm_fp8.hip", "km_gemm_fp8_w32.hip", "km_gemm_blocks.hip", "km_gemm_fused.hip", "km_wo_gemm.hip", "km_wo_dgrad.hip", "km_wo_fwd_bf16.hip", "km_wo_fwd_f16.hip", "km_wo_dgrad_bf16_i8.hip", "km_wo_dgrad_bf16_e4m3.hip", "km_wo_dgrad_bf16_e4m3b.hip",
           "km_wo_dgrad_f16_i8.hip", "km_wo_dgrad_f16_e4m3.hip", "km_wo_dgrad_f16_e4m3b.hip", "km_hadamard.hip", "km_probe.hip")
ARCH = "gfx950"
# packed fp32 instructions are switched off for every device translation unit
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc() -> str:
    path = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(path):
        raise RuntimeError("hipcc not found: the HIP kernels cannot be built here")
    return path


# Per-file additions. The block-recipe GEMM promotes MFMA results on the vector ALU: the MFMAs must
# write ordinary vector registers, or every partial sum is first copied out of an accumulation register.
EXTRA_FLAGS = {"km_gemm_blocks.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def _compile(src: Path, obj: Path) -> None:
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-c", str(src), "-o", str(obj), *DEVICE_FLAGS, *EXTRA_FLAGS.get(src.name, [])]
    done = subprocess.run(cmd, capture_output=True, text=True)
    if done.returncode:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{done.stderr[-6000:]}")


def build(verbose: bool = True) -> Path:
    """Compile every HIP source and link the shared library; returns its path."""
    OUT_DIR.mkdir(exist_ok=True)
    srcs = [CSRC / s for s in SOURCES if (CSRC / s).exists()]
    objs = [OUT_DIR / (s.stem + ".o") for s in srcs]
    # the slowest files first (each takes minutes): the fp8 GEMM, the weight-only forward kernels,
    # then the parts of the weight-only input gradient
    def weight(name: str) -> int:
        for rank, prefix in enumerate(("km_gemm_fp8.", "km_wo_fwd_", "km_wo_dgrad_bf16_e4m3.", "km_wo_dgrad_f16_e4m3.", "km_wo_dgrad_")):
            if name.startswith(prefix):
                return rank
        return 9

    order = sorted(range(len(srcs)), key=lambda i: weight(srcs[i].name))
    srcs, objs = [srcs[i] for i in order], [objs[i] for i in order]
    with ThreadPoolExecutor(max_workers=min(os.cpu_count() or 4, 12, len(srcs))) as pool:
        list(pool.map(lambda p: _compile(*p), zip(srcs, objs)))
    link = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", *map(str, objs), "-o", str(LIB)]
    done = subprocess.run(link, capture_output=True, text=True)
    if done.returncode:
        raise RuntimeError(f"link failed:\n{done.stderr[-4000:]}")
    if verbose:
        print(f"built {LIB}")
    build_hostcheck()
    return LIB


def build_hostcheck() -> Path:
    """The scalar numeric helpers compiled for the host with g++ (CPU bit checks)."""
    OUT_DIR.mkdir(exist_ok=True)
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", str(CSRC / "km_hostcheck.cpp"), "-o", str(HOST_LIB)]
    subprocess.run(cmd, check=True)
    return HOST_LIB


if __name__ == "__main__":
    try:
        build()
    except RuntimeError as err:
        sys.exit(str(err))
