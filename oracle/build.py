"""Build the oracle's C restatement (test infrastructure) with gcc.

    python -m oracle.build

writes `oracle/_build/liboracle_mxq.so`. The reference is pure Python (no C / C++ /
CUDA sources), so there is nothing of it to compile into `oracle/_ref/`.
"""

import ctypes
import subprocess
from pathlib import Path

HERE = Path(__file__).resolve().parent
OUT = HERE / "_build" / "liboracle_mxq.so"


def build(force: bool = True) -> Path:
    OUT.parent.mkdir(exist_ok=True)
    if OUT.exists() and not force:
        return OUT
    cmd = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC", "-std=c11", str(HERE / "mxq.c"), "-lm", "-o", str(OUT)]
    subprocess.run(cmd, check=True)
    return OUT


def load() -> ctypes.CDLL:
    """The built library with argument types set; builds it when it is missing."""
    lib = ctypes.CDLL(str(build(force=False)))
    c = ctypes
    lib.oracle_e4m3_from_f32.argtypes = [c.c_float]
    lib.oracle_e4m3_from_f32.restype = c.c_uint8
    lib.oracle_mx_scale_byte.argtypes = [c.c_float]
    lib.oracle_mx_scale_byte.restype = c.c_uint8
    lib.oracle_mx_quantize_bf16.argtypes = [c.c_void_p, c.c_long, c.c_long, c.c_long, c.c_long, c.c_void_p, c.c_void_p]
    lib.oracle_mx_quantize_bf16.restype = None
    lib.oracle_tensor_quantize_bf16.argtypes = [c.c_void_p, c.c_long, c.c_void_p, c.c_void_p]
    lib.oracle_tensor_quantize_bf16.restype = None
    return lib


if __name__ == "__main__":
    print(build())
