"""The C-ABI library loads on a host without a GPU and exports every symbol that
`include/km_kernels.h` declares (no compute calls here)."""

import ctypes
import re
from pathlib import Path

from kohakumosstrainer_amd import native

ROOT = Path(__file__).resolve().parents[1]


def declared_symbols() -> list[str]:
    text = (ROOT / "include" / "km_kernels.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(km_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    lib = native.load()
    names = declared_symbols()
    assert len(names) >= 11, names
    for name in names:
        assert hasattr(lib, name), f"{name} declared in km_kernels.h but not exported"
    assert set(native.EXPORTS) == set(names), (set(native.EXPORTS) ^ set(names))


def test_abi_version_and_config_catalogue():
    lib = native.load()
    assert lib.km_abi_version() == 1
    for kernel in (native.KERNEL_GEMM_MX, native.KERNEL_GEMM_FP8, native.KERNEL_WO_FWD, native.KERNEL_WO_DGRAD, native.KERNEL_GEMM_BLOCKS):
        cfgs = native.configs(kernel)
        assert cfgs and all({"id", "bm", "bn", "bk"} <= set(c) for c in cfgs)
        assert [c["id"] for c in cfgs] == list(range(len(cfgs)))
    assert lib.km_num_configs(99) < 0 and b"unknown kernel" in lib.km_last_error()
    buf = ctypes.create_string_buffer(64)
    assert lib.km_config_desc(native.KERNEL_GEMM_MX, 99, buf, 64) < 0


def test_argument_errors_are_reported_without_a_gpu():
    lib = native.load()
    assert lib.km_quant_mx(None, 4, 48, 48, 1, native.KM_BF16, None, None, None, None) < 0
    assert b"multiple of 32" in lib.km_last_error()
    assert lib.km_gemm_mx(None, None, None, None, None, None, 64, 64, 96, native.KM_BF16, 0, 0, None) < 0
    assert b"multiple of 128" in lib.km_last_error()
    assert lib.km_quant_blocks(None, 4, 200, 200, 1, native.KM_BF16, native.ROLE_ACT, None, None, None, None) < 0
    assert b"multiple of 128" in lib.km_last_error()
    assert lib.km_quant_blocks(None, 4, 256, 256, 1, native.KM_BF16, 7, None, None, None, None) < 0
    assert b"role" in lib.km_last_error()
    assert lib.km_gemm_fp8_blocks(None, None, None, None, None, None, 64, 64, 256, native.KM_BF16, 5, 0, None) < 0
    assert b"scale layout" in lib.km_last_error()
    assert lib.km_gemm_fp8_blocks(None, None, None, None, None, None, 64, 64, 256, native.KM_BF16, native.SCALES_KMAJOR, 9, None) < 0
    assert b"config" in lib.km_last_error()
    for fused in (lib.km_gemm_mx_fused, lib.km_gemm_fp8_rows_fused, lib.km_gemm_fp8_blocks_fused):
        assert fused(None, 256, None, None, None, None, 8, 48, 256, native.KM_BF16, None) < 0
        assert b"multiple of 32" in lib.km_last_error()
        assert fused(None, 200, None, None, None, None, 8, 64, 200, native.KM_BF16, None) < 0
        assert b"multiple of 128" in lib.km_last_error()
        assert fused(None, 256, None, None, None, None, 8, 64, 256, native.KM_BF16, None) < 0
        assert b"null pointer" in lib.km_last_error()
        assert fused(None, 256, None, None, None, None, 0, 64, 256, native.KM_BF16, None) == 0
    assert lib.km_scales_packed_bytes(16384, 3072) == 16384 * 96
    assert lib.km_scales_packed_bytes(100, 256) == 2 * 1 * 512
    assert lib.km_scales_packed_bytes(100, 96) == -1


def test_weight_only_path_query_names_the_slow_kernel():
    """`km_wo_gemm_path` only looks at extents and pointer alignment: no GPU needed."""
    lib = native.load()
    tiled, slow = 0, 1
    a, q, s, c = 4096, 8192, 1024, 16384  # stand-in addresses, 16-byte aligned
    assert lib.km_wo_gemm_path(native.WO_FWD, a, q, s, c, 64, 256, 512) == tiled
    assert lib.km_wo_gemm_path(native.WO_FWD, a, q, s, c, 64, 256, 516) == slow  # K % 8
    assert lib.km_wo_gemm_path(native.WO_FWD, a + 2, q, s, c, 64, 256, 512) == slow  # alignment
    assert lib.km_wo_gemm_path(native.WO_DGRAD_W16, a, q, s, c, 64, 256, 512) == tiled
    assert lib.km_wo_gemm_path(native.WO_DGRAD_W16, a, q, s, c, 64, 250, 512) == slow  # N % 8
    assert lib.km_wo_gemm_path(native.WO_DGRAD_W16, a, q, s, c, 64, 256, 510) == slow  # K % 4
    assert lib.km_wo_gemm_path(native.WO_DGRAD_W16, a, q, s, c, 300, 2**22, 8) == slow  # 256 rows of dy pass 2^31 bytes
    assert lib.km_wo_gemm_path(native.WO_DGRAD_TRANSPOSED, a, q, s, c, 64, 256, 510) == tiled
    assert lib.km_wo_gemm_path(native.WO_DGRAD_TRANSPOSED, a, q, s, c, 64, 2**22, 8) == slow
    assert lib.km_wo_gemm_path(9, a, q, s, c, 1, 8, 8) < 0


def test_wrappers_refuse_host_tensors():
    import pytest
    import torch

    with pytest.raises(ValueError, match="device tensors"):
        native.quant_mx(torch.zeros(4, 64, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="device tensors"):
        native.wo_gemm_fwd(torch.zeros(4, 64, dtype=torch.bfloat16), torch.zeros(8, 64, dtype=torch.int8), torch.ones(8), None)
