"""CPU build of the kernels' scalar helpers (`csrc/km_numeric.h` compiled with g++)
checked bit by bit against the oracle: the same functions the HIP kernels inline."""

import ctypes

import numpy as np
import pytest
import torch

from kohakumosstrainer_amd import build as km_build
from oracle import formats


@pytest.fixture(scope="module")
def host():
    path = km_build.HOST_LIB if km_build.HOST_LIB.exists() else km_build.build_hostcheck()
    lib = ctypes.CDLL(str(path))
    lib.km_host_e4m3_encode_many.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p]
    lib.km_host_mx_biased_many.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p]
    lib.km_host_bf16_many.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_void_p]
    lib.km_host_e4m3_decode.argtypes = [ctypes.c_uint]
    lib.km_host_e4m3_decode.restype = ctypes.c_float
    lib.km_host_mx_inverse_scale.argtypes = [ctypes.c_uint]
    lib.km_host_mx_inverse_scale.restype = ctypes.c_float
    return lib


def _all_bf16():
    return torch.arange(65536, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16).float()


def _encode(lib, v: torch.Tensor) -> torch.Tensor:
    v = v.contiguous()
    out = torch.empty(v.numel(), dtype=torch.uint8)
    lib.km_host_e4m3_encode_many(v.data_ptr(), v.numel(), out.data_ptr())
    return out


def test_e4m3_encode_equals_torch_cast(host):
    g = torch.Generator().manual_seed(0)
    pools = [_all_bf16() * s for s in (1.0, 0.37, 2.0**-9, 5.0, 1 / 448)]
    pools.append(torch.randn(200000, generator=g) * torch.logspace(-12, 3, 200000))
    pools.append(torch.tensor([0.0, -0.0, 2.0**-10, -(2.0**-10), 3 * 2.0**-10, 2.0**-6, 448.0, 464.0, 1e30, float("inf"), -float("inf")]))
    for v in pools:
        v = v.float()
        want = v.clamp(-448, 448).to(formats.E4M3).view(torch.uint8)
        got = _encode(host, v)
        nan = torch.isnan(v)
        assert torch.equal(got[~nan], want[~nan])
        assert bool(((got[nan] & 0x7F) == 0x7F).all())
        assert torch.equal(got[nan] & 0x80, (v[nan].view(torch.int32) >> 24).to(torch.uint8) & 0x80)


def test_e4m3_decode_is_exact(host):
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(formats.E4M3).float()
    got = torch.tensor([host.km_host_e4m3_decode(int(c)) for c in codes])
    keep = ~torch.isnan(want)
    assert torch.equal(got[keep], want[keep]) and bool(torch.isnan(got[~keep]).all())


def test_mx_exponent_and_inverse_equal_oracle(host):
    g = torch.Generator().manual_seed(1)
    amax = torch.cat([
        _all_bf16().abs(),
        (1 + torch.rand(50000, generator=g)) * 2.0 ** torch.randint(-126, 127, (50000,), generator=g).float(),
        torch.tensor([0.0, 1e-30, 1.75, 1.75 * (1 + 2.0**-7), 448.0, float("inf")]),
    ]).float()
    amax = amax[~torch.isnan(amax)].contiguous()
    out = torch.empty(amax.numel(), dtype=torch.uint8)
    host.km_host_mx_biased_many(amax.data_ptr(), amax.numel(), out.data_ptr())
    want = formats.mx_biased_exponent(amax)
    assert torch.equal(out.int(), want)
    for b in (0, 19, 119, 127, 200, 248, 253):
        assert host.km_host_mx_inverse_scale(b) == formats.pow2_from_biased(torch.tensor([b]), -1).item()


def test_bf16_rounding_equals_torch(host):
    g = torch.Generator().manual_seed(2)
    v = torch.cat([torch.randn(100000, generator=g) * torch.logspace(-20, 20, 100000), torch.tensor([0.0, -0.0, 1.00390625, 1.01171875, float("inf")])]).float().contiguous()
    out = torch.empty(v.numel(), dtype=torch.int16)
    host.km_host_bf16_many(v.data_ptr(), v.numel(), out.data_ptr())
    assert torch.equal(out, v.to(torch.bfloat16).view(torch.int16))
