"""The weight-only input gradient through the entry point that allocates nothing
(`km_wo_gemm_dgrad_static`: transposed codes in the library's static device array) against the
entry point that takes a workspace (`km_wo_gemm_dgrad`), through the C ABI: equal bit for bit,
on two calls in a row, the second with a smaller operand (the array keeps the first call's
bytes), and again with the other code format. (The transposing path has one tile shape; `config`
is range-checked and otherwise unused there.) After one warm-up call on the device, which looks the
array's address up, a call changes neither torch's allocator statistics nor the device's free memory."""

import pytest
import torch

from kohakumosstrainer_amd import native



def operands(m, n, k, fmt, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    dy = torch.randn(m, n, generator=g).to(dtype).cuda()
    if fmt == "int8":
        q = torch.randint(-127, 128, (n, k), generator=g).to(torch.int8).cuda()
    else:
        q = (torch.randn(n, k, generator=g) * 60).clamp_(-448, 448).to(torch.float8_e4m3fn).cuda()
    scale = (torch.rand(n, generator=g) * 1e-2 + 1e-4).cuda()
    return dy, q, scale


def both(dy, q, scale, config):
    want = native.wo_gemm_dgrad_workspace(dy, q, scale, config)
    out = torch.full_like(want, float("nan"))
    got = native.wo_gemm_dgrad_static(dy, q, scale, out, config)
    assert got.data_ptr() == out.data_ptr()
    return got, want


@pytest.mark.gpu
def test_static_workspace_dgrad_equals_workspace_dgrad_on_consecutive_calls():
    for (m, n, k), fmt, dtype, config in (
        ((512, 768, 1024), "int8", torch.bfloat16, 0),
        ((200, 136, 264), "int8", torch.bfloat16, 0),  # smaller: stale bytes of the first call lie beyond it
        ((384, 512, 640), "fp8", torch.float16, 3),
        ((65, 72, 40), "fp8", torch.float16, 3),
        ((33, 50, 30), "int8", torch.bfloat16, 0),  # K % 8 != 0: the element-wise kernel
    ):
        dy, q, scale = operands(m, n, k, fmt, dtype, seed=m)
        got, want = both(dy, q, scale, config)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (m, n, k, fmt)
        del dy, q, scale, got, want
    # The entry point takes no device memory: neither from torch's allocator nor from the driver
    # (`mem_get_info` is the device's own free-byte count and would show a hipMalloc of the 32 KiB
    # this call would need as a 2 MiB granule). The calls above were the warm-up.
    dy, q, scale = operands(128, 256, 128, "int8", torch.bfloat16, seed=9)
    out = torch.empty(128, 128, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()
    held, reserved, free = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    for _ in range(3):
        native.wo_gemm_dgrad_static(dy, q, scale, out, 0)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held and torch.cuda.memory_reserved() == reserved
    assert torch.cuda.mem_get_info()[0] == free, "the device's free memory moved across calls of the no-allocation entry point"


@pytest.mark.gpu
def test_static_dgrad_under_graph_capture_after_a_warm_up_call():
    """The documented use: one call outside capture (it looks up the array's per-device address under
    a lock), then the call is captured; every replay must equal the eager result, with eager work
    and synchronisation between the replays."""
    dy, q, scale = operands(256, 384, 512, "int8", torch.bfloat16, seed=21)
    want = native.wo_gemm_dgrad_workspace(dy, q, scale, 0)
    out = torch.zeros_like(want)
    native.wo_gemm_dgrad_static(dy, q, scale, out, 0)  # warm-up, outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            native.wo_gemm_dgrad_static(dy, q, scale, out, 0)
    torch.cuda.current_stream().wait_stream(side)
    for i in range(3):
        out.fill_(float("nan"))
        dy2, q2, scale2 = operands(96, 64, 128, "int8", torch.bfloat16, seed=30 + i)  # eager work that rewrites the array
        native.wo_gemm_dgrad_static(dy2, q2, scale2, torch.empty(96, 128, dtype=torch.bfloat16, device="cuda"), 0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), f"replay {i}"


def test_static_workspace_rejects_operands_beyond_its_size():
    """A host-side check: no pointer is read and no device is touched."""
    lib = native.load()
    n, k = 16384, 4097  # 16384 * 4097 > 64 Mi codes
    rc = lib.km_wo_gemm_dgrad_static(None, None, None, None, 8, n, k, native.KM_Q_INT8, native.KM_BF16, 0, None)
    assert rc < 0 and b"exceed the static workspace" in lib.km_last_error()
