"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one MXFP8 fused-QKV linear forward at the headline shape: activations
bf16 [16384, 3072] are quantized per 32-block (HIP quantizer) and multiplied with the
pre-quantized weight [9216, 3072] on the block-scaled MFMA with bias and bf16 output
(HIP GEMM). All inputs are resident in HBM before the timed region. Prints ONE JSON
line: whole-step TFLOP/s, the GEMM kernel's roofline fraction against the dense fp8
MFMA peak (from its own event-timed launches), the row- and column-wise quantizer
bandwidth against the HBM peak, and the CPU oracle timed on this host's cores on a
bounded sample of the same workload.
"""

import argparse
import json
import os
import sys
import time

import torch

M, K, N = 16384, 3072, 9216
FP8_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 / MXFP8 MFMA
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
GEMM_FLOP = 2 * M * N * K
QUANT_BYTES = M * K * 2 + M * K + M * K // 32  # bf16 read + codes + scale bytes, per direction
CPU_SAMPLE_ROWS = 16384  # the whole workload: this host's cores finish it in seconds
# HBM-side bytes of one launch of the headline GEMM come from the profiler's FETCH_SIZE / WRITE_SIZE
# counters, each scaled by what the same counter reads for a plain device copy of known size. They
# cannot be read while timing, so the committed summary of those two profiler runs carries them in a
# line `headline_gemm_traffic_bytes: <integer>` that is read here; without the file the field is null.
TRAFFIC_PROFILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "gemm_fp8_and_quant_M16384_K3072_N9216_pmc.txt")


def profiled_traffic_bytes():
    try:
        with open(TRAFFIC_PROFILE) as fh:
            for text in fh:
                if text.startswith("headline_gemm_traffic_bytes:"):
                    return int(text.split(":", 1)[1].split()[0])
    except (OSError, ValueError):
        pass
    return None


def synthetic(device):
    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    g.manual_seed(1)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    bias = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16)
    return x.to(device), w.to(device), bias.to(device)


def event_ms(fn, reps: int) -> float:
    """Average device ms of `reps` back-to-back calls of `fn`, by events on the stream the
    kernels are launched on (torch's current stream)."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / reps


def warm_event_ms(fn, reps: int) -> float:
    """`event_ms` after 50 ms of the same calls."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.05:
        fn()
    return event_ms(fn, reps)


def cpu_baseline(x, wq, ws, bias):
    """The oracle's eager forward (quantize, dequantize both operands, bf16 linear) on the
    first CPU_SAMPLE_ROWS rows of the same activations, all host threads, best of 3."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle import linear

    xs = x[:CPU_SAMPLE_ROWS].cpu()
    wq_c, ws_c, b_c = wq.cpu(), ws.cpu(), bias.cpu()
    best, total, reps = float("inf"), 0.0, 0
    while total < 12.0 and reps < 200:  # about 12 s of CPU work
        t = time.perf_counter()
        linear.fp8_forward(xs, wq_c, ws_c, None, b_c, "mx")
        dt = time.perf_counter() - t
        best, total, reps = min(best, dt), total + dt, reps + 1
    flop = 2 * CPU_SAMPLE_ROWS * N * K
    return {
        "value": flop / best / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"{CPU_SAMPLE_ROWS} of {M} rows, full W [{N},{K}]: quantize x, dequantize x and W, bf16 linear + bias (torch CPU), best of {reps} passes ({best:.2f} s each, {total:.0f} s in all)",
        "other_configs": cpu_other_configs(xs),
    }


def _best_of(fn, budget_s: float, max_reps: int = 50):
    best, total, reps = float("inf"), 0.0, 0
    while total < budget_s and reps < max_reps:
        t = time.perf_counter()
        fn()
        dt = time.perf_counter() - t
        best, total, reps = min(best, dt), total + dt, reps + 1
    return best, total, reps


def cpu_other_configs(x_host):
    """The oracle on the host for the two other benchmark configurations that have a CPU leg: the
    int8 weight-only forward at M4096 K3072 N3072 (the configuration the reference defines on its CPU
    torch path) and the standalone MXFP8 quantizer on bf16 [16384, 3072], row- and column-wise. About
    4 s of CPU work each, all host threads."""
    from oracle import formats, linear

    cores = torch.get_num_threads()
    out = {}
    g = torch.Generator().manual_seed(7)
    m, k, n = 4096, 3072, 3072
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    q = torch.randint(-127, 128, (n, k), generator=g).to(torch.int8)
    scale = torch.randn(n, generator=g).abs() * 0.02 / 127 + 1e-6
    bias = torch.randn(n, generator=g) * 0.01
    best, total, reps = _best_of(lambda: linear.wo_forward(x, q, scale, bias.to(torch.bfloat16)), 4.0)
    out["wo_int8_M4096_K3072_N3072_fwd"] = {"value": 2 * m * n * k / best / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
                                            "sample": f"the whole configuration: dequantize W to bf16, bf16 linear + bias (torch CPU), best of {reps} passes ({best:.3f} s each)"}
    for name, view in (("mx_quantize_rows_16384x3072", x_host), ("mx_quantize_cols_16384x3072", x_host.t())):
        best, total, reps = _best_of(lambda: formats.quantize(view, "mx"), 4.0)
        out[name] = {"value": QUANT_BYTES / best / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
                     "sample": f"the whole bf16 [{M},{K}] tensor, {QUANT_BYTES} algorithmic bytes, best of {reps} passes ({best:.3f} s each)"}
    return out


def mfma_ceiling(a_codes, b_codes):
    """What the card's clocks sustain on the matrix pipes: the block-scaled fp8 MFMA out of registers
    (one wavefront per SIMD on every compute unit, the GEMM's 64 accumulator tiles and 8 + 8 operand
    fragments taken from the benchmark's own codes, no loads, no LDS, no barriers), about 60 ms per
    launch after a launch of the same length to settle the clocks. The implied clock assumes the
    pipe's nominal 8192 flop per cycle and compute unit (dense fp8)."""
    from kohakumosstrainer_amd import native

    trips = 50_000  # 64 MFMAs of 32 cycles each per trip: about 1.1 us
    native.mfma_ceiling_probe(a_codes, b_codes, trips)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    flop = native.mfma_ceiling_probe(a_codes, b_codes, trips)
    end.record()
    end.synchronize()
    ms = start.elapsed_time(end)
    tflops = flop / ms / 1e9
    cus = torch.cuda.get_device_properties(a_codes.device).multi_processor_count
    return {"TFLOPs": tflops, "ms": ms, "frac_of_nominal": tflops / FP8_PEAK_TFLOPS, "implied_clock_GHz": tflops * 1e12 / (cus * 8192) / 1e9,
            "compute_units": cus, "kernel": "mfma_ceiling_kernel: v_mfma_scale_f32_16x16x128_f8f6f4 from registers only, 4 wavefronts per compute unit"}


def other_configs(dev, reps):
    """Device time of the other kernels of the path at their benchmark shapes (event-timed,
    back to back): weight-only int8 / e4m3 GEMMs, the frozen-base MXFP8 forward + input
    gradient of the adapter-training shape, and the row-recipe, block-recipe fp8 and int8 compute
    linears at the headline shape."""
    from kohakumosstrainer_amd import native

    event_ms = warm_event_ms  # each measurement here starts from sustained clocks

    g = torch.Generator(device="cpu").manual_seed(0)
    out = {}
    for name, (m, k, n), fmt in (("wo_int8_M4096_K3072_N3072", (4096, 3072, 3072), "int8"), ("wo_e4m3_M8192_K3072_N12288", (8192, 3072, 12288), "fp8")):
        x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(dev)
        if fmt == "int8":
            # frozen int8 base: codes uniform in [-127, 127], scale |N(0,0.02)|/127 + 1e-6 per output row
            q = torch.randint(-127, 128, (n, k), generator=g).to(torch.int8).to(dev)
            scale = (torch.randn(n, generator=g).abs() * 0.02 / 127 + 1e-6).to(dev)
        else:
            # per-tensor e4m3 base: W ~N(0,0.02) in bf16, one scale amax/448 broadcast to the rows
            w16 = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16).to(dev)
            q, s1 = native.quant_tensor(w16)
            scale = s1.reshape(1).expand(n).contiguous()
            del w16
        bias = (torch.randn(n, generator=g) * 0.01).to(torch.bfloat16).to(dev)
        dy = torch.randn(m, n, generator=g).to(torch.bfloat16).to(dev)
        # the tile configuration per direction as the tuning table would settle it: fastest of all
        f_ms, d_ms = {}, {}
        for cfg in range(len(native.configs(native.KERNEL_WO_FWD))):
            native.wo_gemm_fwd(x, q, scale, bias, cfg)
            native.wo_gemm_dgrad(dy, q, scale, cfg)
            f_ms[cfg] = event_ms(lambda: native.wo_gemm_fwd(x, q, scale, bias, cfg), reps)
            d_ms[cfg] = event_ms(lambda: native.wo_gemm_dgrad(dy, q, scale, cfg), reps)
        (fc, f), (dc, d) = min(f_ms.items(), key=lambda kv: kv[1]), min(d_ms.items(), key=lambda kv: kv[1])
        flop = 2 * m * n * k
        # a rotated base (ConvRot, groups of 256) adds one rotation pass over x in forward and one over dx in the input gradient
        native.group_hadamard(x, 256)
        r = event_ms(lambda: native.group_hadamard(x, 256), reps)
        out[name] = {"fwd_ms": f, "fwd_TFLOPs": flop / f / 1e9, "fwd_config": fc, "dgrad_ms": d, "dgrad_TFLOPs": flop / d / 1e9, "dgrad_config": dc,
                     "peak_TFLOPs": 2500.0, "note": "dgrad reads the codes as stored: no transposed copy, no workspace",
                     "rotation_pass_ms": r, "rotation_share_of_rotated_fwd": r / (r + f), "rotation_share_of_rotated_dgrad": r / (r + d)}
    m, k, n = 2048, 4096, 12288
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    dy = (torch.randn(m, n, generator=g) * 0.01).to(torch.bfloat16).to(dev)
    wq, _, wsp = native.quant_mx(w, natural=False, packed=True)
    wtq, _, wtsp = native.quant_mx(w.t(), natural=False, packed=True)

    def fwd(cfg):
        xq, _, xsp = native.quant_mx(x, natural=False, packed=True)
        return native.gemm_mx(xq, xsp, wq, wsp, None, torch.bfloat16, cfg, packed=True)

    def dgrad(cfg):
        gq, _, gsp = native.quant_mx(dy, natural=False, packed=True)
        return native.gemm_mx(gq, gsp, wtq, wtsp, None, torch.bfloat16, cfg, packed=True)

    # the tile configuration per direction as the tuning table would settle it: fastest of all
    best = {}
    for name, fn in (("fwd", fwd), ("dgrad", dgrad)):
        times = {}
        for cfg in range(len(native.configs(native.KERNEL_GEMM_MX))):
            fn(cfg)
            times[cfg] = event_ms(lambda: fn(cfg), reps)
        best[name] = min(times.items(), key=lambda kv: kv[1])
    flop = 2 * m * n * k
    (fc, f), (dc, d) = best["fwd"], best["dgrad"]
    # the 16-bit input gradient of the same base (no transposed fp8 copy kept): dy in bf16 against the
    # codes as stored, widened in registers with their E8M0 scales; bf16 MFMA, so priced at the bf16 peak
    codes, nat = native.quant_mx(w)[:2]
    codes = codes.view(torch.float8_e4m3fn)
    w16 = {}
    for cfg in (0, 2, 3):  # the tiles built for E8M0-scaled bases: 256 x 256, 256 x 128, 128 x 128
        native.wo_gemm_dgrad(dy, codes, nat, cfg, "mx")
        w16[cfg] = event_ms(lambda: native.wo_gemm_dgrad(dy, codes, nat, cfg, "mx"), reps)
    wc, wt = min(w16.items(), key=lambda kv: kv[1])
    out["mx_frozen_base_M2048_K4096_N12288"] = {"fwd_ms": f, "fwd_TFLOPs": flop / f / 1e9, "fwd_config": fc, "dgrad_ms": d, "dgrad_TFLOPs": flop / d / 1e9, "dgrad_config": dc, "peak_TFLOPs": FP8_PEAK_TFLOPS, "note": "quantizer + GEMM per call",
                                                 "dgrad_w16_ms": wt, "dgrad_w16_TFLOPs": flop / wt / 1e9, "dgrad_w16_config": wc, "dgrad_w16_peak_TFLOPs": 2500.0}
    del codes, nat
    # the row recipe (one fp32 scale per activation row and per weight row) at the headline shape
    m, k, n = 16384, 3072, 9216
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn(n, k, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    bias = torch.zeros(n, dtype=torch.bfloat16, device=dev)
    wq, ws = native.quant_rows(w)
    xq, xs = native.quant_rows(x)
    qbuf, sbuf = torch.empty(m, k, dtype=torch.uint8, device=dev), torch.empty(m, dtype=torch.float32, device=dev)
    lib, stream = native.load(), torch.cuda.current_stream(dev).cuda_stream

    def quant_only():  # the bare entry point: no output allocation in the timed region
        lib.km_quant_rows(x.data_ptr(), m, k, k, 1, native.KM_BF16, qbuf.data_ptr(), sbuf.data_ptr(), stream)

    quant_only()
    qt = event_ms(quant_only, reps)
    gt = event_ms(lambda: native.gemm_fp8_rows(xq, xs, wq, ws, bias, torch.bfloat16, 0), reps)

    def row_step():
        aq, sa = native.quant_rows(x)
        return native.gemm_fp8_rows(aq, sa, wq, ws, bias, torch.bfloat16, 0)

    row_step()
    st = event_ms(row_step, reps)
    flop = 2 * m * n * k
    out["row_recipe_M16384_K3072_N9216"] = {
        "quant_rows_us": qt * 1e3, "quant_rows_GBps": (m * k * 3 + m * 4) / qt / 1e6, "hbm_peak_GBps": HBM_PEAK_GBS,
        "gemm_ms": gt, "gemm_TFLOPs": flop / gt / 1e9, "step_ms": st, "step_TFLOPs": flop / st / 1e9, "peak_TFLOPs": FP8_PEAK_TFLOPS,
    }
    # the per-tensor recipe (one fp32 scale for x, one for W), same shape: abs-max pass + cast, fp8 MFMA GEMM
    wtq, wts = native.quant_tensor(w)
    xtq, xts = native.quant_tensor(x)
    sbuf1 = torch.empty(1, dtype=torch.float32, device=dev)
    amax_work = torch.empty(native.QUANT_TENSOR_WORKSPACE_BYTES // 4, dtype=torch.int32, device=dev)

    def quant_tensor_only():  # the bare entry point: no output allocation in the timed region
        lib.km_quant_tensor(x.data_ptr(), m, k, k, 1, native.KM_BF16, qbuf.data_ptr(), sbuf1.data_ptr(), amax_work.data_ptr(), stream)

    quant_tensor_only()
    qt = event_ms(quant_tensor_only, reps)
    gt = event_ms(lambda: native.gemm_fp8_tensor(xtq, xts, wtq, wts.reshape(1), bias, torch.bfloat16, 0), reps)

    def tensor_step():
        aq, sa = native.quant_tensor(x)
        return native.gemm_fp8_tensor(aq, sa, wtq, wts.reshape(1), bias, torch.bfloat16, 0)

    tensor_step()
    st = event_ms(tensor_step, reps)
    out["tensor_recipe_M16384_K3072_N9216"] = {
        "quant_tensor_us": qt * 1e3, "quant_tensor_GBps": (m * k * 5) / qt / 1e6, "hbm_peak_GBps": HBM_PEAK_GBS,
        "quant_note": "two passes (abs-max over x, then the cast): 2 + 2 bytes read and 1 written per element, the second read mostly from the last-level cache",
        "gemm_ms": gt, "gemm_TFLOPs": flop / gt / 1e9, "step_ms": st, "step_TFLOPs": flop / st / 1e9, "peak_TFLOPs": FP8_PEAK_TFLOPS,
    }
    # the block recipe (fp32 scales per row x 128 columns / per 128 x 128 weight block), same shape
    wbq, wbs = native.quant_blocks(w, "weight")
    xbq, _, xbs = native.quant_blocks(x, "act", natural=False, kmajor=True)  # the GEMM reads the [K/128, M] scale copy
    bsbuf = torch.empty(k // 128, m, dtype=torch.float32, device=dev)

    def quant_blocks_only():
        lib.km_quant_blocks(x.data_ptr(), m, k, k, 1, native.KM_BF16, native.ROLE_ACT, qbuf.data_ptr(), None, bsbuf.data_ptr(), stream)

    quant_blocks_only()
    qt = event_ms(quant_blocks_only, reps)
    times = {}
    for cfg in range(len(native.configs(native.KERNEL_GEMM_BLOCKS))):
        native.gemm_fp8_blocks(xbq, xbs, wbq, wbs, bias, torch.bfloat16, cfg, kmajor=True)
        times[cfg] = event_ms(lambda: native.gemm_fp8_blocks(xbq, xbs, wbq, wbs, bias, torch.bfloat16, cfg, kmajor=True), reps)
    bcfg, gt = min(times.items(), key=lambda kv: kv[1])

    def block_step():
        aq, _, sa = native.quant_blocks(x, "act", natural=False, kmajor=True)
        return native.gemm_fp8_blocks(aq, sa, wbq, wbs, bias, torch.bfloat16, bcfg, kmajor=True)

    block_step()
    st = event_ms(block_step, reps)
    out["block_recipe_M16384_K3072_N9216"] = {
        "quant_blocks_us": qt * 1e3, "quant_blocks_GBps": (m * k * 3 + m * (k // 128) * 4) / qt / 1e6, "hbm_peak_GBps": HBM_PEAK_GBS,
        "gemm_ms": gt, "gemm_TFLOPs": flop / gt / 1e9, "gemm_config": bcfg, "gemm_configs_ms": {str(c): t for c, t in times.items()},
        "step_ms": st, "step_TFLOPs": flop / st / 1e9, "peak_TFLOPs": FP8_PEAK_TFLOPS,
    }
    # short M (launch-bound regime): the one-launch linear that quantizes x inside the GEMM against
    # quantizer + GEMM, bare entry points into preallocated buffers (no allocation in the timed region)
    w_q, _, w_sp = native.quant_mx(w, natural=False, packed=True)
    small = {}
    for ms in (1, 16, 32):
        xs_ = x[:ms].contiguous()
        y_ = torch.empty(ms, n, dtype=torch.bfloat16, device=dev)
        q_ = torch.empty(ms, k, dtype=torch.uint8, device=dev)
        sp_ = torch.zeros(native.packed_scale_bytes(ms, k), dtype=torch.uint8, device=dev)
        cfg_small = len(native.configs(native.KERNEL_GEMM_MX)) - 1  # the 64-row tile

        def fused_call():
            lib.km_gemm_mx_fused(xs_.data_ptr(), k, w_q.data_ptr(), w_sp.data_ptr(), None, y_.data_ptr(), ms, n, k, native.KM_BF16, stream)

        def two_calls():
            lib.km_quant_mx(xs_.data_ptr(), ms, k, k, 1, native.KM_BF16, q_.data_ptr(), None, sp_.data_ptr(), stream)
            lib.km_gemm_mx(q_.data_ptr(), sp_.data_ptr(), w_q.data_ptr(), w_sp.data_ptr(), None, y_.data_ptr(), ms, n, k, native.KM_BF16, native.SCALES_PACKED, cfg_small, stream)

        fused_call()
        two_calls()
        small[f"M{ms}"] = {"fused_us": event_ms(fused_call, reps) * 1e3, "quantizer_plus_gemm_us": event_ms(two_calls, reps) * 1e3}
        # the bound at short M is the weight stream (codes + E8M0 scales read once)
        small[f"M{ms}"]["fused_weight_stream_GBps"] = (n * k + n * k // 32) / small[f"M{ms}"]["fused_us"] / 1e3
        # the block and row recipes at the same shape (weights quantized above: wbq / wbs, wq / ws)
        st_ = torch.empty(k // 128, ms, dtype=torch.float32, device=dev)
        sr_ = torch.empty(ms, dtype=torch.float32, device=dev)

        def fused_block():
            lib.km_gemm_fp8_blocks_fused(xs_.data_ptr(), k, wbq.data_ptr(), wbs.data_ptr(), None, y_.data_ptr(), ms, n, k, native.KM_BF16, stream)

        def two_block():
            lib.km_quant_blocks(xs_.data_ptr(), ms, k, k, 1, native.KM_BF16, native.ROLE_ACT, q_.data_ptr(), None, st_.data_ptr(), stream)
            lib.km_gemm_fp8_blocks(q_.data_ptr(), st_.data_ptr(), wbq.data_ptr(), wbs.data_ptr(), None, y_.data_ptr(), ms, n, k, native.KM_BF16, native.SCALES_KMAJOR, 1, stream)

        def fused_row():
            lib.km_gemm_fp8_rows_fused(xs_.data_ptr(), k, wq.data_ptr(), ws.data_ptr(), None, y_.data_ptr(), ms, n, k, native.KM_BF16, stream)

        def two_row():
            lib.km_quant_rows(xs_.data_ptr(), ms, k, k, 1, native.KM_BF16, q_.data_ptr(), sr_.data_ptr(), stream)
            lib.km_gemm_fp8_rows(q_.data_ptr(), sr_.data_ptr(), wq.data_ptr(), ws.data_ptr(), None, y_.data_ptr(), ms, n, k, native.KM_BF16, cfg_small, stream)

        for fn in (fused_block, two_block, fused_row, two_row):
            fn()
        small[f"M{ms}"].update({"block_fused_us": event_ms(fused_block, reps) * 1e3, "block_quantizer_plus_gemm_us": event_ms(two_block, reps) * 1e3,
                                "row_fused_us": event_ms(fused_row, reps) * 1e3, "row_quantizer_plus_gemm_us": event_ms(two_row, reps) * 1e3})
    out["mx_short_M_K3072_N9216"] = {**small, "weight_MB": n * k / 1e6, "hbm_peak_GBps": HBM_PEAK_GBS, "note": "one launch (x quantized inside the GEMM) vs two; the weight streams once either way"}
    # int8 compute linear (per-row int8 activations, int8 MFMA GEMM, int32 accumulation), same shape
    w_scale = (w.float().abs().amax(1).clamp_min(1e-12) / 127.0)
    w8 = torch.round(w.float() / w_scale[:, None]).clamp_(-127, 127).to(torch.int8)
    x8, x8s = native.quant_rows_i8(x)
    q8buf = torch.empty(m, k, dtype=torch.int8, device=dev)

    def quant8_only():
        lib.km_quant_rows_i8(x.data_ptr(), m, k, k, 1, native.KM_BF16, None, q8buf.data_ptr(), sbuf.data_ptr(), stream)

    def int8_step():
        aq, sa = native.quant_rows_i8(x)
        return native.gemm_i8_rows(aq, sa, w8, w_scale, bias, torch.bfloat16, 0)

    quant8_only()
    int8_step()
    qt = event_ms(quant8_only, reps)
    gt = event_ms(lambda: native.gemm_i8_rows(x8, x8s, w8, w_scale, bias, torch.bfloat16, 0), reps)
    st = event_ms(int8_step, reps)
    # a rotated base (ConvRot, groups of 256): the quantizer rotates the rows on their way in; against
    # the rotation kernel followed by the quantizer
    def quant8_rotated():
        lib.km_quant_rows_i8_rotated(x.data_ptr(), m, k, k, native.KM_BF16, 256, q8buf.data_ptr(), sbuf.data_ptr(), stream)

    xrot = torch.empty_like(x)

    def rotate_then_quant8():
        lib.km_group_hadamard(x.data_ptr(), m, k, native.KM_BF16, 256, xrot.data_ptr(), stream)
        lib.km_quant_rows_i8(xrot.data_ptr(), m, k, k, 1, native.KM_BF16, None, q8buf.data_ptr(), sbuf.data_ptr(), stream)

    quant8_rotated()
    rotate_then_quant8()
    qr = event_ms(quant8_rotated, reps)
    q2 = event_ms(rotate_then_quant8, reps)
    out["int8_compute_M16384_K3072_N9216"] = {
        "quant_rows_us": qt * 1e3, "quant_rows_GBps": (m * k * 3 + m * 4) / qt / 1e6, "hbm_peak_GBps": HBM_PEAK_GBS,
        "gemm_ms": gt, "gemm_TOPs": flop / gt / 1e9, "step_ms": st, "step_TOPs": flop / st / 1e9, "peak_TOPs": 5000.0,
        "rotating_quant_rows_us": qr * 1e3, "rotation_then_quant_rows_us": q2 * 1e3,
        "rotation_share_of_rotated_fwd": max(qr - qt, 0.0) / (st + max(qr - qt, 0.0)),
        "rotation_share_of_rotated_fwd_two_kernels": (q2 - qt) / (st + q2 - qt),
    }
    return out


def same_node(dev, x, w, bias, reps):
    """The vendor library on the same card and the same headline shape, the comparison the reference's
    own benchmark prints (scripts/bench/kernel/fp8.py: bf16 F.linear and torch._scaled_mm): bf16
    GEMM, fp8 GEMM with one scale per tensor, with one scale per row / column, and with E8M0 block
    scales. Each in a try block: what this torch / hipBLASLt build does not offer is reported as such.
    These are library calls timed for reference only; no product path uses them."""
    out = {}
    flop = 2 * x.shape[0] * x.shape[1] * w.shape[0]

    def timed(name, fn, peak):
        try:
            fn()
            ms = event_ms(fn, reps)
            out[name] = {"ms": ms, "TFLOPs": flop / ms / 1e9, "frac": flop / ms / 1e9 / peak}
        except Exception as err:  # noqa: BLE001 - reported, not swallowed
            out[name] = {"unavailable": f"{type(err).__name__}: {str(err)[:160]}"}

    timed("bf16_F_linear", lambda: torch.nn.functional.linear(x, w, bias), 2500.0)
    e4m3 = torch.float8_e4m3fn
    xa, wa = x.float().abs().amax(), w.float().abs().amax()
    sx, sw = (xa / 448.0).reshape(()), (wa / 448.0).reshape(())
    xq8, wq8 = (x.float() / sx).to(e4m3), (w.float() / sw).to(e4m3)
    timed("fp8_scaled_mm_tensor", lambda: torch._scaled_mm(xq8, wq8.t(), scale_a=sx, scale_b=sw, bias=bias, out_dtype=torch.bfloat16), FP8_PEAK_TFLOPS)
    sxr = (x.float().abs().amax(1, keepdim=True) / 448.0).clamp_min(1e-12)
    swr = (w.float().abs().amax(1, keepdim=True) / 448.0).clamp_min(1e-12)
    xqr, wqr = (x.float() / sxr).to(e4m3), (w.float() / swr).to(e4m3)
    timed("fp8_scaled_mm_rows", lambda: torch._scaled_mm(xqr, wqr.t(), scale_a=sxr, scale_b=swr.t(), bias=bias, out_dtype=torch.bfloat16), FP8_PEAK_TFLOPS)
    e8m0 = getattr(torch, "float8_e8m0fnu", None)
    if e8m0 is None:
        out["fp8_scaled_mm_mx"] = {"unavailable": "torch has no float8_e8m0fnu"}
    else:
        from kohakumosstrainer_amd import native

        xq, xs = native.quant_mx(x)[:2]
        wq, ws = native.quant_mx(w)[:2]
        timed("fp8_scaled_mm_mx", lambda: torch._scaled_mm(xq, wq.t(), scale_a=xs.view(e8m0), scale_b=ws.view(e8m0), bias=bias, out_dtype=torch.bfloat16), FP8_PEAK_TFLOPS)
    out["note"] = "vendor library GEMMs alone (no activation quantizer in the timed call), same card, same operands' shape; frac is of the same peak as this build's kernels"
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=200, help="untimed steps first (about 0.1 s: the card needs that long to reach its sustained clocks)")
    ap.add_argument("--config", type=int, default=-1, help="GEMM tile configuration; -1 times every configuration once, as the tuning table does, and takes the fastest")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--headline-only", action="store_true", help="only the headline step and its GEMM (for short profiler runs): no quantizer sweep, no other shapes, no CPU leg")
    ap.add_argument("--calibrate", action="store_true", help="also run 5 plain device copies of the activation tensor (a kernel of known HBM traffic, to scale profiler byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path needs no second GPU); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    from kohakumosstrainer_amd import native

    native.load()
    dev = torch.device("cuda", 0)
    x, w, bias = synthetic(dev)
    # weights are quantized once, outside the step; the GEMM reads the MFMA-packed scale copy
    wq, ws, wsp = native.quant_mx(w, packed=True)

    xq0, _, xsp0 = native.quant_mx(x, natural=False, packed=True)
    config, tried = args.config, {}
    if config < 0:
        for _ in range(100):  # reach sustained clocks before comparing
            native.gemm_mx(xq0, xsp0, wq, wsp, bias, torch.bfloat16, 0, packed=True)
        for cfg in native.configs(native.KERNEL_GEMM_MX):
            run = lambda c=cfg["id"]: native.gemm_mx(xq0, xsp0, wq, wsp, bias, torch.bfloat16, c, packed=True)
            event_ms(run, 5)
            tried[cfg["id"]] = event_ms(run, 20)
        config = min(tried, key=tried.get)

    def step():
        xq, _, xsp = native.quant_mx(x, natural=False, packed=True)
        return native.gemm_mx(xq, xsp, wq, wsp, bias, torch.bfloat16, config, packed=True)

    if args.calibrate:
        sink = torch.empty_like(x)
        for _ in range(5):
            sink.copy_(x)  # reads and writes M*K*2 bytes each
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # per-kernel device time, measured live with events: the GEMM inside the same step sequence
    # (its launch follows the quantizer's, as in the timed region), the quantizers back to back
    marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for before, after in marks:
        xq, _, xsp = native.quant_mx(x, natural=False, packed=True)
        before.record()
        native.gemm_mx(xq, xsp, wq, wsp, bias, torch.bfloat16, config, packed=True)
        after.record()
    torch.cuda.synchronize()
    gemm_ms = sum(b.elapsed_time(a) for b, a in marks) / len(marks)
    if args.headline_only:
        achieved = GEMM_FLOP / (gemm_ms * 1e-3) / 1e12
        print(json.dumps({"ms_per_step": ms_per_step, "gemm_ms": gemm_ms, "gemm_TFLOPs": achieved, "frac": achieved / FP8_PEAK_TFLOPS, "gemm_tile_config": config, "gemm_tile_configs_ms": tried}))
        return
    ceiling = mfma_ceiling(xq0, wq)
    qreps = min(max(args.steps, 10), 100)
    # the same two kernels on a ring of five input tensors whose outputs are kept alive
    # (760 MB in all, three times the last-level cache): every byte comes from and goes to HBM
    # tensors of the standalone-quantizer configuration: N(0,1) with 0.1 % of the entries replaced by +-N(0,50)
    def with_outliers(seed):
        gg = torch.Generator(device=dev).manual_seed(seed)
        t = torch.randn(M, K, device=dev, generator=gg)
        hit = torch.rand(M, K, device=dev, generator=gg) < 1e-3
        return torch.where(hit, torch.randn(M, K, device=dev, generator=gg) * 50.0, t).to(torch.bfloat16)

    ring = [with_outliers(10 + i) for i in range(5)]
    held = [None] * 5
    state = {"i": 0}

    def cold(view):
        def run():
            i = state["i"] = (state["i"] + 1) % 5
            held[i] = native.quant_mx(view(ring[i]))
        return run

    x3 = ring[0]
    rows_ms = event_ms(lambda: native.quant_mx(x3), qreps)
    fused_rows_ms = event_ms(lambda: native.quant_mx(x3, natural=False, packed=True), qreps)
    x3t = x3.t()
    cols_ms = event_ms(lambda: native.quant_mx(x3t), qreps)
    for f in (cold(lambda t: t), cold(lambda t: t.t())):
        event_ms(f, 10)
    rows_cold_ms = event_ms(cold(lambda t: t), qreps)
    cols_cold_ms = event_ms(cold(lambda t: t.t()), qreps)
    # what a plain device copy of the same number of bytes takes on the same ring: the ceiling a
    # streaming kernel can reach on this card (a copy moves QUANT_BYTES / 1.5 * 2 bytes per call of
    # bf16 in and out; scaled to the quantizer's byte count)
    copies = [torch.empty_like(ring[0]) for _ in range(5)]

    def cold_copy():
        i = state["i"] = (state["i"] + 1) % 5
        copies[i].copy_(ring[i])

    event_ms(cold_copy, 10)
    copy_cold_ms = event_ms(cold_copy, qreps)
    copy_bytes = 2 * ring[0].numel() * 2
    copy_GBps = copy_bytes / (copy_cold_ms * 1e-3) / 1e9
    del ring, held, copies
    achieved = GEMM_FLOP / (gemm_ms * 1e-3) / 1e12

    line = {
        "metric": "MXFP8 GEMM TFLOP/s & % fp8 MFMA peak; quantize GB/s & % HBM peak (1 GPU)",
        "value": GEMM_FLOP / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 (E8M0 block scales), fp32 accumulate, bf16 out",
        "data": "synthetic",
        "config": {
            "workload": f"MXFP8 fused-QKV linear forward M={M} K={K} N={N}: per-call activation quantizer + block-scaled GEMM + bias, bf16 out (benchmark configs[3]); quantizer alone on bf16 [{M},{K}] row- and column-wise (configs[2])",
            "gemm_tile_config": config,
            "gemm_tile_configs_ms": tried,
        },
        "roofline": {
            "kernel": "gemm_fp8_kernel (MX)",
            "bound": "mfma",
            "achieved": achieved,
            "peak": FP8_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / FP8_PEAK_TFLOPS,
            "traffic": profiled_traffic_bytes(),
            "traffic_source": "profiles/" + os.path.basename(TRAFFIC_PROFILE),
            "algorithmic_flop": GEMM_FLOP,
            "ms": gemm_ms,
            "peak_sustained": ceiling["TFLOPs"],
            "frac_of_sustained": achieved / ceiling["TFLOPs"],
            "sustained": ceiling,
        },
        "quantizer": {
            "bound": "hbm",
            "bytes_per_launch": QUANT_BYTES,
            "rows_ms": rows_cold_ms,
            "rows_GBps": QUANT_BYTES / (rows_cold_ms * 1e-3) / 1e9,
            "rows_frac": QUANT_BYTES / (rows_cold_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "cols_ms": cols_cold_ms,
            "cols_GBps": QUANT_BYTES / (cols_cold_ms * 1e-3) / 1e9,
            "cols_frac": QUANT_BYTES / (cols_cold_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "rows_warm_ms": rows_ms,
            "rows_warm_packed_scales_ms": fused_rows_ms,
            "rows_warm_GBps": QUANT_BYTES / (rows_ms * 1e-3) / 1e9,
            "rows_warm_frac": QUANT_BYTES / (rows_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "cols_warm_ms": cols_ms,
            "cols_warm_GBps": QUANT_BYTES / (cols_ms * 1e-3) / 1e9,
            "cols_warm_frac": QUANT_BYTES / (cols_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "copy_cold_ms": copy_cold_ms,
            "copy_cold_GBps": copy_GBps,
            "copy_cold_frac": copy_GBps / HBM_PEAK_GBS,
            "rows_cold_vs_copy": (QUANT_BYTES / (rows_cold_ms * 1e-3) / 1e9) / copy_GBps,
            "cols_cold_vs_copy": (QUANT_BYTES / (cols_cold_ms * 1e-3) / 1e9) / copy_GBps,
            "data": "bf16 [16384, 3072], N(0,1) with 0.1 % of the entries replaced by +-N(0,50) (the standalone-quantizer configuration)",
            "note": "rows_/cols_: every launch on another tensor of a ring larger than the 256 MB last-level cache, outputs kept alive (every byte from and to HBM); *_warm_: back-to-back launches on one tensor (the reference's timing method; part of it stays in that cache); copy_cold_: torch's device copy of one ring tensor (read + write) on the same ring, the practical HBM ceiling of a streaming kernel here",
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
        },
    }
    reps = min(max(args.steps // 2, 5), 50)
    line["same_node"] = same_node(dev, x, w, bias, reps)
    line["other_configs"] = other_configs(dev, reps)
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(x, wq, ws, bias)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
