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
CPU_SAMPLE_ROWS = 512


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


def cpu_baseline(x, wq, ws, bias):
    """The oracle's eager forward (quantize, dequantize both operands, bf16 linear) on the
    first CPU_SAMPLE_ROWS rows of the same activations, all host threads, best of 3."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle import linear

    xs = x[:CPU_SAMPLE_ROWS].cpu()
    wq_c, ws_c, b_c = wq.cpu(), ws.cpu(), bias.cpu()
    best = float("inf")
    for _ in range(3):
        t = time.perf_counter()
        linear.fp8_forward(xs, wq_c, ws_c, None, b_c, "mx")
        best = min(best, time.perf_counter() - t)
    flop = 2 * CPU_SAMPLE_ROWS * N * K
    return {
        "value": flop / best / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": f"first {CPU_SAMPLE_ROWS} of {M} rows, full W [{N},{K}]: quantize + dequantize + bf16 linear, best of 3 ({best:.2f} s)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--config", type=int, default=0, help="GEMM tile configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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

    def step():
        xq, _, xsp = native.quant_mx(x, natural=False, packed=True)
        return native.gemm_mx(xq, xsp, wq, wsp, bias, torch.bfloat16, args.config, packed=True)

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

    # per-kernel device time, measured live with events
    xq, _, xsp = native.quant_mx(x, natural=False, packed=True)
    gemm_ms = event_ms(lambda: native.gemm_mx(xq, xsp, wq, wsp, bias, torch.bfloat16, args.config, packed=True), max(args.steps, 10))
    rows_ms = event_ms(lambda: native.quant_mx(x), max(args.steps, 10))
    fused_rows_ms = event_ms(lambda: native.quant_mx(x, natural=False, packed=True), max(args.steps, 10))
    xt = x.t()
    cols_ms = event_ms(lambda: native.quant_mx(xt), max(args.steps, 10))
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
            "workload": f"MXFP8 fused-QKV linear forward M={M} K={K} N={N}: per-call activation quantizer + block-scaled GEMM + bias, bf16 out (BASELINE configs[3]); quantizer alone on bf16 [{M},{K}] row- and column-wise (configs[2])",
            "gemm_tile_config": args.config,
        },
        "roofline": {
            "kernel": "gemm_fp8_kernel (MX)",
            "bound": "mfma",
            "achieved": achieved,
            "peak": FP8_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": achieved / FP8_PEAK_TFLOPS,
            "traffic": None,
            "ms": gemm_ms,
        },
        "quantizer": {
            "bound": "hbm",
            "bytes_per_launch": QUANT_BYTES,
            "rows_ms": rows_ms,
            "rows_packed_scales_ms": fused_rows_ms,
            "rows_GBps": QUANT_BYTES / (rows_ms * 1e-3) / 1e9,
            "rows_frac": QUANT_BYTES / (rows_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "cols_ms": cols_ms,
            "cols_GBps": QUANT_BYTES / (cols_ms * 1e-3) / 1e9,
            "cols_frac": QUANT_BYTES / (cols_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
        },
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(x, wq, ws, bias)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
