#!/usr/bin/env python3
"""Headline benchmark: FP8 e4m3 GEMM M=N=K=8192 on one MI355X.

One "step" = one GEMM launch over operands already resident in HBM (A [M,K] and B [N,K]
e4m3 with per-tensor fp32 scales, C [M,N] bf16). Protocol follows the reference's harness
(kernels/gemm/bf16fp32/mi350x/test_python.py:20-29, 79-101: 500 warm-up and 100 timed
launches, flops = 2*M*N*K). Prints ONE JSON line.

  python bench.py [--gpus 1] [--steps 100] [--warmup 500] [--workload fp8_gemm] [--size 8192]

`roofline` is measured with HIP events on the launch stream around the timed region;
`cpu_baseline` times the CPU oracle path (PyTorch-CPU dequantize + fp32 matmul) on the
host cores over a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5033.0  # MI355X dense FP8 MFMA peak (256 CU x 2.4 GHz x 8192 flop/clk/CU)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--workload", default="fp8_gemm", choices=["fp8_gemm"])
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (--gpus 1); "
              "no multi-GPU path exists for this kernel library.", file=sys.stderr)
        return 2

    import torch

    import hipkittens_amd as hk

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    hk.load_library()  # raises if libhk355.so has not been built
    dev = torch.device("cuda:0")
    n = args.size
    M = N = K = n

    g = torch.Generator(device=dev).manual_seed(0)
    A = torch.randn(M, K, device=dev, generator=g)
    B = torch.randn(N, K, device=dev, generator=g)
    Aq, sa = hk.quant.quantize_fp8_per_tensor(A)
    Bq, sb = hk.quant.quantize_fp8_per_tensor(B)
    del A, B
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    def step():
        hk.tk_kernel.dispatch_fp8_gemm(Aq, Bq, C, sa, sb)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps  # HIP events on the launch stream

    flops = 2.0 * M * N * K
    tflops = flops / (wall_ms * 1e-3) / 1e12
    kern_tflops = flops / (kern_ms * 1e-3) / 1e12

    # parity spot check against the oracle on a row sample (outside the timed region)
    from oracle import gemm as OG
    import numpy as np

    rows = torch.arange(0, M, max(1, M // 16), device=dev)
    ref = OG.fp8_gemm(Aq.view(torch.uint8)[rows].cpu().numpy(), Bq.view(torch.uint8).cpu().numpy(), sa, sb)
    rel = OG.rel_fro_error(C[rows].float().cpu().numpy(), ref)

    cpu = None
    if not args.no_cpu_baseline:
        r = OG.cpu_baseline_fp8_gemm(M, N, K, seed=0, repeats=1)
        cpu = {"value": round(r["tflops"], 4), "unit": "TFLOP/s", "cores": r["threads"], "kind": "port",
               "sample": f"one full {M}x{N}x{K} dequantize+fp32 matmul (torch CPU), {r['seconds']:.2f} s"}

    out = {
        "metric": "FP8 e4m3 GEMM 8192^3 throughput" if n == 8192 else f"FP8 e4m3 GEMM {n}^3 throughput",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": round(tflops / 3327.46, 4) if n == 8192 else None,
        "dtype": "fp8_e4m3 (fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {"workload": f"fp8_gemm M=N=K={n}, A row-major, B [N,K], per-tensor fp32 scales, randn inputs"},
        "pct_of_fp8_peak": round(100.0 * tflops / PEAK_FP8_TFLOPS, 2),
        "rel_fro_err_vs_oracle": rel,
        "roofline": {"bound": "mfma", "achieved": round(kern_tflops, 2), "peak": PEAK_FP8_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(kern_tflops / PEAK_FP8_TFLOPS, 4), "traffic": None,
                     "kernel_ms": round(kern_ms, 5)},
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
