#!/usr/bin/env python3
"""Benchmarks of the quantized-contraction path on one MI355X. Prints ONE JSON line.

Headline (`value`): FP8 e4m3 GEMM M=N=K=8192. One "step" = one GEMM launch over operands that
are already resident in HBM (A [M,K] and B [N,K] e4m3 with per-tensor fp32 scales, C [M,N] bf16).
Protocol follows the reference's harness (kernels/gemm/bf16fp32/mi350x/test_python.py:20-29,
79-101: 500 warm-up and 100 timed launches, flops = 2*M*N*K).

  python bench.py [--gpus 1] [--steps 100] [--warmup 500] [--only-headline] [--no-cpu-baseline]
  python bench.py --traffic-calibration     (a 1 GiB copy + the headline GEMM, for counter runs)
  python bench.py --only LEG[,LEG]          (selected legs of `extra`, for profiler runs)

Clock settling: an MI355X that has been idle runs its first tens of milliseconds of work below the
clock it sustains, so a short warm-up (the driver's `--warmup 5` is 2 ms of work) times the ramp, not
the kernel. Before `--warmup` the headline launch is therefore repeated, untimed, for `--settle-ms`
milliseconds (default 600, about what the reference's 500 warm-up launches of its own protocol take
together with its timed ones); the count is printed as `settle_launches`. The timed region is
unchanged: exactly `--steps` launches between two events on the launch stream.

`roofline` objects: `achieved` = algorithmic flop (or bytes) per call / measured time per call (HIP
events on the launch stream around the timed region); `peak` = the published MI355X figure; `traffic`
= HBM-side bytes per launch from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs scaled by the same
counters' reading for a plain copy (summaries under profiles/), or null where no such run exists.
`cpu_baseline` times the CPU counterpart (PyTorch-CPU dequantize + fp32 matmul; the oracle's MoE
forward on a stated subset) on the host cores.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8 = 5033.0     # MI355X dense FP8 MFMA peak, TFLOP/s (256 CU x 2.4 GHz x 8192 flop/clk/CU)
PEAK_FP4 = 10066.0    # dense MXFP4
PEAK_BF16 = 2516.5    # dense bf16
PEAK_HBM = 8000.0     # GB/s
# HBM-side bytes per launch (`traffic` of the roofline objects): profiles/traffic.json, written by
# `python bench.py --collect-traffic DIR` from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs (one directory
# per run under DIR, see collect_traffic), each counter scaled by its reading for a 1 GiB copy
# (`bench.py --traffic-calibration`). The file is the only source of these figures: a profile refresh
# rewrites it and the next bench line carries the new values.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
# The launches that make up one call of each leg's default workload, as rocprofv3 names the kernels.
TRAFFIC_LEGS = {
    "fp8_gemm_8192": ("calibration", ["fp8_gemm_4wave_ring_kernel<false>"]),
    "mxfp4_gemm": ("mxfp4", ["mxfp4_gemm_4wave_kernel<false>"]),
    "bf16_gemm": ("bf16", ["bf16_gemm_4wave_ring_kernel<false, true>"]),
    "fp8_gemm_decode_m16": ("decode", ["fp8_gemm_skinny_kernel<1, 4, 4, 2, true>"]),
    "moe_mxfp4": ("moe_mxfp4", ["moe_topk_softmax_kernel<16>", "moe_sort_quantize_kernel<false>",
                                "moe_mxfp4_stream4_kernel<0, false, false, true, true>",
                                "moe_mxfp4_stream4_kernel<1, false, false, false, true>", "moe_unpermute_kernel<4>"]),
    "moe_fp8blk": ("moe_fp8blk", ["moe_topk_grouped_sigmoid16_kernel<16>", "moe_sort_count_kernel",
                                  "moe_sort_scan_offsets_kernel", "moe_sort_scatter_kernel", "moe_build_items_kernel",
                                  "moe_fp8blk_stream_kernel<0, true, false, 9>",
                                  "moe_fp8blk_stream_kernel<1, false, false, 9>", "moe_unpermute_kernel<8>"]),
}
_traffic_cache = None


def _traffic(key):
    """HBM-side bytes per call of leg `key` from profiles/traffic.json, or None."""
    global _traffic_cache
    if _traffic_cache is None:
        try:
            with open(TRAFFIC_FILE) as f:
                _traffic_cache = json.load(f).get("legs", {})
        except (OSError, ValueError):
            _traffic_cache = {}
    leg = _traffic_cache.get(key)
    return float(leg["total_bytes"]) if leg else None


def collect_traffic(root):
    """Reads the counter runs under `root` and rewrites profiles/traffic.json.

    Expected below `root`, each the -d directory of one run of
        rocprofv3 --pmc COUNTER --output-format csv -d root/RUN_COUNTER -o x -- python3 bench.py ARGS
    with COUNTER = FETCH_SIZE and WRITE_SIZE: RUN = calibration (ARGS: --traffic-calibration) and one RUN per
    leg of TRAFFIC_LEGS (ARGS: --only RUN --no-cpu-baseline --no-graph --steps 5 --warmup 2 --settle-ms 50).
    A counter's KiB per dispatch are scaled by 1 GiB / its reading for the calibration run's copy kernel."""
    import collections
    import csv
    import glob

    def per_kernel(run, counter, reduce="mean"):
        acc = collections.defaultdict(list)
        files = glob.glob(os.path.join(root, f"{run}_{counter}", "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise RuntimeError(f"no counter_collection.csv under {root}/{run}_{counter}")
        for path in files:
            with open(path) as f:
                for row in csv.DictReader(f):
                    if row["Counter_Name"] == counter:
                        acc[row["Kernel_Name"]].append(float(row["Counter_Value"]))
        return {k: (max(v) if reduce == "max" else sum(v) / len(v)) for k, v in acc.items()}

    def one(avgs, needle, what):
        hits = [v for k, v in avgs.items() if needle in k]
        if len(hits) != 1:
            raise RuntimeError(f"{what}: {len(hits)} kernels match {needle!r} (the leg's launches changed: update TRAFFIC_LEGS)")
        return hits[0]

    factor = {}
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        # the largest dispatch of the runtime's buffer-copy kernel is the 1 GiB copy (smaller copies ride along)
        cal = per_kernel("calibration", counter, reduce="max")
        copies = [v for k, v in cal.items() if "copyBuffer" in k]
        if not copies or max(copies) < 1000.0:
            raise RuntimeError(f"calibration run of {counter}: no 1 GiB copy found among {sorted(cal)}")
        factor[counter] = (1 << 20) / max(copies)           # 1 GiB = 2^20 KiB moved per copy launch
    legs = {}
    for key, (run, kernels) in TRAFFIC_LEGS.items():
        rd = per_kernel(run, "FETCH_SIZE")
        wr = per_kernel(run, "WRITE_SIZE")
        detail = {}
        for name in kernels:
            detail[name] = {"read_bytes": round(one(rd, name, key) * factor["FETCH_SIZE"] * 1024),
                            "written_bytes": round(one(wr, name, key) * factor["WRITE_SIZE"] * 1024)}
        legs[key] = {"read_bytes": sum(d["read_bytes"] for d in detail.values()),
                     "written_bytes": sum(d["written_bytes"] for d in detail.values()), "kernels": detail}
        legs[key]["total_bytes"] = legs[key]["read_bytes"] + legs[key]["written_bytes"]
    out = {"source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, KiB per dispatch x calibration factor (bench.py --collect-traffic)",
           "calibration_factor": {k: round(v, 4) for k, v in factor.items()}, "legs": legs}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    return out


def _roofline(bound, achieved, peak, unit, kernel, traffic=None, **more):
    out = {"bound": bound, "achieved": round(achieved, 2), "peak": peak, "unit": unit,
           "frac": round(achieved / peak, 4), "kernel": kernel, "traffic": traffic}
    out.update(more)
    return out


def _timeit(torch, fn, warmup, iters):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / iters
    return wall, e0.elapsed_time(e1) / iters


def _settle(torch, fn, ms):
    """Repeat `fn` untimed until `ms` milliseconds of GPU work have been queued and finished."""
    n = 0
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(50):
            fn()
        n += 50
        torch.cuda.synchronize()
    return n


def _timeit_graph(torch, fn, out, iters, replays=10):
    """Per-call GPU time of `fn` with the host's launch cost taken out: `iters` calls captured in a
    HIP graph, replayed `replays` times. Calls shorter than the Python call path (about 9 us) are
    otherwise timed by the host, not the GPU. `out` (the tensor `fn` writes) is compared after every
    replay with what an eager call wrote."""
    fn()
    torch.cuda.synchronize()
    want = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(iters):
            fn()
    for _ in range(2):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), "graph replay differs from the eager call"
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16)), "graph replay differs from the eager call"
    return e0.elapsed_time(e1) / (iters * replays)


def _np_bits(t):
    import numpy as np
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


# ------------------------------------------------------------------------------------- FP8 GEMM
def bench_fp8(torch, hk, n, warmup, iters, dev, keep=False, graph=False, settle_ms=0.0):
    g = torch.Generator(device=dev).manual_seed(0)
    Aq, sa = hk.quant.quantize_fp8_per_tensor(torch.randn(n, n, device=dev, generator=g))
    Bq, sb = hk.quant.quantize_fp8_per_tensor(torch.randn(n, n, device=dev, generator=g))
    C = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    call = lambda: hk.tk_kernel.dispatch_fp8_gemm(Aq, Bq, C, sa, sb)
    settled = _settle(torch, call, settle_ms) if settle_ms > 0 else 0
    wall, kern = _timeit(torch, call, warmup, iters)
    res = {"wall_ms": wall, "kernel_ms": kern, "tflops": 2.0 * n ** 3 / (kern * 1e-3) / 1e12, "settle_launches": settled}
    if graph:
        gms = _timeit_graph(torch, call, C, iters)
        res["tflops_graph"] = 2.0 * n ** 3 / (gms * 1e-3) / 1e12
    if keep:
        res.update(A=Aq, B=Bq, C=C, sa=sa, sb=sb)
    return res


def bench_fp8_reference_inputs(torch, hk, n, warmup, iters, dev):
    """The same GEMM on the reference executable's input distribution
    (kernels/gemm/fp8fp32/profile_utils.cpp:35-45: uniform(-1, 1) converted to e4m3, no scales).
    Operand bits set the power the MFMA pipes draw, so the published figure is compared on these."""
    g = torch.Generator(device=dev).manual_seed(42)
    A = (torch.rand(n, n, device=dev, generator=g) * 2 - 1).to(torch.float8_e4m3fn)
    B = (torch.rand(n, n, device=dev, generator=g) * 2 - 1).to(torch.float8_e4m3fn)
    C = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    _, kern = _timeit(torch, lambda: hk.tk_kernel.dispatch_fp8_gemm(A, B, C, 1.0, 1.0), warmup, iters)
    tf = 2.0 * n ** 3 / (kern * 1e-3) / 1e12
    return {"workload": f"fp8_gemm M=N=K={n}, uniform(-1,1) -> e4m3, unit scales", "kernel_ms": round(kern, 5),
            "tflops": round(tf, 1), "vs_reference_3327.46": round(tf / 3327.46, 4) if n == 8192 else None,
            "roofline": _roofline("mfma", tf, PEAK_FP8, "TFLOP/s", "fp8_gemm_4wave_ring_kernel")}


def bench_library_baselines(torch, n, warmup, iters, dev):
    """The vendor library on the same box and the same inputs, for reference only (nothing in the
    product path calls it): hipBLASLt behind torch._scaled_mm for FP8, torch.matmul for bf16. The
    reference's own table gives hipBLASLt 3233 and torch bf16 1521 TFLOP/s at 8192^3 on its MI355X
    (analysis/fp8_gemm/mi350x/mi355x_fp8_gemm.json:20-25, analysis/bf16_gemm/mi350x/mi355x_bf16_gemm.json)."""
    out = {}
    g = torch.Generator(device=dev).manual_seed(0)
    a = torch.randn(n, n, device=dev, generator=g)
    b = torch.randn(n, n, device=dev, generator=g)
    try:
        sa, sb = (a.abs().max() / 448).float(), (b.abs().max() / 448).float()
        A, B = (a / sa).to(torch.float8_e4m3fn), (b / sb).to(torch.float8_e4m3fn)
        _, ms = _timeit(torch, lambda: torch._scaled_mm(A, B.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16),
                        warmup, iters)
        out["hipblaslt_fp8_tflops"] = round(2.0 * n ** 3 / (ms * 1e-3) / 1e12, 1)
        del A, B
    except Exception as ex:  # this torch build may not expose the call: the comparison is optional
        out["hipblaslt_fp8_tflops"] = f"unavailable: {type(ex).__name__}"
    Ab, Bb = a.to(torch.bfloat16), b.to(torch.bfloat16)
    del a, b
    _, ms = _timeit(torch, lambda: torch.matmul(Ab, Bb.t()), warmup, iters)
    out["torch_bf16_matmul_tflops"] = round(2.0 * n ** 3 / (ms * 1e-3) / 1e12, 1)
    return out


def bench_bf16(torch, hk, n, warmup, iters, dev):
    from oracle import gemm as OG

    g = torch.Generator(device=dev).manual_seed(0)
    A = torch.randn(n, n, device=dev, generator=g).to(torch.bfloat16)
    B = torch.randn(n, n, device=dev, generator=g).to(torch.bfloat16)
    C = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    _, kern = _timeit(torch, lambda: hk.tk_kernel.dispatch_bf16_gemm(A, B, C), warmup, iters)
    tf = 2.0 * n ** 3 / (kern * 1e-3) / 1e12
    rows = torch.arange(0, n, max(1, n // 16), device=dev)
    rel = OG.rel_fro_error(C[rows].float().cpu().numpy(), OG.bf16_gemm(_np_bits(A[rows]), _np_bits(B)))
    # reference: 1610.5 TFLOP/s at 8192^3 on MI355X (analysis/bf16_gemm/mi350x/mi355x_bf16_gemm.json)
    return {"workload": f"bf16_gemm M=N=K={n}", "kernel_ms": round(kern, 5), "tflops": round(tf, 1),
            "vs_reference_1610.5": round(tf / 1610.5, 4), "rel_fro_err_vs_oracle": rel,
            "roofline": _roofline("mfma", tf, PEAK_BF16, "TFLOP/s", "bf16 256x256x64 tile kernel", _traffic("bf16_gemm"))}


# A decode step multiplies by every weight matrix of a model once, far more bytes than the 256 MB memory-side
# cache holds; a loop over one and the same matrix would find it there. The decode legs therefore rotate over
# enough matrices of the shape to exceed that cache more than four times (with 600 MB in rotation the FP8 decode
# GEMM still read 10 % faster than with 900 MB or more: the cache does not evict in order of use).
ROTATE_BYTES = 1.2e9


def bench_fp8_decode(torch, hk, warmup, iters, dev, graph=True):
    """Decode-like shapes (few rows, N = K = 8192): HBM bound, weights read once, the calls rotating over
    ROTATE_BYTES of weight matrices. Per-call times include the Python call path (about 9 us, which bounds them
    from below); `us_from_graph` is the GPU time of the same calls replayed from a HIP graph, and the roofline
    figure uses it when it was measured."""
    out = []
    g = torch.Generator(device=dev).manual_seed(0)
    N = K = 8192
    nb = int(ROTATE_BYTES // (N * K)) + 1
    Bs = [torch.randn(N, K, device=dev, generator=g).to(torch.float8_e4m3fn) for _ in range(nb)]
    for M in (16, 64, 128):
        A = torch.randn(M, K, device=dev, generator=g).to(torch.float8_e4m3fn)
        C = torch.empty(nb, M, N, dtype=torch.bfloat16, device=dev)
        ws = torch.empty(max(16, hk.tk_kernel.fp8_gemm_workspace_bytes(M, N, K)), dtype=torch.uint8, device=dev)

        def cycle(workspace=None):
            for j in range(nb):
                hk.tk_kernel.dispatch_fp8_gemm(A, Bs[j], C[j], 1.0, 1.0, workspace=workspace)

        rounds = max(1, iters // nb)
        _, plain = _timeit(torch, cycle, max(1, warmup // nb), rounds)
        _, split = _timeit(torch, lambda: cycle(ws), max(1, warmup // nb), rounds)
        gms = _timeit_graph(torch, lambda: cycle(ws), C, rounds) if graph else None
        plain, split = plain / nb, split / nb
        gms = gms / nb if graph else None
        byts = M * K + N * K + 2 * M * N
        # up to 64 rows both calls run the skinny kernel (no workspace needed); M = 128 has a 64x64 tile for every CU
        # and is not split either (split-K is for fewer tiles: at most one for every second CU)
        kernel = "fp8_gemm_skinny_kernel" if M <= 64 else "fp8_gemm_small_tile_kernel<64,4>"
        best = gms if graph else min(plain, split)
        out.append({"shape": f"M={M} N=K=8192, {nb} weight matrices in rotation",
                    "us_without_workspace": round(plain * 1e3, 1),
                    "us_with_workspace": round(split * 1e3, 1), "us_from_graph": round(gms * 1e3, 1) if graph else None,
                    "roofline": _roofline("hbm", byts / (best * 1e-3) / 1e9, PEAK_HBM, "GB/s", kernel,
                                          _traffic("fp8_gemm_decode_m16") if M == 16 else None)})
    return out


def bench_mxfp4_decode(torch, hk, warmup, iters, dev, graph=True):
    """MXFP4 decode-like shapes: few rows against weight matrices that are read once (rotation and timings as in
    bench_fp8_decode)."""
    out = []
    g = torch.Generator(device=dev).manual_seed(0)
    for M, N, K in ((16, 8192, 8192), (16, 4096, 14336)):
        nb = int(ROTATE_BYTES // (N * (K // 2 + K // 32))) + 1
        A, SA = hk.quant.quantize_mxfp4(torch.randn(M, K, device=dev, generator=g))
        Ws = [hk.quant.quantize_mxfp4(torch.randn(N, K, device=dev, generator=g)) for _ in range(nb)]
        C = torch.empty(nb, M, N, dtype=torch.bfloat16, device=dev)
        ws = torch.empty(max(16, hk.tk_kernel.mxfp4_gemm_workspace_bytes(M, N, K)), dtype=torch.uint8, device=dev)

        def cycle(workspace=None):
            for j in range(nb):
                hk.tk_kernel.dispatch_mxfp4_gemm(A, SA, Ws[j][0], Ws[j][1], C[j], workspace=workspace)

        rounds = max(1, iters // nb)
        _, plain = _timeit(torch, cycle, max(1, warmup // nb), rounds)
        _, split = _timeit(torch, lambda: cycle(ws), max(1, warmup // nb), rounds)
        gms = _timeit_graph(torch, cycle, C, rounds) if graph else None
        plain, split = plain / nb, split / nb
        gms = gms / nb if graph else None
        byts = (M + N) * (K // 2 + K // 32) + 2 * M * N
        best = gms if graph else min(plain, split)
        # both calls run the skinny kernel at these shapes (no workspace needed)
        out.append({"shape": f"M={M} N={N} K={K}, {nb} weight matrices in rotation",
                    "us_without_workspace": round(plain * 1e3, 1),
                    "us_with_workspace": round(split * 1e3, 1), "us_from_graph": round(gms * 1e3, 1) if graph else None,
                    "roofline": _roofline("hbm", byts / (best * 1e-3) / 1e9, PEAK_HBM, "GB/s",
                                          "mxfp4_gemm_skinny_kernel")})
    return out


def bench_mxfp4(torch, hk, n, warmup, iters, dev):
    from oracle import gemm as OG

    g = torch.Generator(device=dev).manual_seed(0)
    A, SA = hk.quant.quantize_mxfp4(torch.randn(n, n, device=dev, generator=g))
    B, SB = hk.quant.quantize_mxfp4(torch.randn(n, n, device=dev, generator=g))
    C = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    _, kern = _timeit(torch, lambda: hk.tk_kernel.dispatch_mxfp4_gemm(A, SA, B, SB, C), warmup, iters)
    tf = 2.0 * n ** 3 / (kern * 1e-3) / 1e12
    # parity spot check against the oracle on a row sample (outside the timed region)
    rows = torch.arange(0, n, max(1, n // 16), device=dev)
    ref = OG.mxfp4_gemm(A[rows].cpu().numpy(), SA[rows].cpu().numpy(), B.cpu().numpy(), SB.cpu().numpy())
    rel = OG.rel_fro_error(C[rows].float().cpu().numpy(), ref)
    return {"workload": f"mxfp4_gemm M=N=K={n}", "kernel_ms": round(kern, 5), "tflops": round(tf, 1),
            "rel_fro_err_vs_oracle": rel,
            "roofline": _roofline("mfma", tf, PEAK_FP4, "TFLOP/s", "mxfp4 256x256x256 tile kernel", _traffic("mxfp4_gemm"))}


def bench_schedules(torch, hk, n, warmup, iters, dev):
    """The schedules of the large-tile GEMMs side by side (kernels/gemm/fp8fp32/README.md:3-5 names the first two
    for the reference): 4 waves with hand-interleaved slots (one wave per SIMD; what the library picks), 8 waves
    in two ping-pong groups (two waves per SIMD), and the wave-specialised 4 producer + 12 consumer waves on a
    192x256 tile (kernels/gemm/bf16fp32/mi350x/micros/producer_consumer in the reference). Same tile format,
    identical bits."""
    out = {}
    g = torch.Generator(device=dev).manual_seed(0)
    a = torch.randn(n, n, device=dev, generator=g)
    b = torch.randn(n, n, device=dev, generator=g)
    C = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    tf = lambda ms: round(2.0 * n ** 3 / (ms * 1e-3) / 1e12, 1)
    A8, sa = hk.quant.quantize_fp8_per_tensor(a)
    B8, sb = hk.quant.quantize_fp8_per_tensor(b)
    out["fp8"] = {name: tf(_timeit(torch, lambda: hk.tk_kernel.dispatch_fp8_gemm(A8, B8, C, sa, sb, variant=v), warmup, iters)[1])
                  for name, v in (("4wave_interleave", 4), ("8wave_pingpong", 1), ("producer_consumer_12c4p", 7))}
    Ab, Bb = a.to(torch.bfloat16), b.to(torch.bfloat16)
    out["bf16"] = {name: tf(_timeit(torch, lambda: hk.tk_kernel.dispatch_bf16_gemm(Ab, Bb, C, variant=v), warmup, iters)[1])
                   for name, v in (("4wave_interleave", 1), ("8wave_pingpong", 4), ("producer_consumer_12c4p", 5))}
    Ap, As = hk.quant.quantize_mxfp4(a)
    Bp, Bs = hk.quant.quantize_mxfp4(b)
    out["mxfp4"] = {name: tf(_timeit(torch, lambda: hk.tk_kernel.dispatch_mxfp4_gemm(Ap, As, Bp, Bs, C, variant=v), warmup, iters)[1])
                    for name, v in (("4wave_interleave", 1), ("8wave_pingpong", 4), ("producer_consumer_12c4p", 5))}
    out["workload"] = f"M=N=K={n}, TFLOP/s"
    return out


# ------------------------------------------------------------------------------------- MoE layers
def bench_moe_mxfp4(torch, hk, warmup, iters, dev, graph=True):
    import numpy as np

    from oracle import formats as F
    from oracle import gemm as OG
    from oracle import moe as OM

    T, E, k, H, I = 4096, 128, 4, 2880, 2880
    g = torch.Generator(device=dev).manual_seed(0)
    x = torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device=dev, generator=g)
    pitch = (H // 32 + 7) // 8 * 8
    w13p = torch.empty((E, 2 * I, H // 2), dtype=torch.uint8, device=dev)
    w13s = torch.empty((E, 2 * I, pitch), dtype=torch.uint8, device=dev)
    w2p = torch.empty((E, H, I // 2), dtype=torch.uint8, device=dev)
    w2s = torch.empty((E, H, pitch), dtype=torch.uint8, device=dev)
    for e in range(E):
        a, s = hk.quant.quantize_mxfp4(torch.randn(2 * I, H, device=dev, generator=g) * 0.02)
        w13p[e], w13s[e] = a, hk.quant.pad_scales(s)
        a, s = hk.quant.quantize_mxfp4(torch.randn(H, I, device=dev, generator=g) * 0.02)
        w2p[e], w2s[e] = a, hk.quant.pad_scales(s)
    W = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(w13p, w13s, w2p, w2s)
    # the oracle's inputs for a sample of tokens: their routing and the plain weights of the experts they use
    sel = np.arange(5, T, T // 32)[:32]
    ids_s, w_s = OM.topk_softmax(logits[torch.from_numpy(sel).to(dev)].cpu().numpy(), k)
    used = np.unique(ids_s)
    ut = torch.from_numpy(used.astype(np.int64)).to(dev)
    plain = [t[ut].cpu().numpy() for t in (w13p, w13s[:, :, :H // 32], w2p, w2s[:, :, :I // 32])]
    del w13p, w13s, w2p, w2s
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=dev)
    y = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    call = lambda: hk.tk_kernel.dispatch_moe_mxfp4(x, logits, W, None, None, None, y, k, ws)
    _, kern = _timeit(torch, call, warmup, iters)
    # parity spot check (outside the timed region)
    remap = {int(e): i for i, e in enumerate(used)}
    ids_l = np.vectorize(remap.get)(ids_s).astype(np.int32)
    st = torch.from_numpy(sel).to(dev)
    want, _ = OM.moe_mxfp4_forward(F.bf16_to_f32(_np_bits(x[st])), ids_l, w_s, *plain)
    got = y[st].float().cpu().numpy()
    rel = OG.rel_fro_error(got, F.bf16_to_f32(want))
    assert float(np.abs(got).max()) > 0.0 and np.isfinite(got).all(), "MoE output sample is empty or not finite"
    # (the FP4 x FP4 products and their fp32 sums are exact for these magnitudes whatever the order of summation,
    # so a relative error of exactly 0 against the oracle is the expected reading here, not an empty comparison)
    # the layer's launches replayed from a HIP graph (no host work or launch gaps between them)
    kern_graph = _timeit_graph(torch, call, y, iters) if graph else None
    flop = 2.0 * T * k * (H * 2 * I + I * H)
    tf = flop / (kern * 1e-3) / 1e12
    # algorithmic bytes: every expert's weights and scales once (unpadded: 4-bit elements + one e8m0 byte
    # per 32), x in, y out (the pre-shuffled tensors pad K 2880 -> 3072 with zeros that are never fetched)
    compulsory = E * 3 * I * H * (0.5 + 1.0 / 32) + 2 * T * H * 2
    # the same layer with the GPT-OSS expert epilogues: biases and clamped SwiGLU (the row order of
    # the source weights was resolved by the pre-shuffle, so the same shuffled weights serve)
    b13 = torch.randn(E, 2 * I, device=dev, generator=g)
    b2 = torch.randn(E, H, device=dev, generator=g)
    _, kern_oai = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_mxfp4(
        x, logits, W, None, None, None, y, k, ws, bias13=b13, bias2=b2, activation="swiglu_oai"), warmup, iters)
    want_oai, _ = OM.moe_mxfp4_forward(F.bf16_to_f32(_np_bits(x[st])), ids_l, w_s, *plain, bias13=b13[ut].cpu().numpy(),
                                       bias2=b2[ut].cpu().numpy(), activation="swiglu_oai")
    rel_oai = OG.rel_fro_error(y[st].float().cpu().numpy(), F.bf16_to_f32(want_oai))
    # the same layer with MXFP8 activations (W4A8: mixed fp4 x fp8 MFMA), checked against the oracle on the sample
    ws8 = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k, act_format="mxfp8"), dtype=torch.uint8,
                      device=dev)
    call8 = lambda: hk.tk_kernel.dispatch_moe_mxfp4(x, logits, W, None, None, None, y, k, ws8, act_format="mxfp8")
    _, kern_a8 = _timeit(torch, call8, warmup, iters)
    want8, _ = OM.moe_mxfp4_forward(F.bf16_to_f32(_np_bits(x[st])), ids_l, w_s, *plain, act_format="mxfp8")
    rel8 = OG.rel_fro_error(y[st].float().cpu().numpy(), F.bf16_to_f32(want8))
    return {"workload": "moe_mxfp4 T=4096 H=2880 I=2880 E=128 top-4 softmax, MXFP4 activations and weights "
                        "(top-k, sort + activation quantization in one launch, 2 grouped GEMMs, un-permute)",
            "ms": round(kern, 5), "tflops": round(tf, 1), "frac_of_mxfp4_peak": round(tf / PEAK_FP4, 4),
            "compulsory_GB": round(compulsory / 1e9, 3), "rel_fro_err_vs_oracle_32_tokens": rel,
            "roofline": _roofline("hbm", compulsory / (kern * 1e-3) / 1e9, PEAK_HBM, "GB/s",
                                  "whole layer (5 launches); dominant: moe_mxfp4 gate+up grouped GEMM",
                                  _traffic("moe_mxfp4")),
            "ms_graph_replay": round(kern_graph, 5) if graph else None, "ms_with_biases_and_clamped_swiglu": round(kern_oai, 5),
            "rel_fro_err_biases_and_clamped_swiglu_vs_oracle_32_tokens": rel_oai,
            "ms_with_mxfp8_activations": round(kern_a8, 5), "rel_fro_err_mxfp8_activations_vs_oracle_32_tokens": rel8}


def cpu_baseline_moe_mxfp4(torch, hk, dev):
    """The CPU oracle's MXFP4 MoE layer (dequantize + fp32 matmuls, expert by expert) timed on a 1/16
    sample of the workload: 8 of the 128 experts and 256 of the 4096 tokens at the full H = I = 2880,
    top-4 routing, i.e. the same 128 rows per expert. Weights are quantized on the GPU beforehand;
    only the oracle's forward pass is timed."""
    import numpy as np

    from oracle import formats as F
    from oracle import moe as OM

    T, E, k, H, I = 256, 8, 4, 2880, 2880
    g = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device=dev, generator=g).cpu().numpy()
    q13 = [hk.quant.quantize_mxfp4(torch.randn(2 * I, H, device=dev, generator=g) * 0.02) for _ in range(E)]
    q2 = [hk.quant.quantize_mxfp4(torch.randn(H, I, device=dev, generator=g) * 0.02) for _ in range(E)]
    w13p = np.stack([a.cpu().numpy() for a, _ in q13]); w13s = np.stack([b.cpu().numpy() for _, b in q13])
    w2p = np.stack([a.cpu().numpy() for a, _ in q2]); w2s = np.stack([b.cpu().numpy() for _, b in q2])
    xf = F.bf16_to_f32(_np_bits(x))
    ids, w = OM.topk_softmax(logits, k)
    best = float("inf")
    for _ in range(2):
        t0 = time.perf_counter()
        OM.moe_mxfp4_forward(xf, ids, w, w13p, w13s, w2p, w2s)
        best = min(best, time.perf_counter() - t0)
    flop = 2.0 * T * k * (H * 2 * I + I * H)
    return {"value": round(flop / best / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count() or 1, "kind": "port",
            "sample": f"oracle MoE forward on 8 of 128 experts x 256 of 4096 tokens (same rows per expert), best of 2: {best:.2f} s"}


def bench_moe_fp8blk(torch, hk, warmup, iters, dev, plain_weights=False):
    import numpy as np

    from oracle import formats as F
    from oracle import gemm as OG
    from oracle import moe as OM

    T, E, k, H, I, G, KG = 8192, 256, 8, 7168, 2048, 8, 4
    g = torch.Generator(device=dev).manual_seed(0)
    xq, xs = hk.quant.quantize_fp8_blocks(torch.randn(T, H, device=dev, generator=g), 1, 128)
    logits = torch.randn(T, E, device=dev, generator=g)
    w13q = torch.empty((E, 2 * I, H), dtype=torch.float8_e4m3fn, device=dev)
    w13s = torch.empty((E, 2 * I // 128, H // 128), dtype=torch.float32, device=dev)
    w2q = torch.empty((E, H, I), dtype=torch.float8_e4m3fn, device=dev)
    w2s = torch.empty((E, H // 128, I // 128), dtype=torch.float32, device=dev)
    for e in range(E):  # per expert: never more than one expert in fp32
        w13q[e], w13s[e] = hk.quant.quantize_fp8_blocks(torch.randn(2 * I, H, device=dev, generator=g) * 0.02, 128, 128)
        w2q[e], w2s[e] = hk.quant.quantize_fp8_blocks(torch.randn(H, I, device=dev, generator=g) * 0.02, 128, 128)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=dev)
    y = torch.empty((T, H), dtype=torch.bfloat16, device=dev)
    # the oracle's inputs for four tokens: their routing and the plain weights of the experts they use
    sel = np.array([3, 2731, 5461, T - 1])
    st = torch.from_numpy(sel).to(dev)
    ids_s, w_s = OM.topk_grouped_sigmoid(logits[st].cpu().numpy(), None, k, G, KG, 1.0)
    used = np.unique(ids_s)
    remap = {int(e): i for i, e in enumerate(used)}
    ids_l = np.vectorize(remap.get)(ids_s).astype(np.int32)
    ut = torch.from_numpy(used.astype(np.int64)).to(dev)
    plain = [w13q[ut].view(torch.uint8).cpu().numpy(), w13s[ut].cpu().numpy(),
             w2q[ut].view(torch.uint8).cpu().numpy(), w2s[ut].cpu().numpy()]
    # algorithmic bytes: weights and their scales once, x (e4m3 + scales) in, y out
    compulsory = w13q.numel() + w2q.numel() + 4 * (w13s.numel() + w2s.numel()) + T * H + 4 * xs.numel() + T * H * 2
    # weights in the pre-shuffled layout (offline step, once per checkpoint): the fast path
    # (--fp8blk-plain-weights: the caller's [E, rows, K] layout instead, served by the LDS-staged kernel)
    if plain_weights:
        _, kern = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_fp8blk(xq, xs, logits, None, w13q, w13s, w2q, w2s, y,
                                                                          k, G, KG, 1.0, ws), warmup, iters)
    else:
        W = hk.tk_kernel.MoeFp8BlkShuffledWeights.from_plain(w13q, w13s, w2q, w2s)
        torch.cuda.synchronize()
        del w13q, w2q
        torch.cuda.empty_cache()
        _, kern = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_fp8blk(xq, xs, logits, None, W, None, None, None, y,
                                                                          k, G, KG, 1.0, ws), warmup, iters)
    # parity spot check (outside the timed region)
    want = F.bf16_to_f32(OM.moe_fp8blk_forward(xq[st].view(torch.uint8).cpu().numpy(), xs[st].cpu().numpy(), ids_l, w_s,
                                               *plain))
    rel = OG.rel_fro_error(y[st].float().cpu().numpy(), want)
    flop = 2.0 * T * k * (H * 2 * I + I * H)
    tf = flop / (kern * 1e-3) / 1e12
    return {"workload": "moe_fp8blk T=8192 H=7168 I=2048 E=256 top-8 sigmoid (8 groups / top-4), e4m3 with "
                        "1x128 / 128x128 fp32 scales, " + ("plain weight layout" if plain_weights else "pre-shuffled weights"),
            "ms": round(kern, 5), "tflops": round(tf, 1), "frac_of_fp8_peak": round(tf / PEAK_FP8, 4),
            "compulsory_GB": round(compulsory / 1e9, 3), "rel_fro_err_vs_oracle_4_tokens": rel,
            "roofline": _roofline("hbm", compulsory / (kern * 1e-3) / 1e9, PEAK_HBM, "GB/s",
                                  "whole layer (7 launches); dominant: moe_fp8blk gate+up grouped GEMM",
                                  None if plain_weights else _traffic("moe_fp8blk"),
                                  note="MFMA time at peak 1.15 ms vs 1.43 ms for the bytes: HBM is the binding roofline")}


def cpu_baseline_moe_fp8blk(torch, hk, dev):
    """The CPU oracle's FP8 block-scaled MoE forward on a 1/32 sample of the DeepSeek-V3-like workload:
    8 of the 256 experts and 256 of the 8192 tokens at the full H = 7168, I = 2048, every token routed
    to all 8 experts (top-8), i.e. the workload's 256 rows per expert. Only the forward pass is timed."""
    import numpy as np

    from oracle import moe as OM

    T, E, k, H, I = 256, 8, 8, 7168, 2048
    g = torch.Generator(device=dev).manual_seed(2)
    xq, xs = hk.quant.quantize_fp8_blocks(torch.randn(T, H, device=dev, generator=g), 1, 128)
    q13 = [hk.quant.quantize_fp8_blocks(torch.randn(2 * I, H, device=dev, generator=g) * 0.02, 128, 128) for _ in range(E)]
    q2 = [hk.quant.quantize_fp8_blocks(torch.randn(H, I, device=dev, generator=g) * 0.02, 128, 128) for _ in range(E)]
    w13q = np.stack([a.view(torch.uint8).cpu().numpy() for a, _ in q13]); w13s = np.stack([b.cpu().numpy() for _, b in q13])
    w2q = np.stack([a.view(torch.uint8).cpu().numpy() for a, _ in q2]); w2s = np.stack([b.cpu().numpy() for _, b in q2])
    logits = torch.randn(T, E, device=dev, generator=g).cpu().numpy()
    ids, w = OM.topk_grouped_sigmoid(logits, None, k, 1, 1, 1.0)
    xqn, xsn = xq.view(torch.uint8).cpu().numpy(), xs.cpu().numpy()
    best = float("inf")
    for _ in range(2):
        t0 = time.perf_counter()
        OM.moe_fp8blk_forward(xqn, xsn, ids, w, w13q, w13s, w2q, w2s)
        best = min(best, time.perf_counter() - t0)
    flop = 2.0 * T * k * (H * 2 * I + I * H)
    return {"value": round(flop / best / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count() or 1, "kind": "port",
            "sample": f"oracle MoE forward on 8 of 256 experts x 256 of 8192 tokens (256 rows per expert), best of 2: {best:.2f} s"}


# ------------------------------------------------------------------------------------- routing
def bench_routing(torch, hk, warmup, iters, dev):
    out = []
    g = torch.Generator(device=dev).manual_seed(0)
    T, E, k = 262144, 128, 4
    logits = torch.randn(T, E, device=dev, generator=g)
    ids = torch.empty((T, k), dtype=torch.int32, device=dev)
    w = torch.empty((T, k), dtype=torch.float32, device=dev)
    _, ms = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_topk_softmax(logits, ids, w), warmup, iters)
    by = T * E * 4 + T * k * 8
    out.append({"kernel": "topk_softmax T=262144 E=128 k=4", "ms": round(ms, 5),
                "roofline": _roofline("hbm", by / ms / 1e6, PEAK_HBM, "GB/s", "moe_topk_softmax_kernel<16>")})
    # the DeepSeek-V3 router: sigmoid scores + selection bias, 8 groups / top-4 groups, top-8
    Tg, Eg, kg = 65536, 256, 8
    lg = torch.randn(Tg, Eg, device=dev, generator=g)
    bg = torch.randn(Eg, device=dev, generator=g) * 0.05
    idg = torch.empty((Tg, kg), dtype=torch.int32, device=dev)
    wg = torch.empty((Tg, kg), dtype=torch.float32, device=dev)
    _, ms = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_topk_grouped_sigmoid(lg, bg, idg, wg, 8, 4, 2.5),
                    warmup, iters)
    by = Tg * Eg * 4 + Tg * kg * 8
    out.append({"kernel": "topk_grouped_sigmoid T=65536 E=256 k=8 (8 groups / top-4)", "ms": round(ms, 5),
                "roofline": _roofline("hbm", by / ms / 1e6, PEAK_HBM, "GB/s", "moe_topk_grouped_sigmoid16_kernel<16>")})
    del lg, idg, wg
    ss = torch.empty(T * k, dtype=torch.int32, device=dev)
    off = torch.empty(E + 1, dtype=torch.int32, device=dev)
    inv = torch.empty(T * k, dtype=torch.int32, device=dev)
    wsb = torch.empty(hk.tk_kernel.moe_sort_workspace_bytes(T, k, E), dtype=torch.uint8, device=dev)
    _, ms = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_sort(ids, ss, off, inv, wsb), warmup, iters)
    by = T * k * 4 + (2 * T * k + E + 1) * 4  # ids in; sorted_slots, slot_to_pos and offsets out
    out.append({"kernel": "moe_sort T*k=1048576 E=128", "ms": round(ms, 5),
                "roofline": _roofline("hbm", by / ms / 1e6, PEAK_HBM, "GB/s", "moe_sort (count, scan, scatter)")})
    T2, k2, H = 8192, 8, 7168
    o = torch.randn(T2 * k2, H, device=dev, generator=g).to(torch.bfloat16)
    w2 = torch.rand(T2, k2, device=dev, generator=g)
    inv2 = torch.randperm(T2 * k2, device=dev, generator=g).to(torch.int32)
    y = torch.empty(T2, H, dtype=torch.bfloat16, device=dev)
    _, ms = _timeit(torch, lambda: hk.tk_kernel.dispatch_moe_unpermute(o, w2, inv2, y), warmup, iters)
    by = T2 * k2 * H * 2 + T2 * H * 2
    out.append({"kernel": "moe_unpermute T=8192 k=8 H=7168", "ms": round(ms, 5),
                "roofline": _roofline("hbm", by / ms / 1e6, PEAK_HBM, "GB/s", "moe_unpermute_kernel")})
    return out


def mfma_ceiling(torch, Aq, dev):
    """Register-only FP8 MFMA loop on operand bits drawn from the benchmark's own A matrix (bench-only
    library libhk355_bench.so, built with the product library but not part of it)."""
    path = os.path.join(ROOT, "hipkittens_amd", "libhk355_bench.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.hkbench_mfma_rate.restype = ctypes.c_int
    lib.hkbench_mfma_rate.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                      ctypes.c_void_p]
    pattern = Aq.view(torch.uint8).flatten()[:65536].contiguous().view(torch.int32)
    blocks, iters = 1024, 2000
    sink = torch.empty(blocks * 512, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream

    def run():
        rc = lib.hkbench_mfma_rate(pattern.data_ptr(), sink.data_ptr(), blocks, iters, 0, ctypes.c_void_p(st))
        assert rc == 0

    _, ms = _timeit(torch, run, 2, 5)
    return blocks * 8 * iters * 32 * 65536.0 / (ms * 1e-3) / 1e12


def mfma_issue_probe(torch, dev):
    """Shader clocks per MFMA of a register-only loop, one wave per SIMD, with 0..6 other instructions behind
    each MFMA (bench-only library; the slot plans of the tile kernels are sized by this table)."""
    path = os.path.join(ROOT, "hipkittens_amd", "libhk355_bench.so")
    lib = ctypes.CDLL(path)
    lib.hkbench_mfma_issue.restype = ctypes.c_int
    lib.hkbench_mfma_issue.argtypes = [ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 4 + [ctypes.c_void_p]
    pattern = torch.zeros(1024, dtype=torch.int32, device=dev)
    out = torch.zeros(2, dtype=torch.int64, device=dev)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    iters = 2000
    modes = {0: ("v_mfma_f32_16x16x128_f8f6f4 fp8", 32), 1: ("v_mfma_scale_f32_16x16x128_f8f6f4 fp4", 32),
             2: ("v_mfma_scale_f32_32x32x64_f8f6f4 fp4", 12)}
    kinds = {0: ("v_add_u32", range(0, 7)), 1: ("s_add_u32", (2, 4, 6)), 2: ("ds_read_b128", (1, 2, 3))}
    table = {}
    for mode, (name, per_trip) in modes.items():
        row = {}
        for kind, (kname, counts) in kinds.items():
            clocks = {}
            for kops in counts:
                for _ in range(2):   # the second launch is the measurement
                    assert lib.hkbench_mfma_issue(pattern.data_ptr(), out.data_ptr(), mode, kind, kops, iters, st) == 0
                    torch.cuda.synchronize()
                clocks[str(kops)] = round(out[0].item() / (iters * per_trip), 1)
            row[kname] = clocks
        table[name] = row
    return {"unit": "shader clocks per MFMA, one wave per SIMD, all-zero operands; key = other instructions per MFMA",
            "clocks": table}


LEGS = ("ceiling", "sweep", "reference_inputs", "decode", "bf16", "library", "mxfp4", "mxfp4_decode", "schedules",
        "moe_mxfp4", "moe_fp8blk", "routing", "issue_probe")
# legs that only run when named with --only
OPT_IN_LEGS = ("issue_probe",)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--size", type=int, default=8192)
    ap.add_argument("--settle-ms", type=float, default=600.0,
                    help="untimed repetitions of the headline launch before --warmup, until this many ms have passed")
    ap.add_argument("--only-headline", action="store_true")
    ap.add_argument("--only", type=str, default="", help="comma-separated legs of `extra` to run: " + ",".join(LEGS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--traffic-calibration", action="store_true")
    ap.add_argument("--collect-traffic", type=str, default="", metavar="DIR",
                    help="rewrite profiles/traffic.json from the rocprofv3 counter runs under DIR (no GPU needed)")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph timings (for runs under a profiler)")
    ap.add_argument("--fp8blk-plain-weights", action="store_true",
                    help="run the FP8-block MoE leg on the plain weight layout (the LDS-staged kernel)")
    args = ap.parse_args()
    if args.collect_traffic:
        out = collect_traffic(args.collect_traffic)
        print(json.dumps({k: v["total_bytes"] for k, v in out["legs"].items()}))
        return 0
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
    legs = set(LEGS) - set(OPT_IN_LEGS) if not args.only else set(args.only.split(","))
    if args.only_headline:
        legs = set()
    unknown = legs - set(LEGS)
    if unknown:
        print(f"bench.py: unknown legs {sorted(unknown)}", file=sys.stderr)
        return 2

    if args.traffic_calibration:
        # For the HBM-traffic counters: a plain copy of known size (1 GiB read + 1 GiB written per
        # launch) next to the headline GEMM, nothing else, so that the FETCH_SIZE / WRITE_SIZE
        # readings of the GEMM can be scaled by what the same counters read for the copy.
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        bench_fp8(torch, hk, n, 5, 5, dev)
        torch.cuda.synchronize()
        print(json.dumps({"traffic_calibration": {"copy_bytes_read": 1 << 30, "copy_bytes_written": 1 << 30,
                                                  "copy_launches": 5, "gemm_launches": 10, "n": n}}))
        return 0

    head = bench_fp8(torch, hk, n, args.warmup, args.steps, dev, keep=True, settle_ms=args.settle_ms)
    tflops = 2.0 * n ** 3 / (head["wall_ms"] * 1e-3) / 1e12

    # parity spot check against the oracle on a row sample (outside the timed region)
    from oracle import gemm as OG

    rows = torch.arange(0, n, max(1, n // 16), device=dev)
    ref = OG.fp8_gemm(head["A"].view(torch.uint8)[rows].cpu().numpy(), head["B"].view(torch.uint8).cpu().numpy(),
                      head["sa"], head["sb"])
    rel = OG.rel_fro_error(head["C"][rows].float().cpu().numpy(), ref)

    extra = {}
    ceiling = None
    quick_w, quick_i = 50, 100
    if "ceiling" in legs:
        ceiling = mfma_ceiling(torch, head["A"], dev)
        extra["mfma_fp8_ceiling_tflops_for_this_data"] = round(ceiling, 1) if ceiling else None
    del head["A"], head["B"], head["C"]
    torch.cuda.empty_cache()
    if "sweep" in legs:
        sweep = {m: bench_fp8(torch, hk, m, 500, 100, dev, graph=m <= 4096 and not args.no_graph)  # the reference's protocol
                 for m in (1024, 2048, 4096, 16384)}
        # per call through the Python boundary (about 9 us of host time per call bounds the small sizes) ...
        extra["fp8_gemm_sweep_tflops"] = {str(m): round(r["tflops"], 1) for m, r in sweep.items()}
        # ... and the same calls replayed from a HIP graph (GPU time only, like the reference's C++ loop)
        extra["fp8_gemm_sweep_tflops_graph_replay"] = {
            str(m): round(r["tflops_graph"], 1) for m, r in sweep.items() if "tflops_graph" in r}
        del sweep
        torch.cuda.empty_cache()
    if "reference_inputs" in legs:
        extra["fp8_gemm_reference_inputs"] = bench_fp8_reference_inputs(torch, hk, n, 500, 100, dev)
    if "decode" in legs:
        extra["fp8_gemm_decode"] = bench_fp8_decode(torch, hk, 50, 50, dev, graph=not args.no_graph)
    if "bf16" in legs:
        extra["bf16_gemm"] = bench_bf16(torch, hk, 8192, 500, 100, dev)
    if "library" in legs:
        extra["library_on_this_box_8192"] = bench_library_baselines(torch, 8192, 500, 100, dev)
        torch.cuda.empty_cache()
    if "mxfp4" in legs:
        extra["mxfp4_gemm"] = bench_mxfp4(torch, hk, 8192, 500, 100, dev)
    if "mxfp4_decode" in legs:
        extra["mxfp4_gemm_decode"] = bench_mxfp4_decode(torch, hk, 50, 50, dev, graph=not args.no_graph)
    if "schedules" in legs:
        extra["gemm_schedules_8192"] = bench_schedules(torch, hk, 8192, 200, 100, dev)
        torch.cuda.empty_cache()
    if "moe_mxfp4" in legs:
        extra["moe_mxfp4"] = bench_moe_mxfp4(torch, hk, quick_w, quick_i, dev, graph=not args.no_graph)
        torch.cuda.empty_cache()
        if not args.no_cpu_baseline:
            extra["moe_mxfp4"]["cpu_baseline"] = cpu_baseline_moe_mxfp4(torch, hk, dev)
    if "moe_fp8blk" in legs:
        extra["moe_fp8blk"] = bench_moe_fp8blk(torch, hk, 10, 20, dev, args.fp8blk_plain_weights)
        torch.cuda.empty_cache()
        if not args.no_cpu_baseline:
            extra["moe_fp8blk"]["cpu_baseline"] = cpu_baseline_moe_fp8blk(torch, hk, dev)
    if "routing" in legs:
        extra["routing"] = bench_routing(torch, hk, quick_w, quick_i, dev)
    if "issue_probe" in legs:
        extra["mfma_issue_probe"] = mfma_issue_probe(torch, dev)

    cpu = None
    if not args.no_cpu_baseline:
        r = OG.cpu_baseline_fp8_gemm(n, n, n, seed=0, repeats=12)
        cpu = {"value": round(r["tflops"], 4), "unit": "TFLOP/s", "cores": r["threads"], "kind": "port",
               "sample": f"12 full {n}x{n}x{n} dequantize+fp32 matmul passes (torch CPU), best {r['seconds']:.2f} s"}

    out = {
        "metric": "FP8 e4m3 GEMM 8192^3 throughput" if n == 8192 else f"FP8 e4m3 GEMM {n}^3 throughput",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_launches": head["settle_launches"],
        "ms_per_step": round(head["wall_ms"], 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": round(tflops / 3327.46, 4) if n == 8192 else None,
        "dtype": "fp8_e4m3 (fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {"workload": f"fp8_gemm M=N=K={n}, A row-major, B [N,K], per-tensor fp32 scales, randn inputs"},
        "pct_of_fp8_peak": round(100.0 * tflops / PEAK_FP8, 2),
        "rel_fro_err_vs_oracle": rel,
        "roofline": _roofline("mfma", head["tflops"], PEAK_FP8, "TFLOP/s", "fp8_gemm_4wave_ring_kernel",
                              _traffic("fp8_gemm_8192") if n == 8192 else None, kernel_ms=round(head["kernel_ms"], 5),
                              # the register-only MFMA loop on the same operand bits: what the power limit
                              # leaves of the nominal peak on this data
                              measured_mfma_ceiling=round(ceiling, 1) if ceiling else None,
                              frac_of_measured_ceiling=round(head["tflops"] / ceiling, 4) if ceiling else None),
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
