"""CPU oracle, part 2: the quantized GEMMs as dequantize + matmul.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

C = A . B^T with both operands K-contiguous and fp32 accumulation is the reference's
mma_ABt (include/ops/warp/register/tile/mma.cuh:382-422; fp8 only exists as ABt,
:397-398). The reference applies no scales (mfma scale operands are zero, :112-125);
the per-tensor scales follow the hipBLASLt convention it benchmarks against
(analysis/baselines/README.md:172-174: scalar scaleA/scaleB, bf16 output).
Error metrics restate kernels/attn/gqa/test_python.py:46-57 (relative L2 / Frobenius)
and kernels/gemm/bf16fp32/mi350x/test_python.py:105-117 (max/mean abs, count above 1 %).

Pinned by: identity/power-of-two known answers, scale linearity, float64 brute force on
small shapes (tests/test_oracle_gemm.py).
"""
from __future__ import annotations

import time

import numpy as np

from . import formats as F


def fp8_gemm(a_codes, b_codes, scale_a=1.0, scale_b=1.0, acc=np.float32) -> np.ndarray:
    """fp32 result (not yet rounded to bf16) of (sa*A)(sb*B)^T from e4m3 codes."""
    a = F.e4m3_decode(a_codes).astype(acc)
    b = F.e4m3_decode(b_codes).astype(acc)
    c = a @ b.T
    return (c * acc(np.float32(scale_a) * np.float32(scale_b))).astype(np.float32)


def fp8_gemm_bf16(a_codes, b_codes, scale_a=1.0, scale_b=1.0) -> np.ndarray:
    """bf16 bit pattern (uint16) of the result, RNE."""
    return F.bf16_round(fp8_gemm(a_codes, b_codes, scale_a, scale_b))


def mxfp4_gemm(a_packed, a_scales, b_packed, b_scales, acc=np.float32) -> np.ndarray:
    a = F.dequantize_mxfp4(a_packed, a_scales).astype(acc)
    b = F.dequantize_mxfp4(b_packed, b_scales).astype(acc)
    return (a @ b.T).astype(np.float32)


def bf16_gemm(a_bits, b_bits, acc=np.float32) -> np.ndarray:
    """fp32 result (not yet rounded to bf16) of A B^T for operands given as bf16 bit patterns
    (uint16). Follows the reference's check C = A @ B.T
    (kernels/gemm/bf16fp32/mi350x/test_python.py:17,32)."""
    a = F.bf16_to_f32(np.asarray(a_bits, dtype=np.uint16)).astype(acc)
    b = F.bf16_to_f32(np.asarray(b_bits, dtype=np.uint16)).astype(acc)
    return (a @ b.T).astype(np.float32)


def rel_fro_error(out: np.ndarray, ref: np.ndarray) -> float:
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.sqrt((ref * ref).sum())
    return float(np.sqrt(((out - ref) ** 2).sum()) / (den if den > 0 else 1.0))


def error_stats(out: np.ndarray, ref: np.ndarray) -> dict:
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.abs(out - ref)
    return {
        "max_abs": float(d.max()) if d.size else 0.0,
        "mean_abs": float(d.mean()) if d.size else 0.0,
        "count_gt_1pct": int((d > 0.01 * np.abs(ref)).sum()),
        "rel_fro": rel_fro_error(out, ref),
    }


def cpu_baseline_fp8_gemm(M: int, N: int, K: int, seed: int = 0, repeats: int = 1) -> dict:
    """Time PyTorch-CPU dequantize + fp32 matmul on all host cores for an MxNxK problem
    (the north star's CPU counterpart of the GPU path). Returns seconds and TFLOP/s."""
    import os

    import torch

    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(0, 256, (M, K), dtype=torch.uint8, generator=g)
    b = torch.randint(0, 256, (N, K), dtype=torch.uint8, generator=g)
    # keep NaN codes out of the timing inputs
    a[(a & 0x7F) == 0x7F] = 0
    b[(b & 0x7F) == 0x7F] = 0
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        af = a.view(torch.float8_e4m3fn).to(torch.float32) * 0.5
        bf = b.view(torch.float8_e4m3fn).to(torch.float32) * 0.25
        c = (af @ bf.t()).to(torch.bfloat16)
        best = min(best, time.perf_counter() - t0)
    del c
    return {"seconds": best, "tflops": 2.0 * M * N * K / best / 1e12, "threads": threads}
