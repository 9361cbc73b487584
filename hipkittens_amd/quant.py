"""Operand preparation with torch ops on the tensor's own device (CPU or GPU).

The reference converts inputs to fp8 on the host with HIP's saturating constructor
(kernels/gemm/fp8fp32/profile_utils.cpp:35-45, include/common/base_types.cuh:348-379).
torch's float8_e4m3fn cast rounds to nearest even like it but does not saturate, so
values are clamped to +-448 first.
"""
from __future__ import annotations

import torch

E4M3_MAX = 448.0


def to_e4m3_saturating(x: torch.Tensor) -> torch.Tensor:
    return x.float().clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)


def quantize_fp8_per_tensor(x: torch.Tensor):
    """(e4m3 tensor, fp32 scale) with scale = amax/448 so that x ~= q.float() * scale."""
    xf = x.float()
    amax = xf.abs().max()
    scale = torch.where(amax > 0, amax / E4M3_MAX, torch.ones_like(amax)).to(torch.float32)
    return to_e4m3_saturating(xf / scale), float(scale)
