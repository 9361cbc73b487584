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
    # tensor / tensor: a correctly rounded division on every device (dividing by a Python scalar
    # may be turned into a multiplication by the reciprocal)
    scale = torch.where(amax > 0, amax / torch.full_like(amax, E4M3_MAX), torch.ones_like(amax)).to(torch.float32)
    return to_e4m3_saturating(xf / scale), float(scale)


def quantize_mxfp4(x: torch.Tensor):
    """OCP MX (v1.0) quantization along the last dim in blocks of 32: shared exponent
    e = floor(log2(amax)) - 2 stored as e8m0 byte e + 127, elements e2m1(x / 2^e) (round to
    nearest even, saturating at 6). Returns (packed uint8 [..., K/2] with the even k in the low
    nibble, scales uint8 [..., K/32])."""
    K = x.shape[-1]
    if K % 32:
        raise RuntimeError("quantize_mxfp4: last dimension must be a multiple of 32")
    xb = x.float().reshape(*x.shape[:-1], K // 32, 32)
    amax = xb.abs().amax(dim=-1)
    _, ex = torch.frexp(amax)
    e = (ex - 3).clamp(-127, 127)
    e = torch.where(amax > 0, e, torch.zeros_like(e))
    scaled = torch.ldexp(xb, (-e).unsqueeze(-1))
    a = scaled.abs().clamp(max=6.0)
    code = torch.where(a < 2.0, torch.round(a * 2.0),
                       torch.where(a < 4.0, 4.0 + torch.round(a - 2.0), 6.0 + torch.round((a - 4.0) * 0.5)))
    code = code.to(torch.uint8) | (torch.signbit(scaled).to(torch.uint8) << 3)
    code = code.reshape(*x.shape[:-1], K)
    packed = code[..., 0::2] | (code[..., 1::2] << 4)
    return packed.contiguous(), (e + 127).to(torch.uint8).contiguous()


def pad_scales(scales: torch.Tensor, multiple: int = 8) -> torch.Tensor:
    """Pad the last dim of an e8m0 scale tensor to a multiple of `multiple` with the neutral byte
    127 (the row pitch the MoE kernels load scales with)."""
    n = scales.shape[-1]
    pad = (-n) % multiple
    if pad == 0:
        return scales.contiguous()
    fill = torch.full((*scales.shape[:-1], pad), 127, dtype=scales.dtype, device=scales.device)
    return torch.cat([scales, fill], dim=-1).contiguous()


def quantize_fp8_blocks(x: torch.Tensor, block_rows: int, block_cols: int):
    """e4m3 with one fp32 scale per block_rows x block_cols block of the last two dims
    (1 x 128 for activations, 128 x 128 for weights): scale = amax/448 (1 for an all-zero block).
    Both dims must be multiples of the block. Returns (e4m3 tensor, fp32 scales [..., R/br, C/bc])."""
    R, C = x.shape[-2:]
    if R % block_rows or C % block_cols:
        raise RuntimeError("quantize_fp8_blocks: dims must be multiples of the block")
    lead = x.shape[:-2]
    xb = x.float().reshape(*lead, R // block_rows, block_rows, C // block_cols, block_cols)
    amax = xb.abs().amax(dim=(-3, -1))
    s = torch.where(amax > 0, amax / torch.full_like(amax, E4M3_MAX), torch.ones_like(amax))
    q = (xb / s[..., :, None, :, None]).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return q.reshape(*lead, R, C).contiguous(), s.contiguous()
