"""Python boundary: `dispatch_*(inputs..., outputs...)` over the C ABI.

Mirrors the reference's pybind11 module `tk_kernel`
(kernels/gemm/bf16fp32/mi325x/256_256_64_16.cpp:233-237, used as
`tk_kernel.dispatch_micro(A, B, C)` in kernels/gemm/bf16fp32/mi350x/test_python.py:80-82):
positional torch tensors, outputs allocated by the caller and written in place, returns
None, launches asynchronously. Argument checks follow include/pyutils/pyutils.cuh:14-47
(must be a Tensor, contiguous, not on the CPU, at most 4 dims) and raise RuntimeError;
unlike the reference, dtypes and shapes are checked too. Launches go to torch's current
stream (the reference uses the null stream).
"""
from __future__ import annotations

import torch

from . import _lib


def _check_tensor(t, name: str, dtypes, ndim: int | None = None):
    if type(t).__name__ not in ("Tensor", "Parameter"):
        raise RuntimeError(f"{name}: expected a torch.Tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name}: tensor must be contiguous")
    if t.device.type == "cpu":
        raise RuntimeError(f"{name}: tensor must be on a GPU device")
    if t.dim() > 4:
        raise RuntimeError(f"{name}: expected at most 4 dimensions")
    if t.dtype not in dtypes:
        raise RuntimeError(f"{name}: dtype {t.dtype} not in {tuple(str(d) for d in dtypes)}")
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError(f"{name}: expected {ndim} dimensions, got {t.dim()}")


def _stream(t) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


_FP8 = (torch.float8_e4m3fn, torch.uint8)


def dispatch_fp8_gemm(A, B, C, scale_a: float = 1.0, scale_b: float = 1.0, variant: int = -1) -> None:
    """C[M,N] (bf16) = (scale_a*A[M,K]) @ (scale_b*B[N,K]).T, A and B e4m3, fp32 accumulation.

    `variant` -1 lets the library choose; 0/1/2 force a kernel (see include/hk355.h)."""
    _check_tensor(A, "A", _FP8, 2)
    _check_tensor(B, "B", _FP8, 2)
    _check_tensor(C, "C", (torch.bfloat16,), 2)
    M, K = A.shape
    N, Kb = B.shape
    if Kb != K or tuple(C.shape) != (M, N):
        raise RuntimeError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)}")
    if A.device != B.device or A.device != C.device:
        raise RuntimeError("A, B and C must be on the same device")
    lib = _lib.load_library()
    if variant < 0:
        st = lib.hk_fp8_gemm(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K,
                             float(scale_a), float(scale_b), _stream(A))
    else:
        st = lib.hk_fp8_gemm_variant(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K,
                                     float(scale_a), float(scale_b), int(variant), _stream(A))
    _lib.check(st, "dispatch_fp8_gemm")


def dispatch_micro(A, B, C) -> None:
    """The reference's GEMM entry point name: C = A @ B.T with unit scales."""
    dispatch_fp8_gemm(A, B, C, 1.0, 1.0)


_U8 = (torch.uint8,)
_FP4 = tuple(d for d in (torch.uint8, getattr(torch, "float4_e2m1fn_x2", None)) if d is not None)
_E8M0 = tuple(d for d in (torch.uint8, getattr(torch, "float8_e8m0fnu", None)) if d is not None)


def dispatch_mxfp4_gemm(A, A_scales, B, B_scales, C, variant: int = -1) -> None:
    """C[M,N] (bf16) = dequant(A) @ dequant(B).T for MXFP4 operands: A [M,K/2] packed e2m1
    (low nibble = even k), A_scales [M,K/32] e8m0, B [N,K/2], B_scales [N,K/32]."""
    _check_tensor(A, "A", _FP4, 2)
    _check_tensor(B, "B", _FP4, 2)
    _check_tensor(A_scales, "A_scales", _E8M0, 2)
    _check_tensor(B_scales, "B_scales", _E8M0, 2)
    _check_tensor(C, "C", (torch.bfloat16,), 2)
    M, Kh = A.shape
    N, Kh2 = B.shape
    K = 2 * Kh
    if Kh2 != Kh or K % 32 != 0 or tuple(A_scales.shape) != (M, K // 32) or \
            tuple(B_scales.shape) != (N, K // 32) or tuple(C.shape) != (M, N):
        raise RuntimeError(
            f"shape mismatch: A {tuple(A.shape)}, A_scales {tuple(A_scales.shape)}, B {tuple(B.shape)}, "
            f"B_scales {tuple(B_scales.shape)}, C {tuple(C.shape)}")
    if len({t.device for t in (A, A_scales, B, B_scales, C)}) != 1:
        raise RuntimeError("all tensors must be on the same device")
    lib = _lib.load_library()
    args = (A.data_ptr(), A_scales.data_ptr(), B.data_ptr(), B_scales.data_ptr(), C.data_ptr(), M, N, K)
    if variant < 0:
        st = lib.hk_mxfp4_gemm(*args, _stream(A))
    else:
        st = lib.hk_mxfp4_gemm_variant(*args, int(variant), _stream(A))
    _lib.check(st, "dispatch_mxfp4_gemm")
