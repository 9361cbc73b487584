"""ctypes loader for libhk355.so. There is no fallback: a missing library is an error."""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_size_t, c_void_p
from pathlib import Path

_LIB_PATH = Path(__file__).resolve().parent / "libhk355.so"
_lib = None

# name -> (restype, argtypes); one entry per symbol declared in include/hk355.h
SIGNATURES = {
    "hk_status_string": (ctypes.c_char_p, [c_int]),
    "hk_version": (c_int, []),
    "hk_gemm_tile_choice": (c_int, [c_int] * 5),
    "hk_fp8_gemm": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_void_p]),
    "hk_fp8_gemm_variant": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_int, c_void_p]),
    "hk_mxfp4_gemm": (c_int, [c_void_p] * 5 + [c_int] * 3 + [c_void_p]),
    "hk_mxfp4_gemm_variant": (c_int, [c_void_p] * 5 + [c_int] * 4 + [c_void_p]),
    "hk_mxfp4_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "hk_mxfp4_gemm_ws": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p] + [c_int] * 3 + [c_void_p, c_size_t, c_void_p]),
    "hk_mxfp4_gemm_pitched": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p] + [c_int] * 3 + [c_void_p]),
    "hk_bf16_gemm": (c_int, [c_void_p] * 3 + [c_int] * 3 + [c_void_p]),
    "hk_fp8_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "hk_bf16_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "hk_bf16_gemm_ws": (c_int, [c_void_p] * 3 + [c_int] * 3 + [c_void_p, c_size_t, c_void_p]),
    "hk_fp8_gemm_ws": (c_int, [c_void_p] * 3 + [c_int] * 3 + [c_float] * 2 + [c_void_p, c_size_t, c_void_p]),
    "hk_fp8_gemm_static_ws_max_bytes": (c_size_t, []),
    "hk_fp8_gemm_static_ws": (c_int, [c_void_p] * 3 + [c_int] * 3 + [c_float] * 2 + [c_void_p]),
    "hk_bf16_gemm_variant": (c_int, [c_void_p] * 3 + [c_int] * 4 + [c_void_p]),
    "hk_moe_topk_softmax": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "hk_moe_topk_grouped_sigmoid": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                            c_void_p, c_void_p, c_void_p]),
    "hk_moe_sort_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "hk_moe_sort": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                            c_void_p]),
    "hk_mxfp4_quantize_rows": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "hk_moe_unpermute": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "hk_moe_unpermute_add": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p,
                                     c_void_p]),
    "hk_moe_mxfp4_workspace_bytes": (c_size_t, [c_int] * 5),
    "hk_moe_mxfp4_experts": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                     c_int, c_void_p, c_size_t, c_void_p]),
    "hk_moe_mxfp4_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                     c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t,
                                     c_void_p]),
    "hk_moe_mxfp4_experts_ex": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                        c_int, c_void_p, c_void_p, c_int, c_float, c_float, c_int, c_void_p,
                                        c_size_t, c_void_p]),
    "hk_moe_mxfp4_forward_ex": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                        c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                        c_int, c_float, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "hk_mxfp8_quantize_rows": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "hk_moe_mxfp4_a8_workspace_bytes": (c_size_t, [c_int] * 5),
    "hk_moe_mxfp4_a8_experts": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                        c_void_p, c_int, c_float, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "hk_moe_mxfp4_a8_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_float,
                                        c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "hk_moe_mxfp4_preshuffle_bytes": (c_int, [c_int, c_int, c_int, c_int, ctypes.POINTER(c_size_t),
                                              ctypes.POINTER(c_size_t)]),
    "hk_moe_mxfp4_preshuffle": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                        c_void_p]),
    "hk_fp8_quantize_rows_1x128": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "hk_moe_fp8blk_workspace_bytes": (c_size_t, [c_int] * 5),
    "hk_moe_fp8blk_experts": (c_int, [c_void_p] * 11 + [c_int] * 5 + [c_void_p, c_size_t, c_void_p]),
    "hk_moe_fp8blk_experts_ex": (c_int, [c_void_p] * 11 + [c_int] * 5 + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "hk_moe_fp8blk_forward_ex": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p,
                                         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                         c_void_p, c_void_p, c_size_t, c_void_p]),
    "hk_moe_fp8blk_preshuffle_bytes": (c_int, [c_int, c_int, c_int, c_int, ctypes.POINTER(c_size_t)]),
    "hk_moe_fp8blk_preshuffle": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "hk_moe_fp8blk_experts_ex2": (c_int, [c_void_p] * 11 + [c_int] * 6 + [c_void_p, c_void_p, c_size_t, c_void_p]),
    "hk_moe_fp8blk_forward_ex2": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p,
                                          c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hk_moe_fp8blk_forward_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p,
                                           c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                           c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "hk_moe_fp8blk_forward": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                      c_void_p, c_size_t, c_void_p]),
}


def lib_path() -> Path:
    return _LIB_PATH


def load_library() -> ctypes.CDLL:
    """Load libhk355.so (built by hipkittens_amd/build.py). Raises RuntimeError if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not _LIB_PATH.exists():
        raise RuntimeError(
            f"{_LIB_PATH} is missing: build it with `python -m hipkittens_amd.build` "
            "(hipcc, gfx950). There is no CPU or PyTorch fallback for these kernels.")
    lib = ctypes.CDLL(str(_LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """Turn a negative hk_status into the RuntimeError the reference's bindings raise
    (std::runtime_error -> RuntimeError, include/pyutils/pyutils.cuh:21-34)."""
    if status != 0:
        msg = load_library().hk_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (hk_status {status})")
