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


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t) -> int:
    """torch's current stream on t's device, as a hipStream_t value."""
    if _raw_stream is not None:  # the same handle without building a Stream object (saves >1 us per call)
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


_FP8 = (torch.float8_e4m3fn, torch.uint8)


def gemm_tile_choice(fmt: str, M: int, N: int, K: int, consult_table: bool = True) -> int:
    """Tile (256, 128 or 64) the library picks for a GEMM of format "fp8", "bf16" or "mxfp4" on the current
    device; consult_table False: the rule alone, without the generated per-shape table (tile_sweep.py)."""
    code = {"fp8": 0, "bf16": 1, "mxfp4": 2}.get(fmt)
    if code is None:
        raise RuntimeError(f"unknown GEMM format {fmt!r}")
    tile = int(_lib.load_library().hk_gemm_tile_choice(code, int(M), int(N), int(K), 1 if consult_table else 0))
    if tile < 0:
        _lib.check(tile, "gemm_tile_choice")
    return tile


def fp8_gemm_workspace_bytes(M: int, N: int, K: int) -> int:
    """Bytes of workspace with which dispatch_fp8_gemm splits K for this shape (0: it would not)."""
    return int(_lib.load_library().hk_fp8_gemm_workspace_bytes(int(M), int(N), int(K)))


def dispatch_fp8_gemm(A, B, C, scale_a: float = 1.0, scale_b: float = 1.0, variant: int = -1,
                      workspace=None) -> None:
    """C[M,N] (bf16) = (scale_a*A[M,K]) @ (scale_b*B[N,K]).T, A and B e4m3, fp32 accumulation.

    `variant` -1 lets the library choose; 0..8 force a kernel (see include/hk355.h). `workspace`
    (uint8, fp8_gemm_workspace_bytes(M, N, K) bytes): lets the library split K for decode-like
    shapes (hk_fp8_gemm_ws)."""
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
    if workspace is not None:
        _check_tensor(workspace, "workspace", (torch.uint8,), 1)
        if variant >= 0:
            raise RuntimeError("workspace and a forced variant exclude each other")
        st = lib.hk_fp8_gemm_ws(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, float(scale_a),
                                float(scale_b), workspace.data_ptr(), workspace.numel(), _stream(A))
    elif variant < 0:
        st = lib.hk_fp8_gemm(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K,
                             float(scale_a), float(scale_b), _stream(A))
    else:
        st = lib.hk_fp8_gemm_variant(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K,
                                     float(scale_a), float(scale_b), int(variant), _stream(A))
    _lib.check(st, "dispatch_fp8_gemm")


def bf16_gemm_workspace_bytes(M: int, N: int, K: int) -> int:
    """Bytes of workspace with which dispatch_bf16_gemm splits K for this shape (0: it would not)."""
    return int(_lib.load_library().hk_bf16_gemm_workspace_bytes(int(M), int(N), int(K)))


def dispatch_bf16_gemm(A, B, C, variant: int = -1, workspace=None) -> None:
    """C[M,N] (bf16) = A[M,K] @ B[N,K].T for bf16 operands, fp32 accumulation
    (include/hk355.h: hk_bf16_gemm). `variant` -1 lets the library choose; 0..6 force a kernel.
    `workspace` (uint8, bf16_gemm_workspace_bytes(M, N, K) bytes): lets the library split K for
    decode-like shapes (hk_bf16_gemm_ws)."""
    _check_tensor(A, "A", _BF16, 2)
    _check_tensor(B, "B", _BF16, 2)
    _check_tensor(C, "C", _BF16, 2)
    M, K = A.shape
    N = B.shape[0]
    if B.shape[1] != K or tuple(C.shape) != (M, N):
        raise RuntimeError(f"shape mismatch: A {tuple(A.shape)}, B {tuple(B.shape)}, C {tuple(C.shape)}")
    lib = _lib.load_library()
    if workspace is not None:
        _check_tensor(workspace, "workspace", (torch.uint8,), 1)
        if variant >= 0:
            raise RuntimeError("workspace and a forced variant exclude each other")
        st = lib.hk_bf16_gemm_ws(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, workspace.data_ptr(),
                                 workspace.numel(), _stream(A))
    elif variant < 0:
        st = lib.hk_bf16_gemm(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, _stream(A))
    else:
        st = lib.hk_bf16_gemm_variant(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, int(variant), _stream(A))
    _lib.check(st, "dispatch_bf16_gemm")


def dispatch_micro(A, B, C) -> None:
    """The reference's GEMM entry point name: C = A @ B.T. bf16 operands run the BF16 GEMM (the
    reference's kernels/gemm/bf16fp32 binding), e4m3 operands the FP8 GEMM with unit scales (its
    kernels/gemm/fp8fp32 executables)."""
    if isinstance(A, torch.Tensor) and A.dtype == torch.bfloat16:
        dispatch_bf16_gemm(A, B, C)
    else:
        dispatch_fp8_gemm(A, B, C, 1.0, 1.0)


_U8 = (torch.uint8,)
_FP4 = tuple(d for d in (torch.uint8, getattr(torch, "float4_e2m1fn_x2", None)) if d is not None)
_E8M0 = tuple(d for d in (torch.uint8, getattr(torch, "float8_e8m0fnu", None)) if d is not None)


def mxfp4_gemm_workspace_bytes(M: int, N: int, K: int) -> int:
    """Bytes of workspace with which dispatch_mxfp4_gemm splits K for this shape (0: it would not)."""
    return int(_lib.load_library().hk_mxfp4_gemm_workspace_bytes(int(M), int(N), int(K)))


def dispatch_mxfp4_gemm(A, A_scales, B, B_scales, C, variant: int = -1, workspace=None) -> None:
    """C[M,N] (bf16) = dequant(A) @ dequant(B).T for MXFP4 operands: A [M,K/2] packed e2m1
    (low nibble = even k), A_scales [M,K/32] e8m0, B [N,K/2], B_scales [N,K/32]. The scale tensors
    may be wider than K/32 (padded rows, e.g. quant.pad_scales: any byte but 0xFF in the padding);
    rows that are a multiple of 8 bytes keep a K that is not a multiple of 256 on the tile kernels.
    `variant` -1 lets the library choose; 0..6 force a kernel (see include/hk355.h).
    `workspace` (uint8, mxfp4_gemm_workspace_bytes(M, N, K) bytes): lets the library split K for
    decode-like shapes (hk_mxfp4_gemm_ws)."""
    _check_tensor(A, "A", _FP4, 2)
    _check_tensor(B, "B", _FP4, 2)
    _check_tensor(A_scales, "A_scales", _E8M0, 2)
    _check_tensor(B_scales, "B_scales", _E8M0, 2)
    _check_tensor(C, "C", (torch.bfloat16,), 2)
    M, Kh = A.shape
    N, Kh2 = B.shape
    K = 2 * Kh
    if Kh2 != Kh or K % 32 != 0 or A_scales.shape[0] != M or A_scales.shape[1] < K // 32 or \
            B_scales.shape[0] != N or B_scales.shape[1] < K // 32 or tuple(C.shape) != (M, N):
        raise RuntimeError(
            f"shape mismatch: A {tuple(A.shape)}, A_scales {tuple(A_scales.shape)}, B {tuple(B.shape)}, "
            f"B_scales {tuple(B_scales.shape)}, C {tuple(C.shape)}")
    if len({t.device for t in (A, A_scales, B, B_scales, C)}) != 1:
        raise RuntimeError("all tensors must be on the same device")
    lib = _lib.load_library()
    args = (A.data_ptr(), A_scales.data_ptr(), B.data_ptr(), B_scales.data_ptr(), C.data_ptr(), M, N, K)
    pa, pb = A_scales.shape[1], B_scales.shape[1]
    if workspace is not None:
        if variant >= 0:
            raise RuntimeError("a workspace and a forced variant exclude each other")
        _check_tensor(workspace, "workspace", (torch.uint8,), 1)
        if workspace.device != A.device:
            raise RuntimeError("all tensors must be on the same device")
        st = lib.hk_mxfp4_gemm_ws(A.data_ptr(), A_scales.data_ptr(), pa, B.data_ptr(), B_scales.data_ptr(), pb,
                                  C.data_ptr(), M, N, K, workspace.data_ptr(), workspace.numel(), _stream(A))
    elif pa != K // 32 or pb != K // 32:
        if variant >= 0:
            raise RuntimeError("padded scale rows and a forced variant exclude each other")
        st = lib.hk_mxfp4_gemm_pitched(A.data_ptr(), A_scales.data_ptr(), pa, B.data_ptr(), B_scales.data_ptr(), pb,
                                       C.data_ptr(), M, N, K, _stream(A))
    elif variant < 0:
        st = lib.hk_mxfp4_gemm(*args, _stream(A))
    else:
        st = lib.hk_mxfp4_gemm_variant(*args, int(variant), _stream(A))
    _lib.check(st, "dispatch_mxfp4_gemm")


# ------------------------------------------------------------------------------ MoE routing
_F32 = (torch.float32,)
_I32 = (torch.int32,)


def dispatch_moe_topk_softmax(logits, ids, weights) -> None:
    """logits [T,E] fp32 -> ids [T,k] int32, weights [T,k] fp32 (k from the output shape)."""
    _check_tensor(logits, "logits", _F32, 2)
    _check_tensor(ids, "ids", _I32, 2)
    _check_tensor(weights, "weights", _F32, 2)
    T, E = logits.shape
    if ids.shape[0] != T or tuple(weights.shape) != tuple(ids.shape):
        raise RuntimeError("shape mismatch between logits, ids and weights")
    st = _lib.load_library().hk_moe_topk_softmax(logits.data_ptr(), T, E, ids.shape[1], ids.data_ptr(),
                                                 weights.data_ptr(), _stream(logits))
    _lib.check(st, "dispatch_moe_topk_softmax")


def dispatch_moe_topk_grouped_sigmoid(logits, bias, ids, weights, n_group: int, topk_group: int,
                                      routed_scale: float = 1.0) -> None:
    """Group-limited sigmoid routing; `bias` [E] fp32 or None."""
    _check_tensor(logits, "logits", _F32, 2)
    if bias is not None:
        _check_tensor(bias, "bias", _F32, 1)
    _check_tensor(ids, "ids", _I32, 2)
    _check_tensor(weights, "weights", _F32, 2)
    T, E = logits.shape
    if ids.shape[0] != T or tuple(weights.shape) != tuple(ids.shape) or (bias is not None and bias.shape[0] != E):
        raise RuntimeError("shape mismatch between logits, bias, ids and weights")
    st = _lib.load_library().hk_moe_topk_grouped_sigmoid(
        logits.data_ptr(), bias.data_ptr() if bias is not None else None, T, E, ids.shape[1],
        int(n_group), int(topk_group), float(routed_scale), ids.data_ptr(), weights.data_ptr(),
        _stream(logits))
    _lib.check(st, "dispatch_moe_topk_grouped_sigmoid")


def moe_sort_workspace_bytes(T: int, k: int, E: int) -> int:
    return int(_lib.load_library().hk_moe_sort_workspace_bytes(T, k, E))


def dispatch_moe_sort(ids, sorted_slots, expert_offsets, slot_to_pos, workspace) -> None:
    """ids [T,k] int32 -> sorted_slots [T*k], expert_offsets [E+1], slot_to_pos [T*k] or None;
    `workspace` is a uint8/int32 tensor of at least moe_sort_workspace_bytes(T, k, E) bytes."""
    _check_tensor(ids, "ids", _I32, 2)
    _check_tensor(sorted_slots, "sorted_slots", _I32, 1)
    _check_tensor(expert_offsets, "expert_offsets", _I32, 1)
    if slot_to_pos is not None:
        _check_tensor(slot_to_pos, "slot_to_pos", _I32, 1)
    _check_tensor(workspace, "workspace", (torch.uint8, torch.int32), 1)
    T, k = ids.shape
    E = expert_offsets.shape[0] - 1
    if sorted_slots.shape[0] != T * k or (slot_to_pos is not None and slot_to_pos.shape[0] != T * k) or E <= 0:
        raise RuntimeError("shape mismatch between ids, sorted_slots, expert_offsets and slot_to_pos")
    st = _lib.load_library().hk_moe_sort(
        ids.data_ptr(), T, k, E, sorted_slots.data_ptr(), expert_offsets.data_ptr(),
        slot_to_pos.data_ptr() if slot_to_pos is not None else None, workspace.data_ptr(),
        workspace.numel() * workspace.element_size(), _stream(ids))
    _lib.check(st, "dispatch_moe_sort")


# ---------------------------------------------------------------------------- MXFP4 fused MoE
_BF16 = (torch.bfloat16,)


def dispatch_mxfp4_quantize_rows(x, packed, scales) -> None:
    """x [R,C] bf16 -> packed [R,C/2] uint8, scales [R,pitch] uint8 (pitch >= C/32, multiple of 8)."""
    _check_tensor(x, "x", _BF16, 2)
    _check_tensor(packed, "packed", _FP4, 2)
    _check_tensor(scales, "scales", _E8M0, 2)
    R, C = x.shape
    if tuple(packed.shape) != (R, C // 2) or scales.shape[0] != R:
        raise RuntimeError("shape mismatch between x, packed and scales")
    st = _lib.load_library().hk_mxfp4_quantize_rows(x.data_ptr(), R, C, packed.data_ptr(), scales.data_ptr(),
                                                    scales.shape[1], _stream(x))
    _lib.check(st, "dispatch_mxfp4_quantize_rows")


def dispatch_mxfp8_quantize_rows(x, codes, scales) -> None:
    """x [R,C] bf16 -> codes [R,C] e4m3 (MX blocks of 32, shared exponent floor(log2 amax) - 8,
    saturating), scales [R,pitch] uint8 e8m0 (pitch >= C/32, multiple of 8)."""
    _check_tensor(x, "x", _BF16, 2)
    _check_tensor(codes, "codes", _FP8, 2)
    _check_tensor(scales, "scales", _E8M0, 2)
    R, C = x.shape
    if tuple(codes.shape) != (R, C) or scales.shape[0] != R:
        raise RuntimeError("shape mismatch between x, codes and scales")
    st = _lib.load_library().hk_mxfp8_quantize_rows(x.data_ptr(), R, C, codes.data_ptr(), scales.data_ptr(),
                                                    scales.shape[1], _stream(x))
    _lib.check(st, "dispatch_mxfp8_quantize_rows")


def dispatch_moe_unpermute(o, weights, slot_to_pos, y, add=None) -> None:
    """y [T,H] bf16 = (add [T,H] bf16 if given) + sum_j weights[t,j] * o[slot_to_pos[t*k+j]] with
    o [T*k,H] bf16."""
    _check_tensor(o, "o", _BF16, 2)
    _check_tensor(weights, "weights", _F32, 2)
    _check_tensor(slot_to_pos, "slot_to_pos", _I32, 1)
    _check_tensor(y, "y", _BF16, 2)
    T, k = weights.shape
    H = y.shape[1]
    if tuple(o.shape) != (T * k, H) or y.shape[0] != T or slot_to_pos.shape[0] != T * k:
        raise RuntimeError("shape mismatch between o, weights, slot_to_pos and y")
    if add is not None:
        _check_tensor(add, "add", _BF16, 2)
        if tuple(add.shape) != (T, H):
            raise RuntimeError("add must be [T, H]")
    st = _lib.load_library().hk_moe_unpermute_add(o.data_ptr(), weights.data_ptr(), slot_to_pos.data_ptr(), T, k,
                                                  H, add.data_ptr() if add is not None else None, y.data_ptr(),
                                                  _stream(o))
    _lib.check(st, "dispatch_moe_unpermute")


def moe_mxfp4_workspace_bytes(T: int, H: int, I: int, E: int, k: int, act_format: str = "mxfp4") -> int:
    """Workspace of the MXFP4-weight MoE; act_format "mxfp8": with MXFP8 activations (W4A8)."""
    lib = _lib.load_library()
    if act_format == "mxfp8":
        return int(lib.hk_moe_mxfp4_a8_workspace_bytes(T, H, I, E, k))
    if act_format != "mxfp4":
        raise RuntimeError("act_format must be 'mxfp4' or 'mxfp8'")
    return int(lib.hk_moe_mxfp4_workspace_bytes(T, H, I, E, k))


class MoeMxfp4ShuffledWeights:
    """Expert weights in the pre-shuffled tile layout (hk_moe_mxfp4_preshuffle): built once,
    offline, from the plain [E, rows, K/2] + [E, rows, K/32] tensors."""

    def __init__(self, w13, w13_scales, w2, w2_scales, E: int, H: int, I: int, interleaved: bool = False):
        self.w13, self.w13_scales, self.w2, self.w2_scales = w13, w13_scales, w2, w2_scales
        self.E, self.H, self.I = E, H, I
        self.interleaved = bool(interleaved)  # row order of the source w13 (and of a bias13 given later)

    @staticmethod
    def _shuffle(w, scales, N: int, K: int, mode: int):
        lib = _lib.load_library()
        E = w.shape[0]
        import ctypes
        wb, sb = ctypes.c_size_t(0), ctypes.c_size_t(0)
        _lib.check(lib.hk_moe_mxfp4_preshuffle_bytes(E, N, K, mode, ctypes.byref(wb), ctypes.byref(sb)),
                   "moe_mxfp4_preshuffle_bytes")
        out_w = torch.empty(wb.value, dtype=torch.uint8, device=w.device)
        out_s = torch.empty(sb.value, dtype=torch.uint8, device=w.device)
        st = lib.hk_moe_mxfp4_preshuffle(w.data_ptr(), scales.data_ptr(), scales.shape[2], E, N, K, mode,
                                         out_w.data_ptr(), out_s.data_ptr(), _stream(w))
        _lib.check(st, "moe_mxfp4_preshuffle")
        return out_w, out_s

    @classmethod
    def from_plain(cls, w13, w13_scales, w2, w2_scales, interleaved: bool = False):
        """`interleaved`: rows 2c / 2c+1 of w13 are gate / up of column c (GPT-OSS checkpoints)
        instead of rows c / I+c."""
        _check_tensor(w13, "w13", _FP4, 3)
        _check_tensor(w13_scales, "w13_scales", _E8M0, 3)
        _check_tensor(w2, "w2", _FP4, 3)
        _check_tensor(w2_scales, "w2_scales", _E8M0, 3)
        E, twoI, Hh = w13.shape
        H, I = 2 * Hh, twoI // 2
        if tuple(w2.shape) != (E, H, I // 2) or tuple(w13_scales.shape[:2]) != (E, twoI) or \
                tuple(w2_scales.shape[:2]) != (E, H) or w13_scales.shape[2] < H // 32 or w2_scales.shape[2] < I // 32:
            raise RuntimeError("shape mismatch between w13, w13_scales, w2 and w2_scales")
        a, sa = cls._shuffle(w13, w13_scales, I, H, 2 if interleaved else 0)
        b, sb = cls._shuffle(w2, w2_scales, H, I, 1)
        return cls(a, sa, b, sb, E, H, I, interleaved)


def _moe_weight_args(x, weights_or_w13, w13_scales, w2, w2_scales, y):
    """-> (T, H, I, E, layout, w13_ptr, s13_ptr, s13_pitch, w2_ptr, s2_ptr, s2_pitch)"""
    _check_tensor(x, "x", _BF16, 2)
    _check_tensor(y, "y", _BF16, 2)
    T, H = x.shape
    if isinstance(weights_or_w13, MoeMxfp4ShuffledWeights):
        W = weights_or_w13
        if W.H != H or tuple(y.shape) != (T, H):
            raise RuntimeError("shape mismatch between x, y and the shuffled weights")
        return (T, H, W.I, W.E, 1, W.w13.data_ptr(), W.w13_scales.data_ptr(), 0, W.w2.data_ptr(),
                W.w2_scales.data_ptr(), 0)
    T, H, I, E = _check_moe_weights(x, weights_or_w13, w13_scales, w2, w2_scales, y)
    return (T, H, I, E, 0, weights_or_w13.data_ptr(), w13_scales.data_ptr(), w13_scales.shape[2], w2.data_ptr(),
            w2_scales.data_ptr(), w2_scales.shape[2])


def _check_moe_weights(x, w13, w13_scales, w2, w2_scales, y):
    _check_tensor(x, "x", _BF16, 2)
    _check_tensor(w13, "w13", _FP4, 3)
    _check_tensor(w13_scales, "w13_scales", _E8M0, 3)
    _check_tensor(w2, "w2", _FP4, 3)
    _check_tensor(w2_scales, "w2_scales", _E8M0, 3)
    _check_tensor(y, "y", _BF16, 2)
    T, H = x.shape
    E, twoI, Hh = w13.shape
    I = twoI // 2
    if Hh * 2 != H or tuple(w2.shape) != (E, H, I // 2) or tuple(y.shape) != (T, H) or \
            tuple(w13_scales.shape[:2]) != (E, twoI) or tuple(w2_scales.shape[:2]) != (E, H):
        raise RuntimeError("shape mismatch between x, w13, w13_scales, w2, w2_scales and y")
    return T, H, I, E


_ACTIVATIONS = {"silu": 0, "swiglu_oai": 1}


def _moe_ext_args(w13, E, H, I, bias13, bias2, activation, interleaved):
    """-> (bias13_ptr, bias2_ptr, activation code, interleaved flag) of the extended entry points."""
    if activation not in _ACTIVATIONS:
        raise RuntimeError(f"activation must be one of {sorted(_ACTIVATIONS)}")
    if isinstance(w13, MoeMxfp4ShuffledWeights):
        if interleaved is not None and bool(interleaved) != w13.interleaved:
            raise RuntimeError("interleaved does not match the layout the weights were shuffled from")
        interleaved = w13.interleaved
    if bias13 is not None:
        _check_tensor(bias13, "bias13", _F32, 2)
        if tuple(bias13.shape) != (E, 2 * I):
            raise RuntimeError("bias13 must be [E, 2I]")
    if bias2 is not None:
        _check_tensor(bias2, "bias2", _F32, 2)
        if tuple(bias2.shape) != (E, H):
            raise RuntimeError("bias2 must be [E, H]")
    return (bias13.data_ptr() if bias13 is not None else None, bias2.data_ptr() if bias2 is not None else None,
            _ACTIVATIONS[activation], 1 if interleaved else 0)


def dispatch_moe_mxfp4_experts(x, w13, w13_scales, w2, w2_scales, weights, sorted_slots, expert_offsets,
                               slot_to_pos, y, workspace, bias13=None, bias2=None, activation: str = "silu",
                               alpha: float = 1.702, limit: float = 7.0, interleaved=None,
                               act_format: str = "mxfp4") -> None:
    """Expert MLP on routed + sorted tokens (see include/hk355.h: hk_moe_mxfp4_experts_ex). `w13` may be
    a MoeMxfp4ShuffledWeights, in which case w13_scales, w2 and w2_scales are ignored (pass None).
    Model-faithful options: bias13 [E, 2I] / bias2 [E, H] fp32, activation "swiglu_oai" (clamped
    SwiGLU with alpha and limit), interleaved gate / up rows of w13 and bias13. act_format "mxfp8":
    activations re-quantized to MXFP8 instead of MXFP4 (hk_moe_mxfp4_a8_experts; pre-shuffled weights
    only)."""
    T, H, I, E, layout, pw13, ps13, pitch13, pw2, ps2, pitch2 = _moe_weight_args(x, w13, w13_scales, w2, w2_scales, y)
    pb13, pb2, act, inter = _moe_ext_args(w13, E, H, I, bias13, bias2, activation, interleaved)
    _check_tensor(weights, "weights", _F32, 2)
    _check_tensor(sorted_slots, "sorted_slots", _I32, 1)
    _check_tensor(expert_offsets, "expert_offsets", _I32, 1)
    _check_tensor(slot_to_pos, "slot_to_pos", _I32, 1)
    _check_tensor(workspace, "workspace", (torch.uint8,), 1)
    k = weights.shape[1]
    if weights.shape[0] != T or sorted_slots.shape[0] != T * k or expert_offsets.shape[0] != E + 1 or \
            slot_to_pos.shape[0] != T * k:
        raise RuntimeError("shape mismatch between routing tensors")
    if _a8(act_format, layout):
        st = _lib.load_library().hk_moe_mxfp4_a8_experts(
            x.data_ptr(), pw13, ps13, pw2, ps2, weights.data_ptr(), sorted_slots.data_ptr(),
            expert_offsets.data_ptr(), slot_to_pos.data_ptr(), y.data_ptr(), T, H, I, E, k,
            pb13, pb2, act, float(alpha), float(limit), inter, workspace.data_ptr(), workspace.numel(), _stream(x))
    else:
        st = _lib.load_library().hk_moe_mxfp4_experts_ex(
            x.data_ptr(), pw13, ps13, pitch13, pw2, ps2, pitch2, weights.data_ptr(), sorted_slots.data_ptr(),
            expert_offsets.data_ptr(), slot_to_pos.data_ptr(), y.data_ptr(), T, H, I, E, k, layout,
            pb13, pb2, act, float(alpha), float(limit), inter, workspace.data_ptr(), workspace.numel(), _stream(x))
    _lib.check(st, "dispatch_moe_mxfp4_experts")


def _a8(act_format: str, layout: int) -> bool:
    if act_format == "mxfp4":
        return False
    if act_format != "mxfp8":
        raise RuntimeError("act_format must be 'mxfp4' or 'mxfp8'")
    if layout != 1:
        raise RuntimeError("MXFP8 activations need pre-shuffled weights (MoeMxfp4ShuffledWeights)")
    return True


def dispatch_moe_mxfp4(x, router_logits, w13, w13_scales, w2, w2_scales, y, topk: int, workspace,
                       bias13=None, bias2=None, activation: str = "silu", alpha: float = 1.702,
                       limit: float = 7.0, interleaved=None, act_format: str = "mxfp4") -> None:
    """Whole MXFP4 MoE layer: top-k softmax routing, sort, expert MLP, un-permute into y. `w13` may be
    a MoeMxfp4ShuffledWeights (then pass None for w13_scales, w2, w2_scales). Options as in
    dispatch_moe_mxfp4_experts."""
    T, H, I, E, layout, pw13, ps13, pitch13, pw2, ps2, pitch2 = _moe_weight_args(x, w13, w13_scales, w2, w2_scales, y)
    pb13, pb2, act, inter = _moe_ext_args(w13, E, H, I, bias13, bias2, activation, interleaved)
    _check_tensor(router_logits, "router_logits", _F32, 2)
    _check_tensor(workspace, "workspace", (torch.uint8,), 1)
    if tuple(router_logits.shape) != (T, E):
        raise RuntimeError("router_logits must be [T, E]")
    if _a8(act_format, layout):
        st = _lib.load_library().hk_moe_mxfp4_a8_forward(
            x.data_ptr(), router_logits.data_ptr(), pw13, ps13, pw2, ps2, y.data_ptr(), T, H, I, E,
            int(topk), pb13, pb2, act, float(alpha), float(limit), inter, workspace.data_ptr(),
            workspace.numel(), _stream(x))
    else:
        st = _lib.load_library().hk_moe_mxfp4_forward_ex(
            x.data_ptr(), router_logits.data_ptr(), pw13, ps13, pitch13, pw2, ps2, pitch2, y.data_ptr(), T, H, I, E,
            int(topk), layout, pb13, pb2, act, float(alpha), float(limit), inter, workspace.data_ptr(),
            workspace.numel(), _stream(x))
    _lib.check(st, "dispatch_moe_mxfp4")


# --------------------------------------------------------------------- FP8 block-scaled MoE
def dispatch_fp8_quantize_rows_1x128(x, q, scales) -> None:
    """x [R,C] bf16 -> q [R,C] e4m3, scales [R,C/128] fp32 (1 x 128 blocks, scale = amax/448)."""
    _check_tensor(x, "x", _BF16, 2)
    _check_tensor(q, "q", _FP8, 2)
    _check_tensor(scales, "scales", _F32, 2)
    R, C = x.shape
    if tuple(q.shape) != (R, C) or tuple(scales.shape) != (R, C // 128):
        raise RuntimeError("shape mismatch between x, q and scales")
    st = _lib.load_library().hk_fp8_quantize_rows_1x128(x.data_ptr(), R, C, q.data_ptr(), scales.data_ptr(),
                                                        _stream(x))
    _lib.check(st, "dispatch_fp8_quantize_rows_1x128")


def moe_fp8blk_workspace_bytes(T: int, H: int, I: int, E: int, k: int) -> int:
    return int(_lib.load_library().hk_moe_fp8blk_workspace_bytes(T, H, I, E, k))


class MoeFp8BlkShuffledWeights:
    """FP8 block-scaled expert weights in the pre-shuffled tile layout (hk_moe_fp8blk_preshuffle): built
    once, offline, from the plain [E, 2I, H] / [E, H, I] e4m3 tensors; the fp32 block scales are kept
    as they are. Pass it as `w13` to the dispatch_moe_fp8blk* functions (w13_scales, w2, w2_scales None)."""

    def __init__(self, w13, w13_scales, w2, w2_scales, E: int, H: int, I: int):
        self.w13, self.w13_scales, self.w2, self.w2_scales = w13, w13_scales, w2, w2_scales
        self.E, self.H, self.I = E, H, I

    @staticmethod
    def _shuffle(w, N: int, K: int, mode: int):
        import ctypes
        lib = _lib.load_library()
        E = w.shape[0]
        nbytes = ctypes.c_size_t(0)
        _lib.check(lib.hk_moe_fp8blk_preshuffle_bytes(E, N, K, mode, ctypes.byref(nbytes)), "moe_fp8blk_preshuffle_bytes")
        out = torch.empty(nbytes.value, dtype=torch.uint8, device=w.device)
        _lib.check(lib.hk_moe_fp8blk_preshuffle(w.data_ptr(), E, N, K, mode, out.data_ptr(), _stream(w)),
                   "moe_fp8blk_preshuffle")
        return out

    @classmethod
    def from_plain(cls, w13, w13_scales, w2, w2_scales):
        _check_tensor(w13, "w13", _FP8, 3)
        _check_tensor(w13_scales, "w13_scales", _F32, 3)
        _check_tensor(w2, "w2", _FP8, 3)
        _check_tensor(w2_scales, "w2_scales", _F32, 3)
        E, twoI, H = w13.shape
        I = twoI // 2
        if H % 128 or I % 128 or tuple(w2.shape) != (E, H, I) or \
                tuple(w13_scales.shape) != (E, twoI // 128, H // 128) or tuple(w2_scales.shape) != (E, H // 128, I // 128):
            raise RuntimeError("shape mismatch between w13, w13_scales, w2 and w2_scales")
        return cls(cls._shuffle(w13, I, H, 0), w13_scales, cls._shuffle(w2, H, I, 1), w2_scales, E, H, I)


def _check_fp8blk(x, x_scales, w13, w13_scales, w2, w2_scales, y, x_dtypes=None):
    """-> (T, H, I, E, weight_layout, w13, w13_scales, w2, w2_scales)"""
    _check_tensor(x, "x", x_dtypes or _FP8, 2)
    if x_scales is not None:
        _check_tensor(x_scales, "x_scales", _F32, 2)
    _check_tensor(y, "y", _BF16, 2)
    T, H = x.shape
    layout = 0
    if isinstance(w13, MoeFp8BlkShuffledWeights):
        W = w13
        w13, w13_scales, w2, w2_scales, layout = W.w13, W.w13_scales, W.w2, W.w2_scales, 1
        E, I = W.E, W.I
        if W.H != H:
            raise RuntimeError("shape mismatch between x and the shuffled weights")
    else:
        _check_tensor(w13, "w13", _FP8, 3)
        _check_tensor(w2, "w2", _FP8, 3)
        E, twoI, H2 = w13.shape
        I = twoI // 2
        if H2 != H or tuple(w2.shape) != (E, H, I):
            raise RuntimeError("shape mismatch between x, w13 and w2")
    _check_tensor(w13_scales, "w13_scales", _F32, 3)
    _check_tensor(w2_scales, "w2_scales", _F32, 3)
    if H % 128 or I % 128 or tuple(y.shape) != (T, H) or \
            (x_scales is not None and tuple(x_scales.shape) != (T, H // 128)) or \
            tuple(w13_scales.shape) != (E, 2 * I // 128, H // 128) or tuple(w2_scales.shape) != (E, H // 128, I // 128):
        raise RuntimeError("shape mismatch between x, x_scales, w13, w13_scales, w2, w2_scales and y")
    if len({t.device for t in (x, w13, w13_scales, w2, w2_scales, y)}) != 1:
        raise RuntimeError("all tensors must be on the same device")
    return T, H, I, E, layout, w13, w13_scales, w2, w2_scales


def _check_y_add(y_add, y):
    if y_add is None:
        return None
    _check_tensor(y_add, "y_add", _BF16, 2)
    if tuple(y_add.shape) != tuple(y.shape):
        raise RuntimeError("y_add must have the shape of y")
    return y_add.data_ptr()


def dispatch_moe_fp8blk_experts(x, x_scales, w13, w13_scales, w2, w2_scales, weights, sorted_slots,
                                expert_offsets, slot_to_pos, y, workspace, y_add=None) -> None:
    """FP8 block-scaled expert MLP on routed + sorted tokens (include/hk355.h: hk_moe_fp8blk_experts_ex).
    y_add [T,H] bf16: residual added before the output rounding (a shared expert's output)."""
    T, H, I, E, layout, w13, w13_scales, w2, w2_scales = _check_fp8blk(x, x_scales, w13, w13_scales, w2, w2_scales, y)
    p_add = _check_y_add(y_add, y)
    _check_tensor(weights, "weights", _F32, 2)
    _check_tensor(sorted_slots, "sorted_slots", _I32, 1)
    _check_tensor(expert_offsets, "expert_offsets", _I32, 1)
    _check_tensor(slot_to_pos, "slot_to_pos", _I32, 1)
    _check_tensor(workspace, "workspace", (torch.uint8,), 1)
    k = weights.shape[1]
    if weights.shape[0] != T or sorted_slots.shape[0] != T * k or expert_offsets.shape[0] != E + 1 or \
            slot_to_pos.shape[0] != T * k:
        raise RuntimeError("shape mismatch between routing tensors")
    st = _lib.load_library().hk_moe_fp8blk_experts_ex2(
        x.data_ptr(), x_scales.data_ptr(), w13.data_ptr(), w13_scales.data_ptr(), w2.data_ptr(),
        w2_scales.data_ptr(), weights.data_ptr(), sorted_slots.data_ptr(), expert_offsets.data_ptr(),
        slot_to_pos.data_ptr(), y.data_ptr(), T, H, I, E, k, layout, p_add, workspace.data_ptr(), workspace.numel(),
        _stream(x))
    _lib.check(st, "dispatch_moe_fp8blk_experts")


def dispatch_moe_fp8blk_shared_expert(x, x_scales, w13, w13_scales, w2, w2_scales, y, workspace) -> None:
    """The dense MLP every token passes through (DeepSeek-V3 shared expert): w13 [1, 2I, H],
    w2 [1, H, I] in the routed experts' format, run as a one-expert layer with identity routing.
    workspace: moe_fp8blk_workspace_bytes(T, H, I, 1, 1) bytes. Its output is what the routed layer
    takes as y_add."""
    T = x.shape[0]
    ones = torch.ones((T, 1), dtype=torch.float32, device=x.device)
    ident = torch.arange(T, dtype=torch.int32, device=x.device)
    offsets = torch.tensor([0, T], dtype=torch.int32, device=x.device)
    dispatch_moe_fp8blk_experts(x, x_scales, w13, w13_scales, w2, w2_scales, ones, ident, offsets, ident, y,
                                workspace)


def dispatch_moe_fp8blk(x, x_scales, router_logits, router_bias, w13, w13_scales, w2, w2_scales, y, topk: int,
                        n_group: int, topk_group: int, routed_scale: float, workspace, y_add=None) -> None:
    """Whole FP8 block-scaled MoE layer with group-limited sigmoid routing (router_bias: the
    selection-only score correction). y_add [T,H] bf16: residual added before the output rounding
    (dispatch_moe_fp8blk_shared_expert's output). `w13` may be a MoeFp8BlkShuffledWeights (then pass None
    for w13_scales, w2, w2_scales). `x` may be bf16 with x_scales None: the layer then quantizes every
    token to e4m3 with 1 x 128 scales itself (hk_moe_fp8blk_forward_bf16)."""
    bf16_in = isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16
    if bf16_in != (x_scales is None):
        raise RuntimeError("x_scales must be given for e4m3 activations and None for bf16 activations")
    T, H, I, E, layout, w13, w13_scales, w2, w2_scales = _check_fp8blk(
        x, x_scales, w13, w13_scales, w2, w2_scales, y, x_dtypes=_BF16 if bf16_in else None)
    p_add = _check_y_add(y_add, y)
    _check_tensor(router_logits, "router_logits", _F32, 2)
    if router_bias is not None:
        _check_tensor(router_bias, "router_bias", _F32, 1)
        if router_bias.shape[0] != E:
            raise RuntimeError("router_bias must be [E]")
    _check_tensor(workspace, "workspace", (torch.uint8,), 1)
    if tuple(router_logits.shape) != (T, E):
        raise RuntimeError("router_logits must be [T, E]")
    lib = _lib.load_library()
    p_bias = router_bias.data_ptr() if router_bias is not None else None
    if bf16_in:
        st = lib.hk_moe_fp8blk_forward_bf16(
            x.data_ptr(), router_logits.data_ptr(), p_bias, int(n_group), int(topk_group), float(routed_scale),
            w13.data_ptr(), w13_scales.data_ptr(), w2.data_ptr(), w2_scales.data_ptr(), y.data_ptr(), T, H, I, E,
            int(topk), layout, p_add, workspace.data_ptr(), workspace.numel(), _stream(x))
    else:
        st = lib.hk_moe_fp8blk_forward_ex2(
            x.data_ptr(), x_scales.data_ptr(), router_logits.data_ptr(), p_bias, int(n_group), int(topk_group),
            float(routed_scale), w13.data_ptr(), w13_scales.data_ptr(), w2.data_ptr(), w2_scales.data_ptr(),
            y.data_ptr(), T, H, I, E, int(topk), layout, p_add, workspace.data_ptr(), workspace.numel(), _stream(x))
    _lib.check(st, "dispatch_moe_fp8blk")
