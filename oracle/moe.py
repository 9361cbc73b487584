"""CPU oracle, part 3: MoE routing, sort/permute and the fused expert MLP.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The reference has no MoE code at all, so every function here is "parity unpinned" with
respect to the reference; the specification is the one fixed for this path and each function
is pinned by brute force / library routines in tests/test_oracle_moe.py:

* top-k softmax routing: ids = first k entries of a stable descending sort of the fp32 logits
  (ties -> lower expert id); weights = softmax over the k selected logits.
* group-limited sigmoid routing (DeepSeek-V3 style): s = sigmoid(logit); selection score
  c = s + bias (bias optional, used for selection only); group score = sum of the two largest c
  in each of n_group contiguous groups; keep the topk_group best groups (ties -> lower group);
  ids = top-k of c among kept groups (stable, ties -> lower id); weights =
  s[ids] / sum(s[ids]) * routed_scale.  To make the integer outputs bit-exact across CPU and
  GPU, sigmoid is *defined* by `sigmoid_f32` below: a fixed sequence of correctly rounded fp32
  operations (no fused multiply-add), which both sides evaluate identically.
* sort: sorted_slots = slot indices t*k+j stably sorted by expert id, expert_offsets =
  exclusive prefix sum of the per-expert counts (E+1 entries), slot_to_pos = inverse map.
* expert MLP: per expert e over its rows: h = silu(x W1g^T) * (x W1u^T) with W13 rows =
  [gate(0..I-1); up(I..2I-1)], h re-quantized exactly like the kernel (MXFP4 per 32 along I,
  or e4m3 with 1x128 scales), o = h W2^T rounded to bf16, y[t] = bf16(sum_j w[t,j] o[pos(t,j)]).
"""
from __future__ import annotations

import numpy as np

from . import formats as F

f32 = np.float32

# exp(x) for x <= 0 in fp32: x = n*ln2 + r, exp(r) by a degree-6 polynomial, every step one
# correctly rounded fp32 operation.
_LOG2E = f32(1.4426950408889634)
_LN2_HI = f32(0.693145751953125)         # 12 significant bits -> n*LN2_HI exact for |n| < 2^11
_LN2_LO = f32(1.4286068203094172e-06)
_EXP_C = [f32(1.0 / 720), f32(1.0 / 120), f32(1.0 / 24), f32(1.0 / 6), f32(0.5), f32(1.0), f32(1.0)]


def exp_neg_f32(x: np.ndarray) -> np.ndarray:
    """exp(x) for x in [-88, 0] as a fixed fp32 operation sequence (inputs are clamped)."""
    x = np.maximum(np.asarray(x, dtype=f32), f32(-87.0))
    n = np.rint((x * _LOG2E).astype(f32)).astype(f32)
    r = (x - (n * _LN2_HI).astype(f32)).astype(f32)
    r = (r - (n * _LN2_LO).astype(f32)).astype(f32)
    p = np.full_like(r, _EXP_C[0])
    for c in _EXP_C[1:]:
        p = ((p * r).astype(f32) + c).astype(f32)
    return np.ldexp(p, n.astype(np.int32)).astype(f32)


def sigmoid_f32(x: np.ndarray) -> np.ndarray:
    """1/(1+exp(-|x|)) mirrored for negative x, all in fp32 with the exp above."""
    x = np.asarray(x, dtype=f32)
    e = exp_neg_f32(-np.abs(x))                       # in (0, 1]
    pos = (f32(1.0) / (f32(1.0) + e).astype(f32)).astype(f32)
    neg = (e / (f32(1.0) + e).astype(f32)).astype(f32)
    return np.where(x >= 0, pos, neg).astype(f32)


def _topk_stable(scores: np.ndarray, k: int) -> np.ndarray:
    """indices of the k largest per row, ties to the lower index (stable descending sort)."""
    order = np.argsort(-scores.astype(np.float64), axis=-1, kind="stable")
    return order[..., :k].astype(np.int32)


def topk_softmax(logits: np.ndarray, k: int):
    logits = np.asarray(logits, dtype=f32)
    ids = _topk_stable(logits, k)
    sel = np.take_along_axis(logits, ids, axis=-1).astype(np.float64)
    ex = np.exp(sel - sel.max(axis=-1, keepdims=True))
    w = (ex / ex.sum(axis=-1, keepdims=True)).astype(f32)
    return ids, w


def topk_grouped_sigmoid(logits, bias, k: int, n_group: int, topk_group: int, routed_scale: float = 1.0):
    logits = np.asarray(logits, dtype=f32)
    T, E = logits.shape
    gs = E // n_group
    s = sigmoid_f32(logits)
    c = s if bias is None else (s + np.asarray(bias, dtype=f32)[None, :]).astype(f32)
    cg = c.reshape(T, n_group, gs)
    top2 = -np.sort(-cg, axis=-1)[..., :2]
    gscore = (top2[..., 0] + top2[..., 1]).astype(f32) if gs >= 2 else top2[..., 0].astype(f32)
    keep = _topk_stable(gscore, topk_group)
    mask = np.zeros((T, n_group), dtype=bool)
    np.put_along_axis(mask, keep, True, axis=-1)
    masked = np.where(np.repeat(mask, gs, axis=1), c, f32(-np.inf))
    ids = _topk_stable(masked, k)
    sel = np.take_along_axis(s, ids, axis=-1)
    # the sum is taken in selection order, in fp32, like the kernel
    tot = np.zeros(T, dtype=f32)
    for j in range(k):
        tot = (tot + sel[:, j]).astype(f32)
    w = ((sel / tot[:, None]).astype(f32) * f32(routed_scale)).astype(f32)
    return ids, w


def moe_sort(ids: np.ndarray, E: int):
    """(sorted_slots [T*k], expert_offsets [E+1], slot_to_pos [T*k]) for ids [T,k]."""
    flat = np.asarray(ids, dtype=np.int32).reshape(-1)
    order = np.argsort(flat, kind="stable").astype(np.int32)
    counts = np.bincount(flat, minlength=E).astype(np.int64)
    offs = np.zeros(E + 1, dtype=np.int32)
    offs[1:] = np.cumsum(counts)
    inv = np.empty_like(order)
    inv[order] = np.arange(order.size, dtype=np.int32)
    return order, offs, inv


def silu(x):
    x = np.asarray(x, dtype=np.float32)
    return (x / (1.0 + np.exp(-x.astype(np.float64)))).astype(np.float32)


def quantize_act_mxfp4(x: np.ndarray):
    """Activation quantizer of the MXFP4 MoE path: MX blocks of 32 along the last axis."""
    return F.quantize_mxfp4(x)


def quantize_act(x: np.ndarray, act_format: str):
    """Activation quantizer of the MXFP4-weight MoE: MX blocks of 32 along the last axis with
    e2m1 ("mxfp4") or e4m3 ("mxfp8") elements. Returns (data, scales, dequantized fp32)."""
    if act_format == "mxfp4":
        q, s = F.quantize_mxfp4(x)
        return q, s, F.dequantize_mxfp4(q, s)
    if act_format == "mxfp8":
        q, s = F.quantize_mxfp8(x)
        return q, s, F.dequantize_mxfp8(q, s)
    raise ValueError(act_format)


def swiglu_clamped(gate, up, alpha: float, limit: float):
    """The gated activation of the GPT-OSS experts (published model code: gate clamped from above,
    up clamped to [-limit, limit], glu = gate * sigmoid(alpha * gate), result (up + 1) * glu).
    No counterpart in the reference repository; evaluated in float64, rounded once to fp32."""
    g = np.minimum(np.asarray(gate, dtype=np.float32), np.float32(limit))
    u = np.clip(np.asarray(up, dtype=np.float32), np.float32(-limit), np.float32(limit))
    glu = g.astype(np.float64) / (1.0 + np.exp(-float(alpha) * g.astype(np.float64)))
    return ((u.astype(np.float64) + 1.0) * glu).astype(np.float32)


def moe_mxfp4_forward(x_bf16_as_f32, ids, w, w13_packed, w13_scales, w2_packed, w2_scales,
                      bias13=None, bias2=None, activation: str = "silu", alpha: float = 1.702,
                      limit: float = 7.0, interleaved: bool = False, act_format: str = "mxfp4"):
    """Reference forward of the MXFP4 MoE. x [T,H] (bf16 values as fp32); ids/w [T,k];
    w13_packed [E, 2I, H/2], w13_scales [E, 2I, H/32]; w2_packed [E, H, I/2], w2_scales
    [E, H, I/32]. Returns (y as bf16 bits [T,H], dict of intermediates).

    Model-faithful options (GPT-OSS): bias13 [E, 2I] / bias2 [E, H] fp32 added to the GEMM
    results before the activation / before the weighted sum; activation "swiglu_oai" =
    swiglu_clamped; interleaved: rows 2i / 2i+1 of w13 (and of bias13) are gate / up of column i
    instead of rows i / I+i. act_format "mxfp8": x and h are quantized to MXFP8 (e4m3 elements,
    [S, I] codes in "hq") instead of MXFP4."""
    T, H = x_bf16_as_f32.shape
    E, twoI, _ = w13_packed.shape
    I = twoI // 2
    k = ids.shape[1]
    order, offs, inv = moe_sort(ids, E)
    xq, xs, xd = quantize_act(x_bf16_as_f32, act_format)
    S = T * k
    hq = np.zeros((S, I // 2 if act_format == "mxfp4" else I), dtype=np.uint8)
    hs = np.zeros((S, I // 32), dtype=np.uint8)
    o = np.zeros((S, H), dtype=np.float32)
    for e in range(E):
        lo, hi = offs[e], offs[e + 1]
        if hi == lo:
            continue
        tok = order[lo:hi] // k
        w13 = F.dequantize_mxfp4(w13_packed[e], w13_scales[e])
        gu = xd[tok] @ w13.T
        if bias13 is not None:
            gu = gu + np.asarray(bias13[e], dtype=np.float32)[None, :]
        gate, up = (gu[:, 0::2], gu[:, 1::2]) if interleaved else (gu[:, :I], gu[:, I:])
        if activation == "silu":
            h = (silu(gate) * up).astype(np.float32)
        elif activation == "swiglu_oai":
            h = swiglu_clamped(gate, up, alpha, limit)
        else:
            raise ValueError(activation)
        q, s, hd = quantize_act(h, act_format)
        hq[lo:hi], hs[lo:hi] = q, s
        w2 = F.dequantize_mxfp4(w2_packed[e], w2_scales[e])
        o[lo:hi] = hd @ w2.T
        if bias2 is not None:
            o[lo:hi] += np.asarray(bias2[e], dtype=np.float32)[None, :]
    o_bf = F.bf16_to_f32(F.bf16_round(o))
    y = np.zeros((T, H), dtype=np.float32)
    for j in range(k):
        y += w[:, j:j + 1].astype(np.float32) * o_bf[inv[np.arange(T) * k + j]]
    return F.bf16_round(y), {"order": order, "offs": offs, "inv": inv, "xq": xq, "xs": xs,
                             "hq": hq, "hs": hs, "o": o}


def moe_fp8blk_forward(x_codes, x_scales, ids, w, w13_codes, w13_scales, w2_codes, w2_scales, y_add=None):
    """Reference forward of the FP8 block-scaled MoE. x_codes [T,H] e4m3 codes with 1x128 scales
    [T,H/128]; w13_codes [E,2I,H] with 128x128 scales [E,2I/128,H/128]; w2_codes [E,H,I] with
    [E,H/128,I/128]. h is re-quantized with 1x128 blocks exactly like the kernel. Returns y as
    bf16 bits [T,H]. y_add [T,H] (bf16 values as fp32): residual the weighted sum starts from, e.g.
    moe_fp8blk_shared_expert's output."""
    T, H = x_codes.shape
    E, twoI, _ = w13_codes.shape
    I = twoI // 2
    k = ids.shape[1]
    order, offs, inv = moe_sort(ids, E)
    xd = F.dequantize_e4m3_blocks(x_codes, x_scales, 1, 128)
    S = T * k
    o = np.zeros((S, H), dtype=np.float32)
    for e in range(E):
        lo, hi = offs[e], offs[e + 1]
        if hi == lo:
            continue
        tok = order[lo:hi] // k
        w13 = F.dequantize_e4m3_blocks(w13_codes[e], w13_scales[e], 128, 128)
        gu = xd[tok] @ w13.T
        h = (silu(gu[:, :I]) * gu[:, I:]).astype(np.float32)
        q, s = F.quantize_e4m3_blocks(h, 1, 128)
        w2 = F.dequantize_e4m3_blocks(w2_codes[e], w2_scales[e], 128, 128)
        o[lo:hi] = F.dequantize_e4m3_blocks(q, s, 1, 128) @ w2.T
    o_bf = F.bf16_to_f32(F.bf16_round(o))
    y = np.zeros((T, H), dtype=np.float32) if y_add is None else np.array(y_add, dtype=np.float32)
    for j in range(k):
        y += w[:, j:j + 1].astype(np.float32) * o_bf[inv[np.arange(T) * k + j]]
    return F.bf16_round(y)


def moe_fp8blk_shared_expert(x_codes, x_scales, w13_codes, w13_scales, w2_codes, w2_scales):
    """The dense MLP every token passes through (DeepSeek-V3's shared expert): weights shaped
    [1, 2I, H] / [1, H, I] like one routed expert, every token routed to it with weight 1.
    Returns bf16 bits [T,H]."""
    T = x_codes.shape[0]
    ids = np.zeros((T, 1), dtype=np.int32)
    return moe_fp8blk_forward(x_codes, x_scales, ids, np.ones((T, 1), np.float32), w13_codes, w13_scales,
                              w2_codes, w2_scales)
