"""Pin the MoE oracle (CPU only): brute force on small inputs, library routines, invariants."""
import math

import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as G
from oracle import moe as O


def test_sigmoid_f32_close_to_libm_and_monotone():
    x = np.linspace(-30, 30, 20001).astype(np.float32)
    s = O.sigmoid_f32(x)
    ref = 1.0 / (1.0 + np.exp(-x.astype(np.float64)))
    assert np.max(np.abs(s - ref) / ref) < 5e-7
    assert np.all(np.diff(s) >= 0)
    assert O.sigmoid_f32(np.array([0.0], np.float32))[0] == 0.5


def test_exp_neg_f32_against_libm_and_its_fixed_points():
    x = np.linspace(-87, 0, 30001).astype(np.float32)
    e = O.exp_neg_f32(x)
    ref = np.exp(x.astype(np.float64))
    assert e.dtype == np.float32
    assert np.max(np.abs(e - ref) / ref) < 3e-7          # a few fp32 ulps over the whole range
    assert np.all(np.diff(e) >= 0)
    assert O.exp_neg_f32(np.array([0.0], np.float32))[0] == 1.0
    # powers of two come out exactly when x is the fp32 nearest to n ln 2 only up to the polynomial's error
    n = np.arange(-60, 0)
    xe = (n * np.log(2.0)).astype(np.float32)
    assert np.max(np.abs(O.exp_neg_f32(xe) - np.exp(xe.astype(np.float64))) / np.exp(xe.astype(np.float64))) < 3e-7
    # below the clamp the value of the clamp is returned (no underflow to a denormal, no zero)
    lo = O.exp_neg_f32(np.array([-87.0, -100.0, -1e30], np.float32))
    assert lo[0] == lo[1] == lo[2] and 0 < lo[0] < 2e-38 * 10


def test_quantize_act_is_the_format_quantizer_plus_its_dequantization():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((7, 96)) * 3).astype(np.float32)
    q4, s4, d4 = O.quantize_act(x, "mxfp4")
    rq, rs = F.quantize_mxfp4(x)
    assert np.array_equal(q4, rq) and np.array_equal(s4, rs) and np.array_equal(d4, F.dequantize_mxfp4(rq, rs))
    aq, as_ = O.quantize_act_mxfp4(x)
    assert np.array_equal(aq, rq) and np.array_equal(as_, rs)
    q8, s8, d8 = O.quantize_act(x, "mxfp8")
    rq, rs = F.quantize_mxfp8(x)
    assert np.array_equal(q8, rq) and np.array_equal(s8, rs) and np.array_equal(d8, F.dequantize_mxfp8(rq, rs))
    # an e4m3 element is within 2^-4 of its input unless it is the block's largest: the block scale maps
    # that one into [256, 512) and 448 is the largest code, so it may lose up to 1 - 448/512
    assert np.max(np.abs(d8 - x) / np.maximum(np.abs(x), 1e-3)) <= 0.125
    assert np.mean(np.abs(d8 - x) / np.maximum(np.abs(x), 1e-3) <= 0.0625) > 0.9
    # e2m1: the largest maps into [4, 8) with 6 the largest code (up to a quarter lost)
    assert np.max(np.abs(d4 - x) / np.max(np.abs(x))) <= 0.25
    try:
        O.quantize_act(x, "int8")
        raise AssertionError("unknown format accepted")
    except ValueError:
        pass


def test_topk_softmax_brute_force():
    rng = np.random.default_rng(0)
    logits = rng.standard_normal((37, 16)).astype(np.float32)
    logits[3, 5] = logits[3, 2]          # exact tie -> lower id first
    logits[4, :] = 0.25                   # all equal -> ids 0..k-1
    ids, w = O.topk_softmax(logits, 4)
    for t in range(logits.shape[0]):
        order = sorted(range(16), key=lambda e: (-float(logits[t, e]), e))[:4]
        assert list(ids[t]) == order
        ex = [math.exp(float(logits[t, e]) - float(logits[t, order[0]])) for e in order]
        assert np.allclose(w[t], np.array(ex) / sum(ex), rtol=1e-6)
    assert list(ids[4]) == [0, 1, 2, 3]
    assert list(ids[3]).index(2) < list(ids[3]).index(5) if 5 in ids[3] and 2 in ids[3] else True
    # library cross-check: torch.topk values agree
    tv, _ = torch.topk(torch.from_numpy(logits), 4, dim=-1)
    assert np.array_equal(np.take_along_axis(logits, ids, axis=-1), tv.numpy())


def test_grouped_sigmoid_brute_force():
    rng = np.random.default_rng(1)
    T, E, G, KG, K = 29, 32, 8, 3, 6
    logits = rng.standard_normal((T, E)).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.1).astype(np.float32)
    for b in (None, bias):
        ids, w = O.topk_grouped_sigmoid(logits, b, K, G, KG, routed_scale=2.5)
        s = O.sigmoid_f32(logits)
        c = s if b is None else (s + b[None, :]).astype(np.float32)
        gs = E // G
        for t in range(T):
            gscore = []
            for g in range(G):
                v = sorted((float(x) for x in c[t, g * gs:(g + 1) * gs]), reverse=True)
                gscore.append(float(np.float32(np.float32(v[0]) + np.float32(v[1]))))
            keep = sorted(range(G), key=lambda g: (-gscore[g], g))[:KG]
            cand = [e for e in range(E) if e // gs in keep]
            want = sorted(cand, key=lambda e: (-float(c[t, e]), e))[:K]
            assert list(ids[t]) == want
            sel = s[t, want]
            tot = np.float32(0)
            for v in sel:
                tot = np.float32(tot + v)
            assert np.array_equal(w[t], (sel / tot).astype(np.float32) * np.float32(2.5))
            assert abs(float(w[t].sum()) - 2.5) < 1e-5


def test_moe_sort_invariants_and_library():
    rng = np.random.default_rng(2)
    T, k, E = 257, 4, 16
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    order, offs, inv = O.moe_sort(ids, E)
    flat = ids.reshape(-1)
    assert sorted(order.tolist()) == list(range(T * k))
    assert offs[0] == 0 and offs[-1] == T * k and np.all(np.diff(offs) >= 0)
    for e in range(E):
        seg = order[offs[e]:offs[e + 1]]
        assert np.all(flat[seg] == e) and np.all(np.diff(seg) > 0)
    assert np.array_equal(order[inv], np.arange(T * k))
    ts = torch.sort(torch.from_numpy(flat.astype(np.int64)), stable=True).indices.numpy()
    assert np.array_equal(order, ts.astype(np.int32))
    # an expert nobody chose gets an empty range
    ids2 = np.zeros((5, 1), dtype=np.int32)
    _, offs2, _ = O.moe_sort(ids2, 3)
    assert list(offs2) == [0, 5, 5, 5]


def test_moe_mxfp4_forward_single_expert_reduces_to_two_gemms():
    """E = 1, k = 1, w = 1: the MoE is quantize -> GEMM -> SiLU-mul -> quantize -> GEMM."""
    rng = np.random.default_rng(3)
    T, H, I = 8, 64, 32
    x = F.bf16_to_f32(F.bf16_round(rng.standard_normal((T, H)).astype(np.float32)))
    w13 = (rng.standard_normal((1, 2 * I, H)) * 0.2).astype(np.float32)
    w2 = (rng.standard_normal((1, H, I)) * 0.2).astype(np.float32)
    w13p, w13s = F.quantize_mxfp4(w13)
    w2p, w2s = F.quantize_mxfp4(w2)
    ids = np.zeros((T, 1), dtype=np.int32)
    w = np.ones((T, 1), dtype=np.float32)
    y, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)
    xd = F.dequantize_mxfp4(*F.quantize_mxfp4(x))
    gu = xd @ F.dequantize_mxfp4(w13p[0], w13s[0]).T
    g, u = gu[:, :I].astype(np.float64), gu[:, I:]
    h = (g / (1 + np.exp(-g)) * u).astype(np.float32)
    hd = F.dequantize_mxfp4(*F.quantize_mxfp4(h))
    o = hd @ F.dequantize_mxfp4(w2p[0], w2s[0]).T
    want = F.bf16_round(F.bf16_to_f32(F.bf16_round(o)))
    assert np.array_equal(y, want)


def test_moe_mxfp4_forward_brute_force_tiny():
    """T=8, E=4, k=2, H=64, I=32: loop over tokens and choices instead of experts."""
    rng = np.random.default_rng(4)
    T, E, k, H, I = 8, 4, 2, 64, 32
    x = F.bf16_to_f32(F.bf16_round(rng.standard_normal((T, H)).astype(np.float32)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ids, w = O.topk_softmax(logits, k)
    w13p, w13s = F.quantize_mxfp4((rng.standard_normal((E, 2 * I, H)) * 0.2).astype(np.float32))
    w2p, w2s = F.quantize_mxfp4((rng.standard_normal((E, H, I)) * 0.2).astype(np.float32))
    y, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)
    xd = F.dequantize_mxfp4(*F.quantize_mxfp4(x))
    want = np.zeros((T, H), dtype=np.float32)
    for j in range(k):
        for t in range(T):
            e = ids[t, j]
            gu = xd[t:t + 1] @ F.dequantize_mxfp4(w13p[e], w13s[e]).T
            h = (O.silu(gu[:, :I]) * gu[:, I:]).astype(np.float32)
            hd = F.dequantize_mxfp4(*F.quantize_mxfp4(h))
            o = F.bf16_to_f32(F.bf16_round(hd @ F.dequantize_mxfp4(w2p[e], w2s[e]).T))
            want[t] += w[t, j] * o[0]
    got = F.bf16_to_f32(y)
    assert np.allclose(got, F.bf16_to_f32(F.bf16_round(want)), rtol=2e-2, atol=1e-6)


def test_moe_mxfp4_forward_mxfp8_activations_brute_force_tiny():
    """act_format "mxfp8": the same token-by-token loop with the MXFP8 activation quantizer; and the
    result lies closer to the forward pass on unquantized activations than the MXFP4 one does."""
    rng = np.random.default_rng(14)
    T, E, k, H, I = 8, 4, 2, 64, 32
    x = F.bf16_to_f32(F.bf16_round(rng.standard_normal((T, H)).astype(np.float32)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ids, w = O.topk_softmax(logits, k)
    w13p, w13s = F.quantize_mxfp4((rng.standard_normal((E, 2 * I, H)) * 0.2).astype(np.float32))
    w2p, w2s = F.quantize_mxfp4((rng.standard_normal((E, H, I)) * 0.2).astype(np.float32))
    y8, mid = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, act_format="mxfp8")
    y4, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)
    assert mid["hq"].shape == (T * k, I) and mid["xq"].shape == (T, H)
    xd = F.dequantize_mxfp8(*F.quantize_mxfp8(x))
    want = np.zeros((T, H), dtype=np.float32)
    exact = np.zeros((T, H), dtype=np.float64)
    for j in range(k):
        for t in range(T):
            e = ids[t, j]
            W13, W2 = F.dequantize_mxfp4(w13p[e], w13s[e]), F.dequantize_mxfp4(w2p[e], w2s[e])
            gu = xd[t:t + 1] @ W13.T
            h = (O.silu(gu[:, :I]) * gu[:, I:]).astype(np.float32)
            hd = F.dequantize_mxfp8(*F.quantize_mxfp8(h))
            want[t] += w[t, j] * F.bf16_to_f32(F.bf16_round(hd @ W2.T))[0]
            gx = x[t:t + 1].astype(np.float64) @ W13.T.astype(np.float64)
            hx = gx[:, :I] / (1 + np.exp(-gx[:, :I])) * gx[:, I:]
            exact[t] += w[t, j] * (hx @ W2.T.astype(np.float64))[0]
    assert np.allclose(F.bf16_to_f32(y8), F.bf16_to_f32(F.bf16_round(want)), rtol=2e-2, atol=1e-6)
    err8 = np.linalg.norm(F.bf16_to_f32(y8) - exact) / np.linalg.norm(exact)
    err4 = np.linalg.norm(F.bf16_to_f32(y4) - exact) / np.linalg.norm(exact)
    assert err8 < 0.5 * err4 and err8 < 0.1, (err8, err4)


def test_moe_fp8blk_forward_single_expert_reduces_to_two_gemms():
    """E = 1, k = 1, w = 1: dequantize -> GEMM -> SiLU-mul -> 1x128 re-quantize -> GEMM, written out
    here with explicit per-block scale products instead of dequantized matrices."""
    rng = np.random.default_rng(5)
    T, H, I = 6, 256, 128
    xq, xs = F.quantize_e4m3_blocks(rng.standard_normal((T, H)).astype(np.float32), 1, 128)
    w13q, w13s = F.quantize_e4m3_blocks((rng.standard_normal((2 * I, H)) * 0.2).astype(np.float32), 128, 128)
    w2q, w2s = F.quantize_e4m3_blocks((rng.standard_normal((H, I)) * 0.2).astype(np.float32), 128, 128)
    ids = np.zeros((T, 1), dtype=np.int32)
    w = np.ones((T, 1), dtype=np.float32)
    y = O.moe_fp8blk_forward(xq, xs, ids, w, w13q[None], w13s[None], w2q[None], w2s[None])
    xv, wv = F.e4m3_decode(xq).astype(np.float64), F.e4m3_decode(w13q).astype(np.float64)
    gu = np.zeros((T, 2 * I))
    for kb in range(H // 128):
        part = xv[:, kb * 128:(kb + 1) * 128] @ wv[:, kb * 128:(kb + 1) * 128].T
        gu += part * xs[:, kb:kb + 1].astype(np.float64) * np.repeat(w13s[:, kb], 128)[None, :]
    g, u = gu[:, :I], gu[:, I:]
    h = (g / (1 + np.exp(-g)) * u).astype(np.float32)
    hq, hs = F.quantize_e4m3_blocks(h, 1, 128)
    o = (F.e4m3_decode(hq).astype(np.float64) * hs.astype(np.float64)) @ \
        (F.e4m3_decode(w2q).astype(np.float64) * np.repeat(np.repeat(w2s, 128, 0), 128, 1)).T
    want = F.bf16_to_f32(F.bf16_round(F.bf16_to_f32(F.bf16_round(o.astype(np.float32)))))
    got = F.bf16_to_f32(y)
    # h may land on a different e4m3 code where fp32 and fp64 accumulation differ by an ulp
    assert np.allclose(got, want, rtol=3e-2, atol=1e-3)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 5e-3


def _tiny_moe(seed=3, T=12, E=3, k=2, H=64, I=32):
    rng = np.random.default_rng(seed)
    x = F.bf16_to_f32(F.bf16_round(rng.standard_normal((T, H)).astype(np.float32)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    w13p, w13s = F.quantize_mxfp4((rng.standard_normal((E, 2 * I, H)) * 0.3).astype(np.float32))
    w2p, w2s = F.quantize_mxfp4((rng.standard_normal((E, H, I)) * 0.3).astype(np.float32))
    ids, w = O.topk_softmax(logits, k)
    return rng, x, ids, w, w13p, w13s, w2p, w2s


def test_swiglu_clamped_against_torch_and_special_cases():
    """The clamped SwiGLU against the library routines (torch.clamp, torch.sigmoid) written the
    way the published model code writes it, plus the cases the formula fixes: above the limit
    the gate saturates, up is clamped on both sides, gate 0 gives 0, and with alpha 1 and no
    clamping it is silu(gate) * (up + 1)."""
    rng = np.random.default_rng(0)
    g = (rng.standard_normal(4096) * 5).astype(np.float32)
    u = (rng.standard_normal(4096) * 5).astype(np.float32)
    alpha, limit = 1.702, 7.0
    tg, tu = torch.from_numpy(g).double(), torch.from_numpy(u).double()
    tg = tg.clamp(max=limit)
    tu = tu.clamp(min=-limit, max=limit)
    want = ((tu + 1) * (tg * torch.sigmoid(tg * alpha))).float().numpy()
    got = O.swiglu_clamped(g, u, alpha, limit)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-7)
    f = np.float32
    assert O.swiglu_clamped(f(100.0), f(2.0), alpha, limit) == O.swiglu_clamped(f(7.0), f(2.0), alpha, limit)
    assert O.swiglu_clamped(f(1.0), f(50.0), alpha, limit) == O.swiglu_clamped(f(1.0), f(7.0), alpha, limit)
    assert O.swiglu_clamped(f(1.0), f(-50.0), alpha, limit) == O.swiglu_clamped(f(1.0), f(-7.0), alpha, limit)
    assert O.swiglu_clamped(f(0.0), f(3.0), alpha, limit) == 0.0
    assert O.swiglu_clamped(f(-100.0), f(3.0), alpha, limit) == pytest.approx(0.0, abs=1e-30)
    assert np.allclose(O.swiglu_clamped(g, u, 1.0, 1e30), O.silu(g) * (u + 1), rtol=1e-6, atol=1e-7)


def test_moe_mxfp4_forward_options_reduce_to_the_plain_forward():
    """Zero biases change nothing; interleaved rows are a pure re-ordering of w13 / bias13; the
    down bias of a top-1, weight-1 layer is added to the output once; a +1 on the up bias with
    SiLU is the clamped SwiGLU with alpha 1 and an unreachable limit."""
    rng, x, ids, w, w13p, w13s, w2p, w2s = _tiny_moe()
    E, twoI, _ = w13p.shape
    I, H = twoI // 2, x.shape[1]
    base, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)
    zero13, zero2 = np.zeros((E, twoI), np.float32), np.zeros((E, H), np.float32)
    same, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, bias13=zero13, bias2=zero2)
    assert np.array_equal(base, same)

    b13 = rng.standard_normal((E, twoI)).astype(np.float32)
    b2 = rng.standard_normal((E, H)).astype(np.float32)
    want, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, bias13=b13, bias2=b2, activation="swiglu_oai")
    perm = np.empty(twoI, dtype=np.int64)      # interleaved row 2c <- gate row c, 2c+1 <- up row I+c
    perm[0::2], perm[1::2] = np.arange(I), I + np.arange(I)
    got, _ = O.moe_mxfp4_forward(x, ids, w, w13p[:, perm], w13s[:, perm], w2p, w2s, bias13=b13[:, perm], bias2=b2,
                                 activation="swiglu_oai", interleaved=True)
    assert np.array_equal(want, got)
    assert not np.array_equal(want, base)

    ids1, w1 = ids[:, :1], np.ones((x.shape[0], 1), np.float32)
    y0 = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids1, w1, w13p, w13s, w2p, w2s)[0])
    y1 = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids1, w1, w13p, w13s, w2p, w2s, bias2=b2)[0])
    assert np.allclose(y1 - y0, b2[ids1[:, 0]], atol=2.0 ** -6 * np.maximum(np.abs(y0), np.abs(y1)).max())

    up_plus_one = zero13.copy()
    up_plus_one[:, I:] = 1.0
    ya = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, bias13=up_plus_one)[0])
    yb = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, activation="swiglu_oai", alpha=1.0,
                                           limit=1e30)[0])
    assert G.rel_fro_error(ya, yb) <= 2e-3  # a last-bit difference in h may flip an MX rounding


def test_moe_fp8blk_shared_expert_and_residual():
    """The shared expert is the one-expert layer; a zero residual changes nothing; with top-1
    weight-1 routing onto a copy of the shared expert's weights the layer output is, up to the
    two bf16 roundings, twice the shared expert's output."""
    rng = np.random.default_rng(4)
    T, H, I = 10, 128, 128
    xq, xs = F.quantize_e4m3_blocks(rng.standard_normal((T, H)).astype(np.float32), 1, 128)
    w13q, w13s = F.quantize_e4m3_blocks((rng.standard_normal((2 * I, H)) * 0.2).astype(np.float32), 128, 128)
    w2q, w2s = F.quantize_e4m3_blocks((rng.standard_normal((H, I)) * 0.2).astype(np.float32), 128, 128)
    w13q, w13s, w2q, w2s = w13q[None], w13s[None], w2q[None], w2s[None]
    shared = O.moe_fp8blk_shared_expert(xq, xs, w13q, w13s, w2q, w2s)
    ids, w = np.zeros((T, 1), np.int32), np.ones((T, 1), np.float32)
    base = O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s)
    assert np.array_equal(shared, base)
    assert np.array_equal(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s, y_add=np.zeros((T, H), np.float32)), base)
    both = F.bf16_to_f32(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s, y_add=F.bf16_to_f32(shared)))
    assert np.array_equal(both, 2 * F.bf16_to_f32(shared))  # doubling is exact in bf16


def test_moe_fp8blk_forward_brute_force_multi_expert():
    """T=9, E=4, k=3: token by token and choice by choice instead of expert by expert, with explicit
    per-block scale products in float64 over the raw codes (no dequantized matrices, no sort, no
    inverse map), so that the oracle's gather by sorted slot, its per-expert weight selection and its
    un-permute are checked against plain indexing by ids[t, j]."""
    rng = np.random.default_rng(8)
    T, E, k, H, I = 9, 4, 3, 256, 128
    xq, xs = F.quantize_e4m3_blocks(rng.standard_normal((T, H)).astype(np.float32), 1, 128)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ids, w = O.topk_grouped_sigmoid(logits, None, k, 2, 2)
    assert len(set(ids.reshape(-1).tolist())) == E          # every expert is used
    w13 = [F.quantize_e4m3_blocks((rng.standard_normal((2 * I, H)) * 0.2).astype(np.float32), 128, 128) for _ in range(E)]
    w2 = [F.quantize_e4m3_blocks((rng.standard_normal((H, I)) * 0.2).astype(np.float32), 128, 128) for _ in range(E)]
    w13q, w13s = np.stack([a for a, _ in w13]), np.stack([s for _, s in w13])
    w2q, w2s = np.stack([a for a, _ in w2]), np.stack([s for _, s in w2])
    y = O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s)

    xv = F.e4m3_decode(xq).astype(np.float64)
    want = np.zeros((T, H), dtype=np.float32)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            wv = F.e4m3_decode(w13q[e]).astype(np.float64)
            gu = np.zeros(2 * I)
            for kb in range(H // 128):
                part = wv[:, kb * 128:(kb + 1) * 128] @ xv[t, kb * 128:(kb + 1) * 128]
                gu += part * float(xs[t, kb]) * np.repeat(w13s[e][:, kb], 128).astype(np.float64)
            g, u = gu[:I], gu[I:]
            h = (g / (1 + np.exp(-g)) * u).astype(np.float32)
            hq, hs = F.quantize_e4m3_blocks(h[None, :], 1, 128)
            hv = F.e4m3_decode(hq[0]).astype(np.float64)
            o = np.zeros(H)
            for kb in range(I // 128):
                part = F.e4m3_decode(w2q[e][:, kb * 128:(kb + 1) * 128]).astype(np.float64) @ hv[kb * 128:(kb + 1) * 128]
                o += part * float(hs[0, kb]) * np.repeat(w2s[e][:, kb], 128).astype(np.float64)
            o_bf = F.bf16_to_f32(F.bf16_round(o.astype(np.float32)))
            want[t] += w[t, j] * o_bf
    got, want = F.bf16_to_f32(y), F.bf16_to_f32(F.bf16_round(want))
    # h may land on a neighbouring e4m3 code where fp32 and fp64 accumulation differ by an ulp
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 5e-3
    # a wrong expert for one (token, choice) or a mis-placed row would be an O(1) error in that row
    row_err = np.linalg.norm(got - want, axis=1) / np.linalg.norm(want, axis=1)
    assert row_err.max() < 2e-2
