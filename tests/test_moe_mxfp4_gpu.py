"""MXFP4 fused MoE on the GPU against the CPU oracle.

Bit-exact: activation quantizer (codes and e8m0 bytes). Floating point (y): relative Frobenius
error <= 1e-2 against the oracle, which quantizes activations with the same MX rule, dequantizes
weights and accumulates in fp32 (north-star tolerance). Size-independent properties at the full
GPT-OSS-like shape: permutation invariance of y under token reordering and linearity in the
routing weights.
"""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as G
from oracle import moe as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


def _bf16(a):
    return F.bf16_to_f32(F.bf16_round(np.asarray(a, dtype=np.float32)))


def _to_bf16_tensor(a):
    return torch.from_numpy(F.bf16_round(a).view(np.int16)).view(torch.bfloat16).to(DEV)


def _weights(rng, E, I, H, std=0.2):
    w13p, w13s = F.quantize_mxfp4((rng.standard_normal((E, 2 * I, H)) * std).astype(np.float32))
    w2p, w2s = F.quantize_mxfp4((rng.standard_normal((E, H, I)) * std).astype(np.float32))
    return w13p, w13s, w2p, w2s


def _pad(s):
    pad = (-s.shape[-1]) % 8
    return np.concatenate([s, np.full((*s.shape[:-1], pad), 127, np.uint8)], axis=-1) if pad else s


@pytest.mark.parametrize("rows,cols", [(64, 256), (33, 2880), (1, 32), (500, 96)])
def test_quantize_rows_bit_exact(hk, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = _bf16(rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-12, 12, size=(rows, 1))))
    x[0, :32] = 0.0
    pitch = (cols // 32 + 7) // 8 * 8
    xt = _to_bf16_tensor(x)
    packed = torch.zeros((rows, cols // 2), dtype=torch.uint8, device=DEV)
    scales = torch.zeros((rows, pitch), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_mxfp4_quantize_rows(xt, packed, scales)
    torch.cuda.synchronize()
    po, so = F.quantize_mxfp4(x)
    assert np.array_equal(packed.cpu().numpy(), po)
    assert np.array_equal(scales.cpu().numpy()[:, :cols // 32], so)
    assert np.all(scales.cpu().numpy()[:, cols // 32:] == 127)


def test_unpermute_matches_oracle(hk):
    rng = np.random.default_rng(0)
    T, k, H = 77, 4, 2880
    o = _bf16(rng.standard_normal((T * k, H)))
    w = rng.random((T, k)).astype(np.float32)
    inv = rng.permutation(T * k).astype(np.int32)
    y = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_unpermute(_to_bf16_tensor(o), torch.from_numpy(w).to(DEV), torch.from_numpy(inv).to(DEV), y)
    torch.cuda.synchronize()
    want = np.zeros((T, H), dtype=np.float64)
    for j in range(k):
        want += w[:, j:j + 1].astype(np.float64) * o[inv[np.arange(T) * k + j]]
    got = y.float().cpu().numpy()
    assert np.abs(got - want).max() <= np.abs(want).max() * 2.0 ** -7
    assert G.rel_fro_error(got, want) <= 4e-3  # one bf16 rounding


def _run_forward(hk, x, logits, w13p, w13s, w2p, w2s, k):
    """Runs the layer with plain and with pre-shuffled weights; both must agree bit for bit."""
    T, H = x.shape
    E, twoI, _ = w13p.shape
    I = twoI // 2
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    tw = [torch.from_numpy(w13p).to(DEV), torch.from_numpy(_pad(w13s)).to(DEV), torch.from_numpy(w2p).to(DEV),
          torch.from_numpy(_pad(w2s)).to(DEV)]
    xt, lt = _to_bf16_tensor(x), torch.from_numpy(logits).to(DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(xt, lt, tw[0], tw[1], tw[2], tw[3], y, k, ws)
    torch.cuda.synchronize()
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(*tw)
    y2 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(xt, lt, shuf, None, None, None, y2, k, ws)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16)), "plain and pre-shuffled weights disagree"
    return y.float().cpu().numpy()


CASES = [
    # T, E, k, H, I
    (8, 4, 2, 64, 32),        # the oracle's tiny brute-force case
    (64, 4, 2, 256, 128),
    (300, 8, 2, 512, 384),    # several m-tiles per expert (about 75 rows each, some > 128 after skew)
    (200, 16, 4, 2880, 2880 // 9 * 1),  # K tail (2880 = 11.25 * 256) with I = 320
    (96, 128, 4, 288, 160),   # many experts, most with 1-5 rows, some empty
]


@pytest.mark.parametrize("T,E,k,H,I", CASES)
def test_moe_mxfp4_forward_matches_oracle(hk, T, E, k, H, I):
    print(f"moe_mxfp4 T={T} E={E} k={k} H={H} I={I}", flush=True)
    rng = np.random.default_rng(T + E + H)
    x = _bf16(rng.standard_normal((T, H)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    got = _run_forward(hk, x, logits, w13p, w13s, w2p, w2s, k)
    ids, w = O.topk_softmax(logits, k)
    want_bits, _ = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)
    want = F.bf16_to_f32(want_bits)
    assert np.isfinite(got).all()
    err = G.rel_fro_error(got, want)
    assert err <= TOL, err


def _interleave_rows(a, I):
    """[E, 2I, ...] with gate rows 0..I-1 / up rows I..2I-1 -> rows 2c / 2c+1 = gate / up of column c."""
    perm = np.empty(2 * I, dtype=np.int64)
    perm[0::2], perm[1::2] = np.arange(I), I + np.arange(I)
    return np.ascontiguousarray(a[:, perm])


OPTION_CASES = [
    # T, E, k, H, I, biases, activation, interleaved
    (64, 4, 2, 256, 128, True, "swiglu_oai", True),     # everything at once (GPT-OSS experts)
    (64, 4, 2, 256, 128, True, "silu", False),          # biases alone
    (64, 4, 2, 256, 128, False, "swiglu_oai", False),   # activation alone
    (64, 4, 2, 256, 128, False, "silu", True),          # row order alone
    (300, 8, 2, 512, 384, True, "swiglu_oai", True),    # several m-tiles per expert, ragged tiles
    (200, 16, 4, 2880, 320, True, "swiglu_oai", True),  # K tail; I not a multiple of 128
    (96, 128, 4, 288, 160, True, "swiglu_oai", False),  # many experts, some empty
]


@pytest.mark.parametrize("T,E,k,H,I,biases,activation,interleaved", OPTION_CASES)
def test_moe_mxfp4_model_faithful_options_match_oracle(hk, T, E, k, H, I, biases, activation, interleaved):
    """Biases, clamped SwiGLU (alpha 1.702, limit 7) and interleaved gate / up rows, with plain and
    with pre-shuffled weights (bit-identical), against the oracle. Gate values are scaled so that
    a good part of them reaches the clamp."""
    print(f"moe_mxfp4 options T={T} E={E} k={k} H={H} I={I} {biases} {activation} {interleaved}", flush=True)
    rng = np.random.default_rng(T + E + H + 17)
    x = _bf16(rng.standard_normal((T, H)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H, std=0.35)
    b13 = (rng.standard_normal((E, 2 * I)) * 2).astype(np.float32) if biases else None
    b2 = rng.standard_normal((E, H)).astype(np.float32) if biases else None
    ids, w = O.topk_softmax(logits, k)
    want_bits, inter = O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, bias13=b13, bias2=b2,
                                           activation=activation)
    want = F.bf16_to_f32(want_bits)
    if activation == "swiglu_oai":  # the clamp must matter in this test
        gu = F.dequantize_mxfp4(*F.quantize_mxfp4(x))[:8] @ F.dequantize_mxfp4(w13p[0], w13s[0]).T
        assert (np.abs(gu) > 7.0).mean() > 0.01

    # device tensors in the caller's row order
    g13p, g13s, gb13 = w13p, w13s, b13
    if interleaved:
        g13p, g13s = _interleave_rows(w13p, I), _interleave_rows(w13s, I)
        gb13 = _interleave_rows(b13, I) if biases else None
    tw = [torch.from_numpy(g13p).to(DEV), torch.from_numpy(_pad(g13s)).to(DEV), torch.from_numpy(w2p).to(DEV),
          torch.from_numpy(_pad(w2s)).to(DEV)]
    opts = dict(bias13=torch.from_numpy(gb13).to(DEV) if biases else None,
                bias2=torch.from_numpy(b2).to(DEV) if biases else None, activation=activation,
                alpha=1.702, limit=7.0)
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    xt, lt = _to_bf16_tensor(x), torch.from_numpy(logits).to(DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(xt, lt, tw[0], tw[1], tw[2], tw[3], y, k, ws, interleaved=interleaved, **opts)
    torch.cuda.synchronize()
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(*tw, interleaved=interleaved)
    y2 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(xt, lt, shuf, None, None, None, y2, k, ws, **opts)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16)), "plain and pre-shuffled weights disagree"
    got = y.float().cpu().numpy()
    assert np.isfinite(got).all()
    err = G.rel_fro_error(got, want)
    assert err <= TOL, err


def test_moe_mxfp4_options_bad_arguments(hk):
    T, E, k, H, I = 16, 4, 2, 64, 32
    rng = np.random.default_rng(0)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    tw = [torch.from_numpy(w13p).to(DEV), torch.from_numpy(_pad(w13s)).to(DEV), torch.from_numpy(w2p).to(DEV),
          torch.from_numpy(_pad(w2s)).to(DEV)]
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    lt = torch.zeros((T, E), dtype=torch.float32, device=DEV)
    y = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, *tw, y, k, ws, activation="gelu")
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, *tw, y, k, ws, bias13=torch.zeros((E, I), device=DEV))
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, *tw, y, k, ws, bias2=torch.zeros((E, H), dtype=torch.float64, device=DEV))
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, *tw, y, k, ws, activation="swiglu_oai", limit=0.0)
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(*tw, interleaved=True)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, shuf, None, None, None, y, k, ws, interleaved=False)


def test_moe_mxfp4_skewed_routing_many_rows_per_expert(hk):
    """All tokens on two experts: 2 x 600 rows -> five m-tiles per expert; others empty."""
    rng = np.random.default_rng(5)
    T, E, k, H, I = 600, 6, 2, 256, 256
    x = _bf16(rng.standard_normal((T, H)))
    logits = np.full((T, E), -5.0, dtype=np.float32)
    logits[:, 1] = 3.0 + rng.random(T).astype(np.float32)
    logits[:, 4] = 2.0 + rng.random(T).astype(np.float32)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    got = _run_forward(hk, x, logits, w13p, w13s, w2p, w2s, k)
    ids, w = O.topk_softmax(logits, k)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)[0])
    assert G.rel_fro_error(got, want) <= TOL


def test_moe_mxfp4_full_shape_properties(hk):
    """GPT-OSS-like shape (T=4096, H=I=2880, E=128, k=4): checks that do not need the CPU oracle
    at full size, plus the oracle on a sample of tokens (experts evaluated only for those tokens)."""
    T, E, k, H, I = 4096, 128, 4, 2880, 2880
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(T, H, device=DEV, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device=DEV, generator=g)
    w13p = torch.empty((E, 2 * I, H // 2), dtype=torch.uint8, device=DEV)
    w13s = torch.empty((E, 2 * I, 96), dtype=torch.uint8, device=DEV)
    w2p = torch.empty((E, H, I // 2), dtype=torch.uint8, device=DEV)
    w2s = torch.empty((E, H, 96), dtype=torch.uint8, device=DEV)
    for e in range(E):  # per expert, to bound temporaries
        a, s = hk.quant.quantize_mxfp4(torch.randn(2 * I, H, device=DEV, generator=g) * 0.02)
        w13p[e], w13s[e] = a, hk.quant.pad_scales(s)
        a, s = hk.quant.quantize_mxfp4(torch.randn(H, I, device=DEV, generator=g) * 0.02)
        w2p[e], w2s[e] = a, hk.quant.pad_scales(s)
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(x, logits, w13p, w13s, w2p, w2s, y, k, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(w13p, w13s, w2p, w2s)
    y3 = torch.empty_like(y)
    hk.tk_kernel.dispatch_moe_mxfp4(x, logits, shuf, None, None, None, y3, k, ws)
    torch.cuda.synchronize()
    assert torch.equal(y3, y)  # pre-shuffled weight layout: identical arithmetic
    # (1) token permutation: y is a per-token function -> permuting inputs permutes outputs exactly
    perm = torch.randperm(T, device=DEV, generator=g)
    y2 = torch.empty_like(y)
    hk.tk_kernel.dispatch_moe_mxfp4(x[perm].contiguous(), logits[perm].contiguous(), w13p, w13s, w2p, w2s, y2, k, ws)
    torch.cuda.synchronize()
    assert torch.equal(y2, y[perm])
    # (2) oracle on 24 sampled tokens
    sel = torch.arange(0, T, T // 24, device=DEV)[:24]
    xs = x[sel].float().cpu().numpy()
    ls = logits[sel].cpu().numpy()
    ids, w = O.topk_softmax(ls, k)
    used = np.unique(ids)
    remap = {int(e): i for i, e in enumerate(used)}
    ids_l = np.vectorize(remap.get)(ids).astype(np.int32)
    ut = torch.from_numpy(used.astype(np.int64)).to(DEV)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(
        xs, ids_l, w, w13p[ut].cpu().numpy(), w13s[ut][:, :, :H // 32].cpu().numpy(),
        w2p[ut].cpu().numpy(), w2s[ut][:, :, :I // 32].cpu().numpy())[0])
    got = y[sel].float().cpu().numpy()
    assert G.rel_fro_error(got, want) <= TOL


def _drawn_layer_shapes(seed, count):
    """Seeded random layer shapes: few and many experts, H and I down to one MX block."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        E = int(rng.choice([1, 2, 3, 8, 33, 128]))
        k = int(rng.integers(1, min(E, 8) + 1))
        T, H, I = int(rng.integers(1, 700)), int(rng.integers(1, 25)) * 32, int(rng.integers(1, 17)) * 32
        while E * I * H > 6e6:
            H, I = max(32, H // 64 * 32), max(32, I // 64 * 32)
        out.append((T, E, k, H, I))
    return out


@pytest.mark.parametrize("T,E,k,H,I", _drawn_layer_shapes(77, 10))
def test_moe_mxfp4_forward_drawn_shapes(hk, T, E, k, H, I):
    print(f"moe_mxfp4 drawn T={T} E={E} k={k} H={H} I={I}", flush=True)
    rng = np.random.default_rng(T * 3 + E + H + I)
    x = _bf16(rng.standard_normal((T, H)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if (T + E) % 2:  # a few hot experts: many rows on some experts, none on others
        logits[:, rng.choice(E, size=max(1, E // 8), replace=False)] += 3.0
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    got = _run_forward(hk, x, logits, w13p, w13s, w2p, w2s, k)
    ids, w = O.topk_softmax(logits, k)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)[0])
    assert np.isfinite(got).all()
    assert G.rel_fro_error(got, want) <= TOL


def _device_layer(hk, T, E, k, H, I, seed):
    """Seeded layer on the device: x, logits, plain weights (scale rows padded to a multiple of 8)."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(T, H, device=DEV, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device=DEV, generator=g)
    pitch = (max(H, I) // 32 + 7) // 8 * 8
    w13p = torch.empty((E, 2 * I, H // 2), dtype=torch.uint8, device=DEV)
    w13s = torch.full((E, 2 * I, (H // 32 + 7) // 8 * 8), 127, dtype=torch.uint8, device=DEV)
    w2p = torch.empty((E, H, I // 2), dtype=torch.uint8, device=DEV)
    w2s = torch.full((E, H, (I // 32 + 7) // 8 * 8), 127, dtype=torch.uint8, device=DEV)
    for e in range(E):
        a, s = hk.quant.quantize_mxfp4(torch.randn(2 * I, H, device=DEV, generator=g) * 0.1)
        w13p[e], w13s[e] = a, hk.quant.pad_scales(s)
        a, s = hk.quant.quantize_mxfp4(torch.randn(H, I, device=DEV, generator=g) * 0.1)
        w2p[e], w2s[e] = a, hk.quant.pad_scales(s)
    del pitch
    return x, logits, w13p, w13s, w2p, w2s


def _oracle_on_sample(x, logits, w13p, w13s, w2p, w2s, k, y, count, act_format="mxfp4"):
    """Oracle on `count` evenly spaced tokens, evaluating only the experts they use."""
    T, H = x.shape
    I = w2p.shape[2] * 2
    sel = torch.arange(0, T, max(1, T // count), device=DEV)[:count]
    ids, w = O.topk_softmax(logits[sel].cpu().numpy(), k)
    used = np.unique(ids)
    remap = {int(e): i for i, e in enumerate(used)}
    ids_l = np.vectorize(remap.get)(ids).astype(np.int32)
    ut = torch.from_numpy(used.astype(np.int64)).to(DEV)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(
        x[sel].float().cpu().numpy(), ids_l, w, w13p[ut].cpu().numpy(), w13s[ut][:, :, :H // 32].cpu().numpy(),
        w2p[ut].cpu().numpy(), w2s[ut][:, :, :I // 32].cpu().numpy(), act_format=act_format)[0])
    return G.rel_fro_error(y[sel].float().cpu().numpy(), want)


# The gate+up kernel fetches its activation rows either by token from x quantized once per token
# (small x; up to 16384 slots the quantization rides in the sort's launch) or from x permuted into
# sorted order; the cases below reach every combination through both entry points.
PATH_CASES = [
    # T, E, k, H, I, act_format
    (300, 8, 2, 512, 384, "mxfp4"),      # gathered rows, one fused sort + quantize launch
    (300, 8, 2, 512, 384, "mxfp8"),
    (8192, 16, 4, 1024, 128, "mxfp4"),   # gathered rows, 32768 slots: three-launch sort, separate quantizer
    (8192, 8, 2, 1664, 256, "mxfp4"),    # x too large to gather: permuted rows
    (4096, 8, 2, 1664, 256, "mxfp8"),    # the same with MXFP8 activations
    (2048, 8, 2, 4352, 128, "mxfp4"),    # gathered rows, K of 17 K-steps: two scale super-steps per item
]


@pytest.mark.parametrize("T,E,k,H,I,act_format", PATH_CASES)
def test_moe_mxfp4_activation_paths_and_experts_entry(hk, T, E, k, H, I, act_format):
    print(f"moe_mxfp4 paths T={T} E={E} k={k} H={H} I={I} {act_format}", flush=True)
    x, logits, w13p, w13s, w2p, w2s = _device_layer(hk, T, E, k, H, I, seed=T + H)
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(w13p, w13s, w2p, w2s)
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k, act_format=act_format), dtype=torch.uint8,
                     device=DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(x, logits, shuf, None, None, None, y, k, ws, act_format=act_format)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    assert _oracle_on_sample(x, logits, w13p, w13s, w2p, w2s, k, y, 32, act_format) <= TOL
    # the extended epilogue with zero biases: the kernel that takes permuted rows; identical arithmetic
    yb = torch.full_like(y, float("nan"))
    hk.tk_kernel.dispatch_moe_mxfp4(x, logits, shuf, None, None, None, yb, k, ws, act_format=act_format,
                                    bias13=torch.zeros((E, 2 * I), device=DEV), bias2=torch.zeros((E, H), device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(yb, y)
    if act_format == "mxfp4":  # plain weight layout (MXFP4 activations only): permuted rows as well
        yp = torch.full_like(y, float("nan"))
        hk.tk_kernel.dispatch_moe_mxfp4(x, logits, w13p, w13s, w2p, w2s, yp, k, ws)
        torch.cuda.synchronize()
        assert torch.equal(yp, y)
    # the experts entry point on the caller's routing
    ids = torch.empty((T, k), dtype=torch.int32, device=DEV)
    wts = torch.empty((T, k), dtype=torch.float32, device=DEV)
    hk.tk_kernel.dispatch_moe_topk_softmax(logits, ids, wts)
    sorted_slots = torch.empty(T * k, dtype=torch.int32, device=DEV)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=DEV)
    inv = torch.empty(T * k, dtype=torch.int32, device=DEV)
    sws = torch.empty(hk.tk_kernel.moe_sort_workspace_bytes(T, k, E), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_moe_sort(ids, sorted_slots, offsets, inv, sws)
    ye = torch.full_like(y, float("nan"))
    ws.fill_(0x5A)
    hk.tk_kernel.dispatch_moe_mxfp4_experts(x, shuf, None, None, None, wts, sorted_slots, offsets, inv, ye, ws,
                                            act_format=act_format)
    torch.cuda.synchronize()
    assert torch.equal(ye, y)


def test_unpermute_skips_positions_outside_the_rows_of_o(hk):
    """A position outside [0, T*k) in slot_to_pos is not read and adds nothing: o sits at the end of a
    NaN-filled pool, so a read past it (or in front of it) would show in y."""
    rng = np.random.default_rng(5)
    for T, k, H in ((50, 4, 512), (9, 8, 1024), (6, 11, 256)):
        S = T * k
        pool = torch.full(((S + 64) * H,), float("nan"), dtype=torch.bfloat16, device=DEV)
        o = pool[32 * H:(32 + S) * H].view(S, H)
        o.copy_(_to_bf16_tensor(_bf16(rng.standard_normal((S, H)))))
        w = rng.random((T, k)).astype(np.float32)
        inv = rng.permutation(S).astype(np.int32)
        bad = rng.random(S) < 0.3
        inv_bad = inv.copy()
        inv_bad[bad] = rng.choice(np.array([-1, -7, S, S + 3, 2 ** 31 - 1, -2 ** 31], dtype=np.int64),
                                  size=int(bad.sum())).astype(np.int32)
        y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
        hk.tk_kernel.dispatch_moe_unpermute(o, torch.from_numpy(w).to(DEV), torch.from_numpy(inv_bad).to(DEV), y)
        # the same call with the bad slots' weights zeroed and their positions valid
        w0 = np.where(bad.reshape(T, k), 0.0, w).astype(np.float32)
        y0 = torch.full_like(y, float("nan"))
        hk.tk_kernel.dispatch_moe_unpermute(o, torch.from_numpy(w0).to(DEV), torch.from_numpy(inv).to(DEV), y0)
        torch.cuda.synchronize()
        assert torch.isfinite(y.float()).all()
        assert torch.equal(y, y0)


def test_moe_mxfp4_experts_with_positions_out_of_range(hk):
    """hk_moe_mxfp4_experts on a slot_to_pos with entries outside [0, T*k): normal exit, finite output,
    and the tokens whose positions are intact get what the intact call gives them."""
    T, E, k, H, I = 200, 8, 2, 512, 256
    x, logits, w13p, w13s, w2p, w2s = _device_layer(hk, T, E, k, H, I, seed=11)
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(w13p, w13s, w2p, w2s)
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    ids = torch.empty((T, k), dtype=torch.int32, device=DEV)
    wts = torch.empty((T, k), dtype=torch.float32, device=DEV)
    hk.tk_kernel.dispatch_moe_topk_softmax(logits, ids, wts)
    sorted_slots = torch.empty(T * k, dtype=torch.int32, device=DEV)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=DEV)
    inv = torch.empty(T * k, dtype=torch.int32, device=DEV)
    sws = torch.empty(hk.tk_kernel.moe_sort_workspace_bytes(T, k, E), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_moe_sort(ids, sorted_slots, offsets, inv, sws)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4_experts(x, shuf, None, None, None, wts, sorted_slots, offsets, inv, y, ws)
    inv_bad = inv.clone()
    broken_tokens = torch.tensor([0, 17, 63, T - 1], device=DEV)
    inv_bad.view(T, k)[broken_tokens, 0] = torch.tensor([-1, T * k, 2 ** 31 - 1, -2 ** 31], dtype=torch.int32, device=DEV)
    yb = torch.full_like(y, float("nan"))
    hk.tk_kernel.dispatch_moe_mxfp4_experts(x, shuf, None, None, None, wts, sorted_slots, offsets, inv_bad, yb, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(yb.float()).all()
    intact = torch.ones(T, dtype=torch.bool, device=DEV)
    intact[broken_tokens] = False
    assert torch.equal(yb[intact], y[intact])
