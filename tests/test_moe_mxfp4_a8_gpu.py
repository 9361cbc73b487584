"""MXFP4-weight MoE with MXFP8 activations (W4A8) on the GPU against the CPU oracle.

Bit-exact: the MXFP8 row quantizer (e4m3 codes and e8m0 bytes, saturation included). Floating point
(y): relative Frobenius error <= 1e-2 against the oracle, which quantizes x and h with the same MX
rule, dequantizes the weights and accumulates in fp32. The mixed fp4 x fp8 MFMA path exists for the
pre-shuffled weight layout only.
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


def _pad(s):
    pad = (-s.shape[-1]) % 8
    return np.concatenate([s, np.full((*s.shape[:-1], pad), 127, np.uint8)], axis=-1) if pad else s


def _weights(rng, E, I, H, std=0.2):
    w13p, w13s = F.quantize_mxfp4((rng.standard_normal((E, 2 * I, H)) * std).astype(np.float32))
    w2p, w2s = F.quantize_mxfp4((rng.standard_normal((E, H, I)) * std).astype(np.float32))
    return w13p, w13s, w2p, w2s


def _interleave_rows(a, I):
    perm = np.empty(2 * I, dtype=np.int64)
    perm[0::2], perm[1::2] = np.arange(I), I + np.arange(I)
    return np.ascontiguousarray(a[:, perm])


@pytest.mark.parametrize("rows,cols", [(64, 256), (33, 2880), (1, 32), (500, 96)])
def test_mxfp8_quantize_rows_bit_exact(hk, rows, cols):
    """Codes and scale bytes of the device quantizer against the oracle, with block maxima of
    every kind: ordinary, in the saturating range [1.75, 2) * 2^n, exact powers of two, zero
    blocks, and ties between two e4m3 values."""
    print(f"mxfp8 quantize rows {rows}x{cols}", flush=True)
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-12, 12, size=(rows, 1)))
    x[0, :32] = 0.0
    x[rows // 2, 0] = 1.9 * 2.0 ** 5       # block maximum that saturates: 1.9 * 2^5 / 2^(5-8) = 486 > 448
    x[rows // 2, 1] = 17.0 / 16 * 2.0 ** 2  # 1.0625 * 2^2: a tie between two codes after scaling
    x[rows - 1, cols - 32:] = 0.0
    x[rows - 1, cols - 1] = -2.0 ** 7
    x = _bf16(x)
    pitch = (cols // 32 + 7) // 8 * 8
    codes = torch.zeros((rows, cols), dtype=torch.float8_e4m3fn, device=DEV)
    scales = torch.zeros((rows, pitch), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_mxfp8_quantize_rows(_to_bf16_tensor(x), codes, scales)
    torch.cuda.synchronize()
    co, so = F.quantize_mxfp8(x)
    assert np.array_equal(scales.cpu().numpy()[:, :cols // 32], so)
    assert np.all(scales.cpu().numpy()[:, cols // 32:] == 127)
    got = codes.view(torch.uint8).cpu().numpy()
    # +0 and -0 codes of zero elements are both correct encodings of zero: compare values there
    same = (got == co) | ((got & 0x7F) == 0) & ((co & 0x7F) == 0)
    assert same.all(), np.argwhere(~same)[:5]


CASES = [
    # T, E, k, H, I
    (8, 4, 2, 64, 32),
    (64, 4, 2, 256, 128),
    (300, 8, 2, 512, 384),     # several m-tiles per expert (128-row items), ragged tiles
    (200, 16, 4, 2880, 320),   # K tail in both GEMMs (2880 = 11.25 * 256, 320 = 1.25 * 256)
    (96, 128, 4, 288, 160),    # many experts, most with 1-5 rows, some empty
]


def _run(hk, x, logits, w13p, w13s, w2p, w2s, k, interleaved=False, **opts):
    T, H = x.shape
    E, twoI, _ = w13p.shape
    I = twoI // 2
    tw = [torch.from_numpy(w13p).to(DEV), torch.from_numpy(_pad(w13s)).to(DEV), torch.from_numpy(w2p).to(DEV),
          torch.from_numpy(_pad(w2s)).to(DEV)]
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(*tw, interleaved=interleaved)
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k, act_format="mxfp8"), dtype=torch.uint8,
                     device=DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_mxfp4(_to_bf16_tensor(x), torch.from_numpy(logits).to(DEV), shuf, None, None, None, y,
                                    k, ws, act_format="mxfp8", **opts)
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


@pytest.mark.parametrize("T,E,k,H,I", CASES)
def test_moe_mxfp4_a8_forward_matches_oracle(hk, T, E, k, H, I):
    print(f"moe_mxfp4 a8 T={T} E={E} k={k} H={H} I={I}", flush=True)
    rng = np.random.default_rng(T + E + H + 3)
    x = _bf16(rng.standard_normal((T, H)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    got = _run(hk, x, logits, w13p, w13s, w2p, w2s, k)
    ids, w = O.topk_softmax(logits, k)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, act_format="mxfp8")[0])
    assert np.isfinite(got).all()
    err = G.rel_fro_error(got, want)
    assert err <= TOL, err
    # and it is the MXFP8 path that ran: the MXFP4-activation result differs by far more than the tolerance
    want4 = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s)[0])
    assert G.rel_fro_error(got, want4) > 5 * max(err, 1e-3)


def test_moe_mxfp4_a8_skewed_routing_many_rows_per_expert(hk):
    """All tokens on two experts: 2 x 600 rows -> five 128-row items per expert; others empty."""
    rng = np.random.default_rng(5)
    T, E, k, H, I = 600, 6, 2, 256, 256
    x = _bf16(rng.standard_normal((T, H)))
    logits = np.full((T, E), -5.0, dtype=np.float32)
    logits[:, 1] = 3.0 + rng.random(T).astype(np.float32)
    logits[:, 4] = 2.0 + rng.random(T).astype(np.float32)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    got = _run(hk, x, logits, w13p, w13s, w2p, w2s, k)
    ids, w = O.topk_softmax(logits, k)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, act_format="mxfp8")[0])
    assert G.rel_fro_error(got, want) <= TOL


@pytest.mark.parametrize("T,E,k,H,I,interleaved", [(64, 4, 2, 256, 128, True), (300, 8, 2, 512, 384, False),
                                                   (200, 16, 4, 2880, 320, True)])
def test_moe_mxfp4_a8_model_faithful_options_match_oracle(hk, T, E, k, H, I, interleaved):
    """Biases, clamped SwiGLU and interleaved gate / up rows with MXFP8 activations."""
    print(f"moe_mxfp4 a8 options T={T} E={E} k={k} H={H} I={I} {interleaved}", flush=True)
    rng = np.random.default_rng(T + E + H + 29)
    x = _bf16(rng.standard_normal((T, H)))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H, std=0.35)
    b13 = (rng.standard_normal((E, 2 * I)) * 2).astype(np.float32)
    b2 = rng.standard_normal((E, H)).astype(np.float32)
    ids, w = O.topk_softmax(logits, k)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(x, ids, w, w13p, w13s, w2p, w2s, bias13=b13, bias2=b2,
                                             activation="swiglu_oai", act_format="mxfp8")[0])
    g13p, g13s, gb13 = w13p, w13s, b13
    if interleaved:
        g13p, g13s, gb13 = _interleave_rows(w13p, I), _interleave_rows(w13s, I), _interleave_rows(b13, I)
    got = _run(hk, x, logits, g13p, g13s, w2p, w2s, k, interleaved=interleaved,
               bias13=torch.from_numpy(gb13).to(DEV), bias2=torch.from_numpy(b2).to(DEV),
               activation="swiglu_oai", alpha=1.702, limit=7.0)
    assert np.isfinite(got).all()
    err = G.rel_fro_error(got, want)
    assert err <= TOL, err


def test_moe_mxfp4_a8_needs_preshuffled_weights(hk):
    T, E, k, H, I = 16, 4, 2, 64, 32
    rng = np.random.default_rng(0)
    w13p, w13s, w2p, w2s = _weights(rng, E, I, H)
    tw = [torch.from_numpy(w13p).to(DEV), torch.from_numpy(_pad(w13s)).to(DEV), torch.from_numpy(w2p).to(DEV),
          torch.from_numpy(_pad(w2s)).to(DEV)]
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k, act_format="mxfp8"), dtype=torch.uint8,
                     device=DEV)
    x = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    lt = torch.zeros((T, E), dtype=torch.float32, device=DEV)
    y = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, *tw, y, k, ws, act_format="mxfp8")
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, *tw, y, k, ws, act_format="fp16")
    # the MXFP4-activation workspace is too small for MXFP8 activations: refused, not overrun
    small = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(*tw)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_moe_mxfp4(x, lt, shuf, None, None, None, y, k, small, act_format="mxfp8")


def test_moe_mxfp4_a8_full_shape_properties(hk):
    """GPT-OSS-like shape (T=4096, H=I=2880, E=128, k=4) with MXFP8 activations: token-permutation
    equivariance (bit for bit), the extended epilogue with zero biases and SiLU equals the plain
    one (bit for bit: two instantiations of the kernel), and the oracle on 16 sampled tokens."""
    T, E, k, H, I = 4096, 128, 4, 2880, 2880
    print("moe_mxfp4 a8 full shape", flush=True)
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
    shuf = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(w13p, w13s, w2p, w2s)
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k, act_format="mxfp8"), dtype=torch.uint8,
                     device=DEV)
    run = lambda xx, ll, out, **kw: hk.tk_kernel.dispatch_moe_mxfp4(xx, ll, shuf, None, None, None, out, k, ws,
                                                                   act_format="mxfp8", **kw)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    run(x, logits, y)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    perm = torch.randperm(T, device=DEV, generator=g)
    y2 = torch.empty_like(y)
    run(x[perm].contiguous(), logits[perm].contiguous(), y2)
    torch.cuda.synchronize()
    assert torch.equal(y2, y[perm])
    y3 = torch.empty_like(y)
    run(x, logits, y3, bias13=torch.zeros((E, 2 * I), device=DEV), bias2=torch.zeros((E, H), device=DEV))
    torch.cuda.synchronize()
    assert torch.equal(y3, y)
    sel = torch.arange(0, T, T // 16, device=DEV)[:16]
    ids, w = O.topk_softmax(logits[sel].cpu().numpy(), k)
    used = np.unique(ids)
    remap = {int(e): i for i, e in enumerate(used)}
    ids_l = np.vectorize(remap.get)(ids).astype(np.int32)
    ut = torch.from_numpy(used.astype(np.int64)).to(DEV)
    want = F.bf16_to_f32(O.moe_mxfp4_forward(
        x[sel].float().cpu().numpy(), ids_l, w, w13p[ut].cpu().numpy(), w13s[ut][:, :, :H // 32].cpu().numpy(),
        w2p[ut].cpu().numpy(), w2s[ut][:, :, :I // 32].cpu().numpy(), act_format="mxfp8")[0])
    assert G.rel_fro_error(y[sel].float().cpu().numpy(), want) <= TOL
