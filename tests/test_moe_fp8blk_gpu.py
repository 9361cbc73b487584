"""FP8 block-scaled fused MoE on the GPU against the CPU oracle.

Bit-exact: the 1x128 activation quantizer (codes and fp32 scales). Floating point (y): relative
Frobenius error <= 1e-2 against the oracle (dequantize + fp32 matmul, h re-quantized with the same
1x128 rule), the north-star tolerance. The kernel folds one fp32 partial sum per 128-wide K block
into the accumulator, the oracle multiplies dequantized operands; both are exact products of the
same scales, so only summation order and the bf16 roundings differ.
"""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as GM
from oracle import moe as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


def _bf16(a):
    return F.bf16_to_f32(F.bf16_round(np.asarray(a, dtype=np.float32)))


def _fp8(t):
    return torch.from_numpy(t).to(DEV).view(torch.float8_e4m3fn)


@pytest.mark.parametrize("rows,cols", [(64, 256), (33, 7168), (1, 128), (500, 384)])
def test_quantize_rows_1x128_bit_exact(hk, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = _bf16(rng.standard_normal((rows, cols)) * np.exp2(rng.integers(-8, 8, size=(rows, 1))))
    x[0, :128] = 0.0
    xt = torch.from_numpy(F.bf16_round(x).view(np.int16)).view(torch.bfloat16).to(DEV)
    q = torch.zeros((rows, cols), dtype=torch.uint8, device=DEV)
    s = torch.zeros((rows, cols // 128), dtype=torch.float32, device=DEV)
    hk.tk_kernel.dispatch_fp8_quantize_rows_1x128(xt, q, s)
    torch.cuda.synchronize()
    qo, so = F.quantize_e4m3_blocks(x, 1, 128)
    assert np.array_equal(s.cpu().numpy(), so)
    assert np.array_equal(q.cpu().numpy(), qo)
    # the torch-side helper follows the same rule
    qt, st = hk.quant.quantize_fp8_blocks(torch.from_numpy(x).to(DEV), 1, 128)
    assert np.array_equal(st.cpu().numpy(), so) and np.array_equal(qt.view(torch.uint8).cpu().numpy(), qo)


def _case(rng, T, E, H, I, std=0.2):
    x = rng.standard_normal((T, H)).astype(np.float32)
    xq, xs = F.quantize_e4m3_blocks(x, 1, 128)
    w13 = (rng.standard_normal((E, 2 * I, H)) * std).astype(np.float32)
    w2 = (rng.standard_normal((E, H, I)) * std).astype(np.float32)
    w13q = np.empty((E, 2 * I, H), np.uint8); w13s = np.empty((E, 2 * I // 128, H // 128), np.float32)
    w2q = np.empty((E, H, I), np.uint8); w2s = np.empty((E, H // 128, I // 128), np.float32)
    for e in range(E):
        w13q[e], w13s[e] = F.quantize_e4m3_blocks(w13[e], 128, 128)
        w2q[e], w2s[e] = F.quantize_e4m3_blocks(w2[e], 128, 128)
    return xq, xs, w13q, w13s, w2q, w2s


CASES = [
    # T, E, k, G, KG, H, I
    (16, 4, 2, 2, 1, 128, 128),
    (64, 8, 2, 4, 2, 256, 128),
    (300, 8, 4, 4, 2, 512, 384),      # several m-tiles per expert
    (200, 32, 8, 8, 4, 1024, 256),    # DeepSeek-like routing parameters, small dims
    (96, 64, 4, 8, 4, 384, 128),      # many experts with few rows, some empty
    (600, 8, 4, 4, 2, 256, 128),      # about 300 rows per expert: two items of up to 160 rows per expert
    (520, 4, 2, 2, 1, 128, 256),      # 260 rows per expert, a single K-step in the gate+up GEMM
    (1000, 4, 2, 2, 1, 256, 128),     # about 500 rows per expert: four items, the rows spread evenly over them
    (330, 2, 2, 1, 1, 128, 128),      # 330 rows per expert (every token takes both experts): 112 + 112 + 106
]


@pytest.mark.parametrize("T,E,k,G,KG,H,I", CASES)
def test_moe_fp8blk_forward_matches_oracle(hk, T, E, k, G, KG, H, I):
    print(f"moe_fp8blk T={T} E={E} k={k} H={H} I={I}", flush=True)
    rng = np.random.default_rng(T + E + H + I)
    xq, xs, w13q, w13s, w2q, w2s = _case(rng, T, E, H, I)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.05).astype(np.float32)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk(
        _fp8(xq), torch.from_numpy(xs).to(DEV), torch.from_numpy(logits).to(DEV), torch.from_numpy(bias).to(DEV),
        _fp8(w13q), torch.from_numpy(w13s).to(DEV), _fp8(w2q), torch.from_numpy(w2s).to(DEV), y, k, G, KG, 2.5, ws)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    ids, w = O.topk_grouped_sigmoid(logits, bias, k, G, KG, 2.5)
    want = F.bf16_to_f32(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s))
    assert np.isfinite(got).all()
    err = GM.rel_fro_error(got, want)
    assert err <= TOL, err


@pytest.mark.parametrize("T,E,k,G,KG,H,I", CASES + [(40, 4, 2, 2, 1, 2048, 1024), (1, 8, 8, 1, 1, 256, 384),
                                                     (700, 16, 8, 4, 2, 896, 640)])
def test_moe_fp8blk_preshuffled_weights_give_identical_bits(hk, T, E, k, G, KG, H, I):
    """Weights in the pre-shuffled layout (loaded straight into MFMA operand registers, the fast path)
    against the plain layout (both operands through LDS): same MFMA, same K order, same scaling FMAs,
    so y must agree bit for bit; the plain path is the one the oracle tests above cover. Includes
    a single K-step per GEMM, experts without rows, one token, and several items per expert."""
    print(f"moe_fp8blk preshuffled T={T} E={E} k={k} H={H} I={I}", flush=True)
    rng = np.random.default_rng(T + E + H + I + 7)
    xq, xs, w13q, w13s, w2q, w2s = _case(rng, T, E, H, I)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    X, XS, LG = _fp8(xq), dev(xs), dev(logits)
    W13, S13, W2, S2 = _fp8(w13q), dev(w13s), _fp8(w2q), dev(w2s)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y0 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk(X, XS, LG, None, W13, S13, W2, S2, y0, k, G, KG, 1.0, ws)
    torch.cuda.synchronize()
    W = hk.tk_kernel.MoeFp8BlkShuffledWeights.from_plain(W13, S13, W2, S2)
    y1 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws.fill_(0xFF)
    hk.tk_kernel.dispatch_moe_fp8blk(X, XS, LG, None, W, None, None, None, y1, k, G, KG, 1.0, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(y1.float()).all()
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    # and directly against the oracle
    ids, w = O.topk_grouped_sigmoid(logits, None, k, G, KG, 1.0)
    want = F.bf16_to_f32(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s))
    assert GM.rel_fro_error(y1.float().cpu().numpy(), want) <= TOL


def test_moe_fp8blk_bf16_activations_are_quantized_once_per_token(hk):
    """The bf16-input layer = hk_fp8_quantize_rows_1x128 (bit-exact against the oracle, tested above)
    followed by the e4m3 layer: identical bits, plain and pre-shuffled weights."""
    T, E, k, G, KG, H, I = 150, 16, 4, 4, 2, 512, 256
    rng = np.random.default_rng(5)
    _, _, w13q, w13s, w2q, w2s = _case(rng, 1, E, H, I)
    x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).to(DEV)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    W13, S13, W2, S2 = _fp8(w13q), dev(w13s), _fp8(w2q), dev(w2s)
    xq = torch.zeros((T, H), dtype=torch.uint8, device=DEV)
    xs = torch.zeros((T, H // 128), dtype=torch.float32, device=DEV)
    hk.tk_kernel.dispatch_fp8_quantize_rows_1x128(x, xq, xs)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y0 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk(xq.view(torch.float8_e4m3fn), xs, logits, None, W13, S13, W2, S2, y0, k, G, KG, 1.0, ws)
    torch.cuda.synchronize()
    for weights in ((W13, S13, W2, S2), (hk.tk_kernel.MoeFp8BlkShuffledWeights.from_plain(W13, S13, W2, S2), None, None, None)):
        y1 = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
        ws.fill_(0xFF)
        hk.tk_kernel.dispatch_moe_fp8blk(x, None, logits, None, *weights, y1, k, G, KG, 1.0, ws)
        torch.cuda.synchronize()
        assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    with pytest.raises(RuntimeError):   # bf16 activations come without scales, e4m3 ones with
        hk.tk_kernel.dispatch_moe_fp8blk(x, xs, logits, None, W13, S13, W2, S2, y1, k, G, KG, 1.0, ws)


@pytest.mark.parametrize("T,E,k,G,KG,H,I,IS", [(64, 8, 2, 4, 2, 256, 128, 256), (200, 32, 8, 8, 4, 1024, 256, 128)])
def test_moe_fp8blk_with_shared_expert_matches_oracle(hk, T, E, k, G, KG, H, I, IS):
    """DeepSeek-V3 layer: routed experts (selection-only score bias) + a shared expert of
    intermediate size IS whose output is the residual of the weighted sum; y_add aliases y."""
    print(f"moe_fp8blk shared T={T} E={E} k={k} H={H} I={I} IS={IS}", flush=True)
    rng = np.random.default_rng(T + E + H + I + 1)
    xq, xs, w13q, w13s, w2q, w2s = _case(rng, T, E, H, I)
    _, _, s13q, s13s, s2q, s2s = _case(rng, 1, 1, H, IS)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    bias = (rng.standard_normal(E) * 0.05).astype(np.float32)
    dev = lambda a: torch.from_numpy(a).to(DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    ws_s = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, IS, 1, 1), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk_shared_expert(_fp8(xq), dev(xs), _fp8(s13q), dev(s13s), _fp8(s2q), dev(s2s), y, ws_s)
    torch.cuda.synchronize()
    shared_want = F.bf16_to_f32(O.moe_fp8blk_shared_expert(xq, xs, s13q, s13s, s2q, s2s))
    assert GM.rel_fro_error(y.float().cpu().numpy(), shared_want) <= TOL
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk(_fp8(xq), dev(xs), dev(logits), dev(bias), _fp8(w13q), dev(w13s), _fp8(w2q),
                                     dev(w2s), y, k, G, KG, 2.5, ws, y_add=y)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    ids, w = O.topk_grouped_sigmoid(logits, bias, k, G, KG, 2.5)
    want = F.bf16_to_f32(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s, y_add=shared_want))
    routed_only = F.bf16_to_f32(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s))
    assert np.isfinite(got).all()
    assert GM.rel_fro_error(got, want) <= TOL
    assert GM.rel_fro_error(got, routed_only) > 0.1  # the residual is not a rounding-level effect


def test_moe_unpermute_add_is_exact_for_representable_sums(hk):
    """Small integers: add + sum_j w_j o_j is exact in fp32 and in bf16."""
    rng = np.random.default_rng(2)
    T, k, H = 50, 3, 256
    o = rng.integers(-8, 9, size=(T * k, H)).astype(np.float32)
    add = rng.integers(-8, 9, size=(T, H)).astype(np.float32)
    w = rng.integers(1, 4, size=(T, k)).astype(np.float32)
    inv = rng.permutation(T * k).astype(np.int32)
    to_bf = lambda a: torch.from_numpy(a).to(DEV).to(torch.bfloat16)
    y = torch.zeros((T, H), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_unpermute(to_bf(o), torch.from_numpy(w).to(DEV), torch.from_numpy(inv).to(DEV), y,
                                        add=to_bf(add))
    torch.cuda.synchronize()
    want = add.copy()
    for j in range(k):
        want += w[:, j:j + 1] * o[inv[np.arange(T) * k + j]]
    assert np.array_equal(y.float().cpu().numpy(), want)


def test_moe_fp8blk_full_width_properties(hk):
    """DeepSeek-V3-like widths (H=7168, I=2048, E=256, k=8, 8 groups / top-4) at a reduced token
    count and expert storage that still fits the test budget: permutation invariance over tokens
    and the oracle on a sample of tokens."""
    T, E, k, G, KG, H, I = 1024, 256, 8, 8, 4, 7168, 2048
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randn(T, H, device=DEV, generator=g)
    xq, xs = hk.quant.quantize_fp8_blocks(x, 1, 128)
    logits = torch.randn(T, E, device=DEV, generator=g)
    # 32 distinct expert weight sets, repeated 8 times, keep device memory modest
    base13 = torch.randn(32, 2 * I, H, device=DEV, generator=g) * 0.02
    w13q32, w13s32 = hk.quant.quantize_fp8_blocks(base13, 128, 128)
    del base13
    base2 = torch.randn(32, H, I, device=DEV, generator=g) * 0.02
    w2q32, w2s32 = hk.quant.quantize_fp8_blocks(base2, 128, 128)
    del base2
    w13q, w13s = w13q32.repeat(8, 1, 1), w13s32.repeat(8, 1, 1)
    w2q, w2s = w2q32.repeat(8, 1, 1), w2s32.repeat(8, 1, 1)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk(xq, xs, logits, None, w13q, w13s, w2q, w2s, y, k, G, KG, 1.0, ws)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all()
    perm = torch.randperm(T, device=DEV, generator=g)
    y2 = torch.empty_like(y)
    hk.tk_kernel.dispatch_moe_fp8blk(xq[perm].contiguous(), xs[perm].contiguous(), logits[perm].contiguous(), None,
                                     w13q, w13s, w2q, w2s, y2, k, G, KG, 1.0, ws)
    torch.cuda.synchronize()
    assert torch.equal(y2, y[perm])
    sel = torch.arange(0, T, T // 8, device=DEV)[:8]
    ls = logits[sel].cpu().numpy()
    ids, w = O.topk_grouped_sigmoid(ls, None, k, G, KG, 1.0)
    used = np.unique(ids)
    remap = {int(e): i for i, e in enumerate(used)}
    ids_l = np.vectorize(remap.get)(ids).astype(np.int32)
    ut = torch.from_numpy(used.astype(np.int64)).to(DEV)
    want = F.bf16_to_f32(O.moe_fp8blk_forward(
        xq[sel].view(torch.uint8).cpu().numpy(), xs[sel].cpu().numpy(), ids_l, w,
        w13q[ut].view(torch.uint8).cpu().numpy(), w13s[ut].cpu().numpy(),
        w2q[ut].view(torch.uint8).cpu().numpy(), w2s[ut].cpu().numpy()))
    assert GM.rel_fro_error(y[sel].float().cpu().numpy(), want) <= TOL


def _drawn_layer_shapes(seed, count):
    """Seeded random layer shapes and routing parameters; H and I down to one 128-wide block."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        G = int(rng.choice([1, 2, 4, 8]))
        per = int(rng.choice([1, 2, 4, 8, 16]))
        KG = int(rng.integers(1, G + 1))
        k = int(rng.integers(1, min(KG * per, 8) + 1))
        T, H, I = int(rng.integers(1, 900)), int(rng.integers(1, 7)) * 128, int(rng.integers(1, 5)) * 128
        while G * per * I * H > 6e6 and (H > 128 or I > 128):
            H, I = max(128, H // 256 * 128), max(128, I // 256 * 128)
        out.append((T, G * per, k, G, KG, H, I))
    return out


@pytest.mark.parametrize("T,E,k,G,KG,H,I", _drawn_layer_shapes(78, 10))
def test_moe_fp8blk_forward_drawn_shapes(hk, T, E, k, G, KG, H, I):
    print(f"moe_fp8blk drawn T={T} E={E} k={k} G={G} KG={KG} H={H} I={I}", flush=True)
    rng = np.random.default_rng(T * 3 + E + H + I)
    xq, xs, w13q, w13s, w2q, w2s = _case(rng, T, E, H, I)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if (T + E) % 2:
        logits[:, rng.choice(E, size=max(1, E // 8), replace=False)] += 3.0
    bias = (rng.standard_normal(E) * 0.05).astype(np.float32)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.full((T, H), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_moe_fp8blk(
        _fp8(xq), torch.from_numpy(xs).to(DEV), torch.from_numpy(logits).to(DEV), torch.from_numpy(bias).to(DEV),
        _fp8(w13q), torch.from_numpy(w13s).to(DEV), _fp8(w2q), torch.from_numpy(w2s).to(DEV), y, k, G, KG, 2.5, ws)
    torch.cuda.synchronize()
    got = y.float().cpu().numpy()
    ids, w = O.topk_grouped_sigmoid(logits, bias, k, G, KG, 2.5)
    want = F.bf16_to_f32(O.moe_fp8blk_forward(xq, xs, ids, w, w13q, w13s, w2q, w2s))
    assert np.isfinite(got).all()
    assert GM.rel_fro_error(got, want) <= TOL
