"""The GEMM kernels for few rows of A (at most 64; FP8 variant 8, BF16 and MXFP4 variant 6) against the CPU
oracle, through the C ABI.

Tolerance: relative Frobenius error <= 5e-3 on the bf16 output (the north-star bound is 1e-2; accumulation
order and the single bf16 rounding are the only differences, ~2e-3 observed). Exactly representable cases
are checked bit for bit. Operands sit inside pools of NaN codes and C between NaN guards: a fetch past a
row's K, past the last row or a store outside C would show.
"""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as G

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# (M, N, K): every row-fragment count (M <= 16 / 32 / 64), N not a multiple of 32 or of 4, K tails
# (K % 128 != 0), fewer K-steps than waves, the MoE models' 2880
SHAPES = [(1, 32, 128), (16, 32, 128), (16, 64, 1024), (7, 100, 144), (16, 101, 272), (17, 96, 2880),
          (32, 200, 2048), (33, 72, 640), (48, 31, 16), (64, 520, 6160), (3, 2880, 2880), (64, 64, 8192)]


def _in_pool(codes: np.ndarray, fill: int, dtype):
    """The array's bytes in the middle of a device buffer filled with `fill`, viewed as `dtype`."""
    raw = torch.from_numpy(codes.view(np.uint8).reshape(codes.shape[0], -1)).to(DEV)
    rows, row_bytes = raw.shape
    n = rows * row_bytes
    pad = (n + 4096 + 255) // 256 * 256
    pool = torch.full((pad + n + pad,), fill, dtype=torch.uint8, device=DEV)
    view = pool[pad:pad + n].view(rows, row_bytes)
    view.copy_(raw)
    return view.view(dtype), pool


def _guarded_c(M, N):
    buf = torch.full((512 + M * N + 512,), float("nan"), dtype=torch.bfloat16, device=DEV)
    return buf[512:512 + M * N].view(M, N), buf


def _check_guards(buf, M, N):
    assert torch.isnan(buf[:512]).all() and torch.isnan(buf[512 + M * N:]).all(), "store outside C"


def _fp8(hk, a, b, sa, sb, variant):
    A, _pa = _in_pool(a, 0x7F, torch.float8_e4m3fn)   # e4m3fn NaN code
    B, _pb = _in_pool(b, 0x7F, torch.float8_e4m3fn)
    C, buf = _guarded_c(a.shape[0], b.shape[0])
    hk.tk_kernel.dispatch_fp8_gemm(A, B, C, sa, sb, variant=variant)
    torch.cuda.synchronize()
    _check_guards(buf, a.shape[0], b.shape[0])
    return C.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _bf16(hk, a_bits, b_bits, variant):
    A, _pa = _in_pool(a_bits, 0xFF, torch.bfloat16)   # 0xFFFF: a bf16 NaN
    B, _pb = _in_pool(b_bits, 0xFF, torch.bfloat16)
    C, buf = _guarded_c(a_bits.shape[0], b_bits.shape[0])
    hk.tk_kernel.dispatch_bf16_gemm(A, B, C, variant=variant)
    torch.cuda.synchronize()
    _check_guards(buf, a_bits.shape[0], b_bits.shape[0])
    return C.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _fp8_codes(rng, rows, K):
    return F.quantize_e4m3_per_tensor(rng.standard_normal((rows, K)).astype(np.float32))


@pytest.mark.parametrize("shape", SHAPES)
def test_fp8_skinny_matches_oracle(hk, shape):
    M, N, K = shape
    print(f"fp8 skinny shape={shape}", flush=True)
    rng = np.random.default_rng(77 + M + N + K)
    (a, sa), (b, sb) = _fp8_codes(rng, M, K), _fp8_codes(rng, N, K)
    out = F.bf16_to_f32(_fp8(hk, a, b, float(sa), float(sb), 8))
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.fp8_gemm(a, b, sa, sb)) <= 5e-3


@pytest.mark.parametrize("shape", SHAPES)
def test_bf16_skinny_matches_oracle(hk, shape):
    M, N, K = shape
    K = max(8, K // 2)   # the same row lengths in bytes; K % 8 == 0
    print(f"bf16 skinny shape={(M, N, K)}", flush=True)
    rng = np.random.default_rng(78 + M + N + K)
    a = F.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    b = F.bf16_round(rng.standard_normal((N, K)).astype(np.float32))
    out = F.bf16_to_f32(_bf16(hk, a, b, 6))
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.bf16_gemm(a, b)) <= 5e-3


@pytest.mark.parametrize("shape", [(16, 96, 1024), (40, 100, 400), (64, 256, 2064)])
def test_skinny_small_integers_exact(hk, shape):
    """Operands in {-2..2}: all products and partial sums are exact in fp32, so the result does not
    depend on the order of the waves' partial sums and must equal the integer matmul."""
    M, N, K = shape
    rng = np.random.default_rng(11 + M)
    ai, bi = rng.integers(-2, 3, size=(M, K)), rng.integers(-2, 3, size=(N, K))
    expect = (ai @ bi.T).astype(np.float32)
    out = _fp8(hk, F.e4m3_encode(ai.astype(np.float32)), F.e4m3_encode(bi.astype(np.float32)), 0.5, 4.0, 8)
    assert np.array_equal(out, F.bf16_round(expect * np.float32(2.0)))
    out = _bf16(hk, F.bf16_round(ai.astype(np.float32)), F.bf16_round(bi.astype(np.float32)), 6)
    assert np.array_equal(out, F.bf16_round(expect))


def test_skinny_identity_is_bit_exact(hk):
    """A = the first 64 rows of I: C = bf16(B[:, :64])^T exactly; every e4m3 value is a bf16 value."""
    K = 384
    rng = np.random.default_rng(3)
    a = np.zeros((64, K), dtype=np.uint8)
    a[np.arange(64), np.arange(64)] = 0x38  # 1.0
    b = rng.integers(0, 256, size=(200, K), dtype=np.uint8)
    b[(b & 0x7F) == 0x7F] = 0x00  # no NaN
    out = _fp8(hk, a, b, 1.0, 1.0, 8)
    expect = F.bf16_round(F.e4m3_decode(b)[:, :64].T)
    assert np.array_equal(F.bf16_to_f32(out), F.bf16_to_f32(expect))


def test_skinny_is_what_the_entry_points_pick_for_decode_shapes(hk):
    """hk_fp8_gemm / hk_bf16_gemm, with and without a workspace, give the skinny kernel's bits at
    M = 16, N = 1024, K = 8192 and the 64x64-tile kernel's at M = 128 (sums in another order: the bits of
    the other kernel differ somewhere); two runs give the same bits."""
    rng = np.random.default_rng(5)
    N, K = 1024, 8192
    for M, fp8_variant, bf16_variant in ((16, 8, 6), (128, 6, 3)):
        (a, sa), (b, sb) = _fp8_codes(rng, M, K), _fp8_codes(rng, N, K)
        forced = _fp8(hk, a, b, float(sa), float(sb), fp8_variant)
        assert np.array_equal(forced, _fp8(hk, a, b, float(sa), float(sb), fp8_variant))
        assert np.array_equal(forced, _fp8(hk, a, b, float(sa), float(sb), -1))
        other = _fp8(hk, a, b, float(sa), float(sb), 6 if fp8_variant == 8 else 5)
        assert G.rel_fro_error(F.bf16_to_f32(other), F.bf16_to_f32(forced)) <= 5e-3
        if M == 16:
            A = torch.from_numpy(a).to(DEV).view(torch.float8_e4m3fn)
            B = torch.from_numpy(b).to(DEV).view(torch.float8_e4m3fn)
            C = torch.zeros((M, N), dtype=torch.bfloat16, device=DEV)
            need = hk.tk_kernel.fp8_gemm_workspace_bytes(M, N, K)
            ws = torch.full((max(need, 16),), 0xFF, dtype=torch.uint8, device=DEV)
            hk.tk_kernel.dispatch_fp8_gemm(A, B, C, float(sa), float(sb), workspace=ws)
            torch.cuda.synchronize()
            assert np.array_equal(C.view(torch.int16).cpu().numpy().view(np.uint16), forced)
            assert bool((ws == 0xFF).all()), "the skinny kernel leaves the workspace alone"
        ab = F.bf16_round(rng.standard_normal((M, K // 2)).astype(np.float32))
        bb = F.bf16_round(rng.standard_normal((N, K // 2)).astype(np.float32))
        assert np.array_equal(_bf16(hk, ab, bb, bf16_variant), _bf16(hk, ab, bb, -1))


def test_skinny_refuses_more_than_64_rows(hk):
    rng = np.random.default_rng(7)
    (a, _), (b, _) = _fp8_codes(rng, 65, 256), _fp8_codes(rng, 64, 256)
    with pytest.raises(RuntimeError):
        _fp8(hk, a, b, 1.0, 1.0, 8)
    with pytest.raises(RuntimeError):
        _bf16(hk, F.bf16_round(np.ones((65, 64), np.float32)), F.bf16_round(np.ones((64, 64), np.float32)), 6)


# ---------------------------------------------------------------------------------------------- MXFP4
def _rand_mx(rng, rows, K):
    x = rng.standard_normal((rows, K)).astype(np.float32)
    x *= np.exp2(rng.integers(-6, 7, size=(rows, K // 32))).repeat(32, axis=1).astype(np.float32)   # scales that matter
    return F.quantize_mxfp4(x)


def _mxfp4(hk, a, sa, b, sb, variant, misalign=0, pitches=None, workspace=False):
    """Every operand array inside a pool of 0xFF bytes (a scale byte fetched in front of or behind an array
    would be the e8m0 NaN), the scale arrays `misalign` bytes off a 16-byte boundary."""
    views, pools = [], []
    for arr, mis in ((a, 0), (sa, misalign), (b, 0), (sb, misalign)):
        pool = torch.full((16 + mis + arr.size + 272,), 0xFF, dtype=torch.uint8, device=DEV)
        view = pool[16 + mis:16 + mis + arr.size].view(arr.shape)
        view.copy_(torch.from_numpy(arr).to(DEV))
        pools.append(pool)
        views.append(view)
    A, SA, B, SB = views
    C, buf = _guarded_c(a.shape[0], b.shape[0])
    ws = None
    if workspace:
        ws = torch.full((max(16, hk.tk_kernel.mxfp4_gemm_workspace_bytes(a.shape[0], b.shape[0], a.shape[1] * 2)),),
                        0xFF, dtype=torch.uint8, device=DEV)
    hk.tk_kernel.dispatch_mxfp4_gemm(A, SA, B, SB, C, variant=variant, workspace=ws)
    torch.cuda.synchronize()
    _check_guards(buf, a.shape[0], b.shape[0])
    return C.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


# K / 32 scale bytes per row: a single one, every remainder modulo 4 (the last K-step's scales are then fetched
# byte by byte), more than one 128-byte scale tile per row (K > 4096), waves that start inside a scale tile
MX_SHAPES = [(1, 32, 32), (16, 32, 256), (16, 64, 4096), (7, 100, 32 * 17), (16, 101, 2880), (17, 96, 2880),
             (32, 200, 8192), (32, 72, 32 * 263), (3, 31, 96), (16, 2880, 2880), (24, 520, 32 * 47), (16, 256, 32 * 530),
             (33, 32, 256), (64, 101, 2880), (48, 200, 8192), (64, 72, 32 * 263)]


@pytest.mark.parametrize("shape", MX_SHAPES)
def test_mxfp4_skinny_matches_oracle(hk, shape):
    M, N, K = shape
    print(f"mxfp4 skinny shape={shape}", flush=True)
    rng = np.random.default_rng(79 + M + N + K)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    ref = G.mxfp4_gemm(a, sa, b, sb)
    first = None
    for mis in (0, 1, 3):
        bits = _mxfp4(hk, a, sa, b, sb, 6, mis)
        out = F.bf16_to_f32(bits)
        assert np.isfinite(out).all(), mis
        assert G.rel_fro_error(out, ref) <= 5e-3, mis
        first = bits if first is None else first
        assert np.array_equal(bits, first), mis


def test_mxfp4_skinny_exact_and_scale_positions(hk):
    """Elements in {-2..2} with scales 2^-2 .. 2^2 that differ from block to block: every partial sum is exact in
    fp32 (below 2^18 in units of 2^-4), so the result is the exact value rounded once, whatever the order of the
    waves' sums; a scale applied to the wrong 32-block or row would show."""
    rng = np.random.default_rng(21)
    codes = np.array([0, 2, 4, 10, 12], dtype=np.uint8)  # e2m1 codes of 0, 1, 2, -1, -2

    def make(rows, K):
        c = codes[rng.integers(0, 5, size=(rows, K))]
        return ((c[:, 0::2] | (c[:, 1::2] << 4)).astype(np.uint8),
                rng.integers(125, 130, size=(rows, K // 32)).astype(np.uint8))

    for M, N, K in ((16, 96, 1024), (30, 100, 32 * 19), (9, 64, 32 * 270), (64, 40, 32 * 21)):
        (a, sa), (b, sb) = make(M, K), make(N, K)
        exact = F.dequantize_mxfp4(a, sa).astype(np.float64) @ F.dequantize_mxfp4(b, sb).astype(np.float64).T
        assert np.array_equal(_mxfp4(hk, a, sa, b, sb, 6, 1), F.bf16_round(exact.astype(np.float32)))


def test_mxfp4_skinny_is_what_the_entry_points_pick_and_takes_padded_rows(hk):
    """hk_mxfp4_gemm with and without a workspace gives the skinny kernel's bits at M = 16, N = 1024, K = 8192
    and leaves the workspace alone; scale rows padded to a pitch give the same bits as dense rows."""
    rng = np.random.default_rng(6)
    M, N, K = 16, 1024, 8192
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    forced = _mxfp4(hk, a, sa, b, sb, 6)
    assert np.array_equal(forced, _mxfp4(hk, a, sa, b, sb, -1))
    assert np.array_equal(forced, _mxfp4(hk, a, sa, b, sb, -1, workspace=True))
    pad = lambda s, pitch: np.concatenate([s, rng.integers(0, 255, size=(s.shape[0], pitch - s.shape[1]), dtype=np.uint8)], axis=1)
    assert np.array_equal(forced, _mxfp4(hk, a, pad(sa, 264), b, pad(sb, 259), -1))
    (a2, sa2), (b2, sb2) = _rand_mx(rng, 65, 256), _rand_mx(rng, 64, 256)
    with pytest.raises(RuntimeError):
        _mxfp4(hk, a2, sa2, b2, sb2, 6)


def test_skinny_drawn_shapes_match_oracle(hk):
    """36 seeded random shapes (M <= 64, N < 400, K up to 150 K-steps with every kind of tail), twelve per
    format, each against the oracle; MXFP4 scale arrays at a drawn misalignment."""
    rng = np.random.default_rng(2024)
    for it in range(36):
        fmt = ("fp8", "bf16", "mxfp4")[it % 3]
        M, N = int(rng.integers(1, 65)), int(rng.integers(1, 400))
        if fmt == "fp8":
            K = 16 * int(rng.integers(1, 1200))
            (a, sa), (b, sb) = _fp8_codes(rng, M, K), _fp8_codes(rng, N, K)
            out, ref = _fp8(hk, a, b, float(sa), float(sb), 8), G.fp8_gemm(a, b, sa, sb)
        elif fmt == "bf16":
            K = 8 * int(rng.integers(1, 1200))
            a = F.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
            b = F.bf16_round(rng.standard_normal((N, K)).astype(np.float32))
            out, ref = _bf16(hk, a, b, 6), G.bf16_gemm(a, b)
        else:
            K = 32 * int(rng.integers(1, 1200))
            (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
            out, ref = _mxfp4(hk, a, sa, b, sb, 6, int(rng.integers(0, 4))), G.mxfp4_gemm(a, sa, b, sb)
        print(f"skinny drawn {fmt} M={M} N={N} K={K}", flush=True)
        out = F.bf16_to_f32(out)
        assert np.isfinite(out).all(), (fmt, M, N, K)
        assert G.rel_fro_error(out, ref) <= 5e-3, (fmt, M, N, K)
