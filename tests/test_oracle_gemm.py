"""Pins of the GEMM oracle (oracle/gemm.py) that involve no GPU and do not restate its formula.

The GPU tests judge the kernels against oracle.gemm, so the oracle itself is tied down here by
things that are known independently of it: closed-form answers (identity, powers of two), an
integer matmul, a scalar triple loop in float64 over element values decoded by hand, torch's CPU
cast + matmul, and hand-computed error metrics. Each case is chosen so that a plausible mistake
(a missing transpose, a scale on the wrong operand or squared, a nibble or scale-block index
off by one, a norm without the square root) fails it.

Convention restated: C = A . B^T with both operands K-contiguous
(include/ops/warp/register/tile/mma.cuh:382-422), error metric of
kernels/attn/gqa/test_python.py:46-57.
"""
import numpy as np
import torch

from oracle import formats as F
from oracle import gemm as G


# ------------------------------------------------------------------ hand decoders (no oracle code)
def _e4m3_value(code: int) -> float:
    """OCP e4m3fn value of one code, written from the format definition."""
    s = -1.0 if code & 0x80 else 1.0
    e, m = (code >> 3) & 0xF, code & 7
    if e == 0:
        return s * m / 512.0
    return s * (1.0 + m / 8.0) * 2.0 ** (e - 7)


_E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]


def _mx_value(packed_row, scale_row, k: int) -> float:
    """Element k of an MXFP4 row: nibble k % 2 of byte k // 2 (low nibble = even k), times
    2^(scale byte of block k // 32 - 127)."""
    byte = int(packed_row[k // 2])
    nib = (byte >> 4) if (k & 1) else (byte & 0xF)
    v = _E2M1[nib & 7] * (-1.0 if nib & 8 else 1.0)
    return v * 2.0 ** (int(scale_row[k // 32]) - 127)


def _codes(rng, rows, K):
    c = rng.integers(0, 256, size=(rows, K), dtype=np.uint8)
    c[(c & 0x7F) == 0x7F] = 0x38  # no NaN codes
    return c


# ------------------------------------------------------------------------------------ FP8
def test_fp8_gemm_identity_and_power_of_two_known_answers():
    """A = I: C = B^T exactly (so the operand that is transposed is B, and C is [M, N] with N
    taken from B's rows); a power-of-two multiple of I and power-of-two scales scale it exactly."""
    rng = np.random.default_rng(0)
    K, N = 48, 20
    eye = np.zeros((K, K), np.uint8)
    eye[np.arange(K), np.arange(K)] = 0x38                    # 1.0
    b = _codes(rng, N, K)
    bt = np.array([[_e4m3_value(int(b[n, k])) for n in range(N)] for k in range(K)], np.float32)
    out = G.fp8_gemm(eye, b)
    assert out.shape == (K, N) and out.dtype == np.float32
    assert np.array_equal(out, bt)
    four = np.zeros_like(eye)
    four[np.arange(K), np.arange(K)] = 0x48                   # 4.0
    assert np.array_equal(G.fp8_gemm(four, b, 0.5, 8.0), bt * np.float32(16.0))
    # the two scales multiply (not add, not square one of them)
    assert np.array_equal(G.fp8_gemm(eye, b, 2.0, 1.0), G.fp8_gemm(eye, b, 1.0, 2.0))
    assert np.array_equal(G.fp8_gemm(eye, b, 4.0, 1.0), G.fp8_gemm(eye, b, 2.0, 2.0))


def test_fp8_gemm_small_integers_equal_the_integer_matmul():
    rng = np.random.default_rng(1)
    M, N, K = 37, 23, 64
    ai = rng.integers(-4, 5, size=(M, K))
    bi = rng.integers(-4, 5, size=(N, K))
    enc = {0: 0x00, 1: 0x38, 2: 0x40, 3: 0x44, 4: 0x48}       # e4m3 codes of 0, 1, 2, 3, 4
    to_code = np.vectorize(lambda v: enc[abs(int(v))] | (0x80 if v < 0 else 0), otypes=[np.uint8])
    out = G.fp8_gemm(to_code(ai), to_code(bi), 0.5, 4.0)
    assert np.array_equal(out, (ai @ bi.T).astype(np.float32) * np.float32(2.0))
    assert np.array_equal(G.fp8_gemm_bf16(to_code(ai), to_code(bi)),
                          torch.from_numpy((ai @ bi.T).astype(np.float32)).to(torch.bfloat16)
                          .view(torch.int16).numpy().view(np.uint16))


def test_fp8_gemm_float64_triple_loop_non_square_with_scales():
    """Scalar loops over hand-decoded values; M, N and K all differ, scales are not powers of two."""
    rng = np.random.default_rng(2)
    M, N, K = 7, 13, 64
    a, b = _codes(rng, M, K), _codes(rng, N, K)
    sa, sb = 0.37, 1.9
    want = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            acc = 0.0
            for k in range(K):
                acc += _e4m3_value(int(a[m, k])) * _e4m3_value(int(b[n, k]))
            want[m, n] = acc * float(np.float32(sa) * np.float32(sb))
    out = G.fp8_gemm(a, b, sa, sb)
    assert out.shape == (M, N)
    # random e4m3 codes span 2^-9 .. 448: compare against the size of the terms, not of the sum
    mag = np.abs(F.e4m3_decode(a)).astype(np.float64) @ np.abs(F.e4m3_decode(b)).astype(np.float64).T
    assert np.all(np.abs(out - want) <= 1e-5 * mag * sa * sb + 1e-30)
    assert np.abs(want).max() > 1.0  # not vacuous


def test_fp8_gemm_256_cubed_against_torch_cpu_dequantize_matmul():
    """The CPU-runnable configuration: N(0,1) inputs, per-tensor amax/448 scales, torch's own
    e4m3 decode and matmul as the library routine."""
    g = torch.Generator().manual_seed(0)
    n = 256
    A, B = torch.randn(n, n, generator=g), torch.randn(n, n, generator=g)
    sa, sb = A.abs().max() / 448.0, B.abs().max() / 448.0
    Aq = (A / sa).clamp(-448, 448).to(torch.float8_e4m3fn)
    Bq = (B / sb).clamp(-448, 448).to(torch.float8_e4m3fn)
    want = ((Aq.double() * sa.double()) @ (Bq.double() * sb.double()).t()).numpy()
    out = G.fp8_gemm(Aq.view(torch.uint8).numpy(), Bq.view(torch.uint8).numpy(), float(sa), float(sb))
    assert G.rel_fro_error(out, want) < 1e-6
    # and the quantized product is close to the unquantized one (the scales are on the right side)
    assert G.rel_fro_error(out, (A.double() @ B.double().t()).numpy()) < 0.06
    bits = G.fp8_gemm_bf16(Aq.view(torch.uint8).numpy(), Bq.view(torch.uint8).numpy(), float(sa), float(sb))
    tb = torch.from_numpy(out).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bits, tb)


# ------------------------------------------------------------------------------------ MXFP4
def test_mxfp4_gemm_known_answers_nibble_order_and_scale_blocks():
    """Rows with a single nonzero element: C[m, n] is one product, so the nibble order (low = even
    k) and the block a scale byte belongs to are checked one position at a time."""
    K = 96
    M = N = K
    a = np.zeros((M, K // 2), np.uint8)
    sa = np.full((M, K // 32), 127, np.uint8)
    for m in range(M):                                        # row m: 1.0 at k = m, block scale 2^(m // 32)
        a[m, m // 2] = 0x02 << (4 * (m & 1))
        sa[m, m // 32] = 127 + 1 + m // 32
    rng = np.random.default_rng(3)
    b = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    sb = rng.integers(120, 134, size=(N, K // 32)).astype(np.uint8)
    out = G.mxfp4_gemm(a, sa, b, sb)
    want = np.array([[2.0 ** (1 + m // 32) * _mx_value(b[n], sb[n], m) for n in range(N)] for m in range(M)])
    assert np.array_equal(out, want.astype(np.float32))


def test_mxfp4_gemm_float64_triple_loop_non_square():
    rng = np.random.default_rng(4)
    M, N, K = 5, 9, 64
    a = rng.integers(0, 256, size=(M, K // 2), dtype=np.uint8)
    b = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    sa = rng.integers(118, 136, size=(M, K // 32)).astype(np.uint8)
    sb = rng.integers(118, 136, size=(N, K // 32)).astype(np.uint8)
    want = np.zeros((M, N))
    for m in range(M):
        for n in range(N):
            for k in range(K):
                want[m, n] += _mx_value(a[m], sa[m], k) * _mx_value(b[n], sb[n], k)
    out = G.mxfp4_gemm(a, sa, b, sb)
    assert out.shape == (M, N)
    mag = np.abs(F.dequantize_mxfp4(a, sa)).astype(np.float64) @ np.abs(F.dequantize_mxfp4(b, sb)).astype(np.float64).T
    assert np.all(np.abs(out - want) <= 1e-5 * mag)
    assert np.abs(want).max() > 1.0


def test_mxfp4_gemm_quantized_product_tracks_the_fp32_product():
    """randn quantized along K to MXFP4 (OCP rule): the product of the quantized operands stays
    within the format's error of the fp64 product; a wrong scale exponent or block would not."""
    rng = np.random.default_rng(5)
    M, N, K = 64, 48, 512
    x = rng.standard_normal((M, K)).astype(np.float32) * np.exp2(rng.integers(-8, 9, size=(M, 1))).astype(np.float32)
    y = rng.standard_normal((N, K)).astype(np.float32)
    (a, sa), (b, sb) = F.quantize_mxfp4(x), F.quantize_mxfp4(y)
    out = G.mxfp4_gemm(a, sa, b, sb)
    assert G.rel_fro_error(out, x.astype(np.float64) @ y.astype(np.float64).T) < 0.2
    # block scales are powers of two: doubling one operand's scale bytes doubles the result exactly
    assert np.array_equal(G.mxfp4_gemm(a, (sa + 1).astype(np.uint8), b, sb), out * np.float32(2.0))


# ------------------------------------------------------------------------------------ BF16
def test_bf16_gemm_against_torch():
    g = torch.Generator().manual_seed(1)
    A = torch.randn(33, 80, generator=g).to(torch.bfloat16)
    B = torch.randn(17, 80, generator=g).to(torch.bfloat16)
    out = G.bf16_gemm(A.view(torch.int16).numpy().view(np.uint16), B.view(torch.int16).numpy().view(np.uint16))
    assert out.shape == (33, 17)
    assert G.rel_fro_error(out, (A.double() @ B.double().t()).numpy()) < 1e-6


# ------------------------------------------------------------------------------------ metrics
def test_rel_fro_error_and_error_stats_on_hand_computed_pairs():
    ref = np.array([[3.0, 4.0], [0.0, 0.0]])                  # ||ref|| = 5
    out = np.array([[3.0, 4.0], [0.0, 1.0]])                  # ||out - ref|| = 1
    assert G.rel_fro_error(out, ref) == 0.2
    assert G.rel_fro_error(ref, ref) == 0.0
    assert G.rel_fro_error(2 * ref, ref) == 1.0               # not squared: 2x off is 100 %
    assert G.rel_fro_error(out, np.zeros_like(ref)) == np.sqrt(26.0)   # zero reference: absolute norm
    # order of the arguments matters (the denominator is the reference's norm)
    assert G.rel_fro_error(ref, 2 * ref) == 0.5
    st = G.error_stats(np.array([1.0, 2.0, 4.5]), np.array([1.0, 2.2, 4.0]))
    assert st["max_abs"] == 0.5 and abs(st["mean_abs"] - 0.7 / 3) < 1e-15
    assert st["count_gt_1pct"] == 2
    assert abs(st["rel_fro"] - np.sqrt(0.29) / np.sqrt(1 + 4.84 + 16)) < 1e-15
