"""CPU oracle, part 1: number formats and quantizers (numpy, bit level).

TEST INFRASTRUCTURE ONLY. Nothing under oracle/ is imported by the shipped
package; it is the checker used by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.

What each function restates and what pins it:

* e4m3 (OCP e4m3fn: bias 7, max 448, no inf, NaN = 0x7F/0xFF) is the
  reference's ``fp8e4m3`` on CDNA4 (include/common/base_types.cuh:40-52); its
  float->fp8 conversion is HIP's saturating round-to-nearest-even constructor
  (include/common/base_types.cuh:348-379). Pinned by the closed form of the
  format, by an exhaustive 256-code comparison with torch's float8_e4m3fn
  decode, and by comparison with torch's RNE cast on inputs within +-448
  (tests/test_oracle_formats.py).
* bf16 round-to-nearest-even restates the packed convertor
  (include/common/base_types.cuh:297-305); pinned against torch's cast.
* e2m1 / e8m0 / MX block quantization, the 1x128 and 128x128 fp32 block scales and
  the per-tensor amax/448 scale have no counterpart in the reference ("parity
  unpinned" with respect to it); they follow the OCP Microscaling v1.0 rules and
  are pinned by closed forms, committed decode tables (tests/golden) and brute
  force on small blocks.
"""
from __future__ import annotations

import numpy as np

E4M3_MAX = 448.0
E2M1_MAX = 6.0
E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


# ----------------------------------------------------------------------------- e4m3
def e4m3_decode_table() -> np.ndarray:
    """float32 value of each of the 256 e4m3fn codes (NaN for 0x7F and 0xFF)."""
    out = np.empty(256, dtype=np.float32)
    for c in range(256):
        sign = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 7
        if e == 0xF and m == 7:
            v = float("nan")
        elif e == 0:
            v = sign * m * 2.0 ** -9
        else:
            v = sign * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out[c] = v
    return out


_E4M3_TABLE = e4m3_decode_table()


def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    return _E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """float -> e4m3fn code, round to nearest even, saturating to +-448 (inf too);
    NaN -> 0x7F with the sign bit kept."""
    x = np.asarray(x, dtype=np.float32)
    a = np.abs(x).astype(np.float64)
    sign = (np.signbit(x).astype(np.uint8)) << 7
    nan = np.isnan(x)
    a = np.where(nan, 0.0, a)
    a = np.minimum(a, E4M3_MAX)
    # subnormal range (< 2^-6): units of 2^-9; rint is round-half-even and a*512 is exact
    sub = np.rint(a * 512.0)
    mant, exp = np.frexp(a)  # a = mant * 2^exp, mant in [0.5, 1)
    e = exp - 1  # a = (2*mant) * 2^e, 2*mant in [1, 2)
    q = np.rint((2.0 * mant - 1.0) * 8.0)
    carry = q == 8
    e = np.where(carry, e + 1, e)
    q = np.where(carry, 0, q)
    normal = ((e + 7).astype(np.int64) << 3) | q.astype(np.int64)
    code = np.where(a < 2.0 ** -6, sub.astype(np.int64), normal)
    code = np.minimum(code, 0x7E)
    code = np.where(nan, 0x7F, code)
    return (code.astype(np.uint8) | sign).astype(np.uint8)


def quantize_e4m3_per_tensor(x: np.ndarray):
    """Per-tensor scale s = amax/448 (fp32); codes = e4m3(x / s). amax == 0 -> s = 1."""
    x = np.asarray(x, dtype=np.float32)
    amax = np.float32(np.max(np.abs(x))) if x.size else np.float32(0)
    s = np.float32(amax / np.float32(E4M3_MAX)) if amax > 0 else np.float32(1.0)
    return e4m3_encode((x / s).astype(np.float32)), s


def quantize_e4m3_blocks(x: np.ndarray, block_rows: int, block_cols: int):
    """fp32 block scales s = amax(block)/448 over block_rows x block_cols blocks of a 2-D
    array (1x128 for activations, 128x128 for weights). Returns (codes, scales)."""
    x = np.asarray(x, dtype=np.float32)
    R, C = x.shape
    nbr, nbc = -(-R // block_rows), -(-C // block_cols)
    pad = np.zeros((nbr * block_rows, nbc * block_cols), dtype=np.float32)
    pad[:R, :C] = x
    blk = pad.reshape(nbr, block_rows, nbc, block_cols)
    amax = np.abs(blk).max(axis=(1, 3)).astype(np.float32)
    s = np.where(amax > 0, amax / np.float32(E4M3_MAX), np.float32(1.0)).astype(np.float32)
    q = e4m3_encode((blk / s[:, None, :, None]).astype(np.float32))
    q = q.reshape(nbr * block_rows, nbc * block_cols)[:R, :C]
    return np.ascontiguousarray(q), s


def dequantize_e4m3_blocks(q: np.ndarray, s: np.ndarray, block_rows: int, block_cols: int):
    v = e4m3_decode(q)
    R, C = v.shape
    if R % block_rows == 0 and C % block_cols == 0:   # whole blocks: broadcast instead of repeating the scales
        blk = v.reshape(R // block_rows, block_rows, C // block_cols, block_cols)
        blk *= np.asarray(s, dtype=np.float32)[:, None, :, None]   # v is a fresh array (table lookup)
        return v
    sr = np.repeat(np.repeat(s, block_rows, axis=0)[:R], block_cols, axis=1)[:, :C]
    return (v * sr).astype(np.float32)


# ----------------------------------------------------------------------------- bf16
def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bits (uint16), round to nearest even; NaN stays NaN."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = np.isnan(np.asarray(x, dtype=np.float32))
    rounded = np.where(nan, (u >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------------- e2m1 / e8m0 / MX
def e2m1_decode_table() -> np.ndarray:
    """float32 value of each of the 16 e2m1 codes (bit 3 = sign)."""
    return np.concatenate([E2M1_VALUES, -E2M1_VALUES]).astype(np.float32)


def e2m1_encode(x: np.ndarray) -> np.ndarray:
    """float -> 4-bit e2m1 code, round to nearest, ties to the even code, saturating at 6."""
    x = np.asarray(x, dtype=np.float32)
    a = np.minimum(np.abs(x).astype(np.float64), E2M1_MAX)
    a = np.where(np.isnan(a), E2M1_MAX, a)
    # representable magnitudes have spacing 0.5 below 2, 1 in [2,4), 2 in [4,6]
    code = np.where(
        a < 2.0, np.rint(a * 2.0),  # codes 0..4 (4 = 2.0)
        np.where(a < 4.0, 4 + np.rint(a - 2.0),  # 2->4, 3->5, 4->6 ; rint ties to even
                 6 + np.rint((a - 4.0) / 2.0)))  # 4->6, 6->7
    # rint ties-to-even above acts on the scaled value; the even *code* coincides with the
    # even scaled integer in each segment (segment starts 0, 4 and 6 are even codes).
    code = code.astype(np.uint8)
    return (code | (np.signbit(x).astype(np.uint8) << 3)).astype(np.uint8)


def e8m0_decode(b: np.ndarray) -> np.ndarray:
    """2^(b-127) as float32 (b = 255 is NaN in the format and never produced here)."""
    return np.ldexp(np.float32(1.0), np.asarray(b, dtype=np.int32) - 127).astype(np.float32)


def quantize_mxfp4(x: np.ndarray):
    """OCP MX quantization along the last axis in blocks of 32.

    Shared exponent e = floor(log2(amax)) - 2 (2 = emax of e2m1), clamped to [-127, 127]
    and stored as e + 127; elements = e2m1(x / 2^e), saturating. amax == 0 -> byte 127.
    Returns (packed uint8 [..., K/2] with the even K index in the low nibble,
             scales uint8 [..., K/32])."""
    x = np.asarray(x, dtype=np.float32)
    K = x.shape[-1]
    assert K % 32 == 0
    blk = x.reshape(*x.shape[:-1], K // 32, 32)
    amax = np.abs(blk).max(axis=-1)
    _, ex = np.frexp(amax.astype(np.float64))  # amax = m * 2^ex, m in [0.5,1) -> floor(log2) = ex-1
    e = np.clip(ex - 1 - 2, -127, 127)
    e = np.where(amax > 0, e, 0).astype(np.int32)
    scaled = blk.astype(np.float64) * np.ldexp(1.0, -e)[..., None]
    codes = e2m1_encode(scaled.astype(np.float32)).reshape(*x.shape[:-1], K)
    packed = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
    return packed, (e + 127).astype(np.uint8)


def quantize_mxfp8(x: np.ndarray):
    """OCP MX quantization along the last axis in blocks of 32 with e4m3 elements (MXFP8).

    Shared exponent e = floor(log2(amax)) - 8 (8 = emax of e4m3: 448 = 1.75 * 2^8), clamped to
    [-127, 127] and stored as e + 127; elements = e4m3(x / 2^e), round to nearest even,
    saturating at +-448 (a block maximum in [1.75, 2) * 2^(e+8) saturates). amax == 0 -> byte 127.
    Returns (codes uint8 [..., K], scales uint8 [..., K/32]). No counterpart in the reference
    repository; the rule is the one of the OCP Microscaling Formats specification v1.0."""
    x = np.asarray(x, dtype=np.float32)
    K = x.shape[-1]
    assert K % 32 == 0
    blk = x.reshape(*x.shape[:-1], K // 32, 32)
    amax = np.abs(blk).max(axis=-1)
    _, ex = np.frexp(amax.astype(np.float64))
    e = np.clip(ex - 1 - 8, -127, 127)
    e = np.where(amax > 0, e, 0).astype(np.int32)
    scaled = blk.astype(np.float64) * np.ldexp(1.0, -e)[..., None]
    codes = e4m3_encode(scaled.astype(np.float32)).reshape(*x.shape[:-1], K)
    return codes, (e + 127).astype(np.uint8)


def dequantize_mxfp8(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    v = e4m3_decode(codes)
    s = np.repeat(e8m0_decode(scales), 32, axis=-1)
    return (v * s).astype(np.float32)


def dequantize_mxfp4(packed: np.ndarray, scales: np.ndarray) -> np.ndarray:
    packed = np.asarray(packed, dtype=np.uint8)
    tbl = e2m1_decode_table()
    lo, hi = tbl[packed & 0xF], tbl[packed >> 4]
    v = np.stack([lo, hi], axis=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)
    s = np.repeat(e8m0_decode(scales), 32, axis=-1)
    return (v * s).astype(np.float32)


# ------------------------------------------------------------------ reference inputs
def reference_random_init(M: int, N: int, K: int):
    """The reference executable's input generator, restated from
    kernels/gemm/fp8fp32/profile_utils.cpp:35-45: std::mt19937(42), one
    uniform_real_distribution<float>(-1, 1) draw per element, A (M*K) first then B (N*K),
    each converted to e4m3 (saturating RNE). libstdc++ draws one 32-bit word per float:
    u = float(word) / 2^32 (forced below 1), value = -1 + 2u, all in fp32.
    Returns e4m3 codes A [M,K], B [N,K]."""
    rs = np.random.RandomState(42)  # init_genrand(42), the same seeding as std::mt19937(42)
    words = rs.randint(0, 2 ** 32, size=M * K + N * K, dtype=np.uint64).astype(np.uint32)
    u = words.astype(np.float32) / np.float32(4294967296.0)
    u = np.where(u >= np.float32(1.0), np.nextafter(np.float32(1.0), np.float32(0.0)), u)
    v = (np.float32(2.0) * u + np.float32(-1.0)).astype(np.float32)
    codes = e4m3_encode(v)
    return codes[: M * K].reshape(M, K), codes[M * K:].reshape(N, K)
