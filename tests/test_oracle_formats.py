"""Pin the oracle's number formats (CPU only): closed forms, exhaustive tables, library casts."""
import json
import os

import numpy as np
import torch

from oracle import formats as F

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_e4m3_decode_exhaustive_vs_torch_and_golden():
    tbl = F.e4m3_decode_table()
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    nan = np.isnan(tbl)
    assert list(np.nonzero(nan)[0]) == [0x7F, 0xFF]
    assert np.array_equal(np.isnan(tt), nan)
    assert np.array_equal(tbl[~nan], tt[~nan])
    assert tbl[0x7E] == 448.0 and tbl[0x08] == 2.0 ** -6 and tbl[0x01] == 2.0 ** -9 and tbl[0x38] == 1.0
    gold = json.load(open(os.path.join(GOLDEN, "format_tables.json")))
    assert [None if np.isnan(v) else float(v) for v in tbl] == gold["e4m3_decode"]


def test_e4m3_encode_round_trip_and_rne_vs_torch():
    codes = np.arange(256, dtype=np.uint8)
    vals = F.e4m3_decode(codes)
    ok = ~np.isnan(vals)
    rt = F.e4m3_encode(vals[ok])
    # -0.0 keeps its sign bit; every finite code round-trips
    assert np.array_equal(rt, codes[ok])
    # every fp16 value inside the range: compare with torch's RNE cast
    h = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    h = h[np.isfinite(h) & (np.abs(h) <= 448.0)]
    mine = F.e4m3_encode(h)
    ref = torch.from_numpy(h).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mine, ref)


def test_e4m3_encode_ties_saturation_nan():
    x = np.array([1.0625, 1.1875, 17.0, 19.0, 2.0 ** -10, 3 * 2.0 ** -10, 448.0, 449.0, 464.0, 1e9, -1e9,
                  np.inf, -np.inf], dtype=np.float32)
    exp = [1.0, 1.25, 16.0, 20.0, 0.0, 2.0 ** -8, 448.0, 448.0, 448.0, 448.0, -448.0, 448.0, -448.0]
    assert list(F.e4m3_decode(F.e4m3_encode(x))) == exp
    assert F.e4m3_encode(np.array([np.nan], dtype=np.float32))[0] & 0x7F == 0x7F


def test_per_tensor_scale_closed_form():
    x = np.array([[0.5, -3.0], [1.5, 0.25]], dtype=np.float32)
    q, s = F.quantize_e4m3_per_tensor(x)
    assert s == np.float32(3.0) / np.float32(448.0)
    assert F.e4m3_decode(q)[0, 1] == -448.0
    z, sz = F.quantize_e4m3_per_tensor(np.zeros((2, 2), np.float32))
    assert sz == 1.0 and not z.any()


def test_bf16_round_vs_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 1e3,
                        np.array([1.00390625, 1.01171875, 0.0, -0.0, 3.3895314e38], dtype=np.float32)])
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(F.bf16_round(x), ref)
    assert np.array_equal(F.bf16_to_f32(ref), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


def test_e2m1_table_and_encode_brute_force():
    tbl = F.e2m1_decode_table()
    gold = json.load(open(os.path.join(GOLDEN, "format_tables.json")))
    assert [float(v) for v in tbl] == gold["e2m1_decode"]
    pos = tbl[:8].astype(np.float64)
    # brute force: nearest representable value, ties to the even code, saturate at 6
    xs = np.concatenate([np.linspace(0, 8, 6401), np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 100.0])])
    for x in xs:
        d = np.abs(pos - x)
        best = np.flatnonzero(d == d.min())
        want = int(best[0]) if len(best) == 1 else int([b for b in best if b % 2 == 0][0])
        got = int(F.e2m1_encode(np.array([x], dtype=np.float32))[0])
        assert got == want, (x, got, want)
        assert int(F.e2m1_encode(np.array([-x], dtype=np.float32))[0]) == (want | 8)


def test_e8m0_decode_vs_torch():
    b = np.arange(255, dtype=np.uint8)
    ref = torch.from_numpy(b).view(torch.float8_e8m0fnu).float().numpy()
    assert np.array_equal(F.e8m0_decode(b), ref)


def test_mx_quantize_rules():
    x = np.zeros((1, 64), dtype=np.float32)
    x[0, :32] = np.linspace(-6, 6, 32)      # amax 6 -> e = floor(log2 6) - 2 = 0
    x[0, 32:] = 0.0                          # amax 0 -> scale byte 127, all codes 0
    p, s = F.quantize_mxfp4(x)
    assert list(s[0]) == [127, 127]
    assert not p[0, 16:].any()
    d = F.dequantize_mxfp4(p, s)
    assert d[0, 0] == -6.0 and d[0, 31] == 6.0
    # scale is floor(log2(amax)) - 2, not round-to-nearest: amax 7.9 -> e = 0, element saturates at 6
    y = np.zeros((1, 32), dtype=np.float32); y[0, 0] = 7.9; y[0, 1] = 3.0
    p, s = F.quantize_mxfp4(y)
    assert s[0, 0] == 127 and F.dequantize_mxfp4(p, s)[0, 0] == 6.0 and F.dequantize_mxfp4(p, s)[0, 1] == 3.0
    # amax 8 -> e = 1: 8/2 = 4 exactly
    y[0, 0] = 8.0
    p, s = F.quantize_mxfp4(y)
    assert s[0, 0] == 128 and F.dequantize_mxfp4(p, s)[0, 0] == 8.0
    # packing: even k in the low nibble
    z = np.zeros((1, 32), dtype=np.float32); z[0, 0] = 1.0; z[0, 1] = -2.0; z[0, 2] = 4.0
    p, s = F.quantize_mxfp4(z)
    assert s[0, 0] == 127 and p[0, 0] == (0x2 | (0xC << 4)) and p[0, 1] == 0x6
    # tiny / huge magnitudes clamp the exponent and never emit 255
    w = np.array([[1e-45] * 32 + [3e38] * 32], dtype=np.float32)
    p, s = F.quantize_mxfp4(w)
    assert s.max() < 255


def test_mx_quantize_error_bound_random():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    p, s = F.quantize_mxfp4(x)
    d = F.dequantize_mxfp4(p, s)
    scale = np.repeat(F.e8m0_decode(s), 32, axis=1)
    # inside the unsaturated range the error is at most half the local spacing (<= 1 * scale)
    unsat = np.abs(x) <= 6 * scale
    assert np.all(np.abs(d - x)[unsat] <= 1.0 * scale[unsat] + 1e-12)


def test_mxfp8_quantize_rules_and_brute_force():
    """MXFP8 (e4m3 elements, e8m0 per 32): the shared exponent is floor(log2(amax)) - 8, elements
    round to the nearest e4m3 value (ties to the even code) and saturate at 448. Pinned by known
    answers and by a brute-force nearest-value search over the 254 finite e4m3 codes."""
    x = np.zeros((1, 96), dtype=np.float32)
    x[0, 0] = 448.0; x[0, 1] = -1.0; x[0, 2] = 2.0 ** -9            # amax 448 -> e = 0
    x[0, 32] = 500.0; x[0, 33] = 17.0                               # amax 500 -> e = 0: 500 saturates to 448
    x[0, 64] = 512.0; x[0, 65] = 1.0                                # amax 512 -> e = 1: 256 exactly
    c, s = F.quantize_mxfp8(x)
    assert list(s[0]) == [127, 127, 128]
    d = F.dequantize_mxfp8(c, s)
    assert d[0, 0] == 448.0 and d[0, 1] == -1.0 and d[0, 2] == 2.0 ** -9
    assert c[0, 0] == 0x7E and c[0, 1] == 0xB8
    assert d[0, 32] == 448.0 and d[0, 33] == 16.0                   # 17 lies between 16 and 18: tie -> even mantissa
    assert d[0, 64] == 512.0 and d[0, 65] == 1.0
    z, sz = F.quantize_mxfp8(np.zeros((2, 32), dtype=np.float32))
    assert not z.any() and np.all(sz == 127)
    # brute force: nearest finite e4m3 value of x / 2^e, ties to the even code
    rng = np.random.default_rng(8)
    y = (rng.standard_normal((16, 64)) * np.exp2(rng.integers(-20, 20, size=(16, 1)))).astype(np.float32)
    c, s = F.quantize_mxfp8(y)
    tbl = F.e4m3_decode_table().astype(np.float64)
    pos = np.array([i for i in range(0x7F)], dtype=np.int64)           # finite non-negative codes, ascending values
    vals = tbl[pos]
    amax = np.abs(y.reshape(16, 2, 32)).max(-1)
    e = np.floor(np.log2(amax)).astype(np.int64) - 8
    assert np.array_equal(s.astype(np.int64) - 127, e)
    scaled = np.abs(y.astype(np.float64)) / np.repeat(np.exp2(e.astype(np.float64)), 32, axis=1)
    for a, code in zip(scaled.ravel(), (c & 0x7F).ravel()):
        dist = np.abs(vals - min(a, 448.0))
        best = np.flatnonzero(dist == dist.min())
        want = best[0] if len(best) == 1 else [b for b in best if b % 2 == 0][0]
        assert code == want, (a, code, want)
    assert np.array_equal((c >> 7).astype(bool), np.signbit(y))


def test_block_quant_1x128_and_128x128():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((130, 300)).astype(np.float32)
    for br, bc in ((1, 128), (128, 128)):
        q, s = F.quantize_e4m3_blocks(x, br, bc)
        assert s.shape == (-(-130 // br), -(-300 // bc))
        # closed form for one block
        blk = x[:br, :bc]
        assert s[0, 0] == np.float32(np.abs(blk).max() / np.float32(448.0))
        d = F.dequantize_e4m3_blocks(q, s, br, bc)
        assert np.abs(d - x).max() <= np.abs(x).max() * 2.0 ** -4


def test_block_dequantize_element_by_element():
    """dequantize_e4m3_blocks against a scalar loop (value of the code times the scale of the block
    the element lies in), for whole blocks and for ragged last blocks, with distinct scales per block
    so that a transposed or shifted scale index shows."""
    rng = np.random.default_rng(3)
    tbl = F.e4m3_decode_table()
    for (R, C, br, bc) in ((256, 384, 128, 128), (3, 256, 1, 128), (130, 300, 128, 128), (5, 130, 1, 128)):
        q = rng.integers(0, 0x7E, size=(R, C), dtype=np.uint8)
        s = (1.0 + np.arange(-(-R // br) * -(-C // bc), dtype=np.float32)).reshape(-(-R // br), -(-C // bc))
        d = F.dequantize_e4m3_blocks(q, s, br, bc)
        assert d.shape == (R, C) and d.dtype == np.float32
        for r, c in [(0, 0), (R - 1, C - 1), (R - 1, 0), (0, C - 1)] + [(int(rng.integers(R)), int(rng.integers(C))) for _ in range(200)]:
            assert d[r, c] == np.float32(tbl[q[r, c]] * s[r // br, c // bc])


def test_reference_random_init_matches_std_mt19937():
    # first outputs of std::mt19937(42) are 1608637542, 3421126067, 4083286876 (known values)
    rs = np.random.RandomState(42)
    w = rs.randint(0, 2 ** 32, size=3, dtype=np.uint64)
    assert list(w) == [1608637542, 3421126067, 4083286876]
    a, b = F.reference_random_init(4, 2, 16)
    v0 = np.float32(2.0) * (np.float32(1608637542) / np.float32(4294967296.0)) + np.float32(-1.0)
    assert a[0, 0] == F.e4m3_encode(np.array([v0], dtype=np.float32))[0]
    assert a.shape == (4, 16) and b.shape == (2, 16)
    assert np.all(np.abs(F.e4m3_decode(a)) <= 1.0)


def test_oracle_bf16_gemm_against_torch():
    """oracle.gemm.bf16_gemm is the fp32 matmul of the bf16 values (torch CPU as the library routine)."""
    import torch
    from oracle import gemm as G
    rng = np.random.default_rng(0)
    a = F.bf16_round(rng.standard_normal((33, 96)).astype(np.float32))
    b = F.bf16_round(rng.standard_normal((17, 96)).astype(np.float32))
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).float()
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).float()
    ref = (ta.double() @ tb.double().t()).numpy()
    out = G.bf16_gemm(a, b)
    assert np.abs(out - ref).max() <= 1e-4 * np.abs(ref).max()
    # identity: exact
    eye = F.bf16_round(np.eye(96, dtype=np.float32))
    assert np.array_equal(G.bf16_gemm(eye, b), F.bf16_to_f32(b).T)
