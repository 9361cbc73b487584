"""MXFP4 GEMM: HIP path (through the C ABI) against the CPU oracle (dequantize + fp32 matmul).

Tolerance: relative Frobenius error <= 1e-2 on the bf16 output (north-star bound). The MFMA
applies the e8m0 block scales exactly (powers of two) and accumulates in fp32, so only
accumulation order and the final bf16 rounding differ from the oracle (~2e-3 observed).
"""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as G

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _run(hk, a, sa, b, sb, variant=-1):
    dev = torch.device("cuda:0")
    t = [torch.from_numpy(x).to(dev) for x in (a, sa, b, sb)]
    C = torch.full((a.shape[0], b.shape[0]), float("nan"), dtype=torch.bfloat16, device=dev)
    hk.tk_kernel.dispatch_mxfp4_gemm(t[0], t[1], t[2], t[3], C, variant=variant)
    torch.cuda.synchronize()
    return C.view(torch.int16).cpu().numpy().view(np.uint16)


def _rand_mx(rng, rows, K, spread=True):
    x = rng.standard_normal((rows, K)).astype(np.float32)
    if spread:  # different magnitudes per block so that the scales matter
        x *= np.exp2(rng.integers(-6, 7, size=(rows, K // 32))).repeat(32, axis=1).astype(np.float32)
    return F.quantize_mxfp4(x)


SHAPES = [(256, 256, 256), (256, 256, 512), (512, 768, 1024), (1024, 1024, 2048)]
RAGGED = [(300, 200, 256), (257, 255, 512), (64, 72, 768), (1000, 520, 512), (1, 200, 512), (5, 7, 256), (130, 70, 1280)]


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, -1])
@pytest.mark.parametrize("shape", SHAPES + RAGGED)
def test_mxfp4_gemm_matches_oracle(hk, shape, variant):
    M, N, K = shape
    print(f"mxfp4_gemm shape={shape} variant={variant}", flush=True)
    rng = np.random.default_rng(99 + M + N + K)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    out = F.bf16_to_f32(_run(hk, a, sa, b, sb, variant))
    ref = G.mxfp4_gemm(a, sa, b, sb)
    assert np.isfinite(out).all()
    err = G.rel_fro_error(out, ref)
    assert err <= TOL, (shape, variant, err)
    assert err <= 5e-3


@pytest.mark.parametrize("variant", [0, -1])
def test_mxfp4_gemm_k_not_multiple_of_256(hk, variant):
    M, N, K = 96, 80, 160
    rng = np.random.default_rng(7)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    out = F.bf16_to_f32(_run(hk, a, sa, b, sb, variant))
    assert G.rel_fro_error(out, G.mxfp4_gemm(a, sa, b, sb)) <= 5e-3


def test_mxfp4_gemm_tile_kernel_rejects_k_tail(hk):
    """Dense scale rows of fewer than 16 bytes (K < 512) that are not whole groups of 8: portable kernel only."""
    rng = np.random.default_rng(7)
    (a, sa), (b, sb) = _rand_mx(rng, 64, 160), _rand_mx(rng, 64, 160)
    with pytest.raises(RuntimeError):
        _run(hk, a, sa, b, sb, 1)


def _run_in_pool(hk, a, sa, b, sb, variant, misalign, workspace=False):
    """The GEMM with every operand array surrounded by bytes 0xFF (a scale byte fetched in front of or behind an
    array would be the e8m0 NaN) and the scale arrays starting `misalign` bytes off a 16-byte boundary."""
    dev = torch.device("cuda:0")
    views, pools = [], []
    for arr, mis in ((a, 0), (sa, misalign), (b, 0), (sb, misalign)):
        pool = torch.full((16 + mis + arr.size + 64,), 0xFF, dtype=torch.uint8, device=dev)
        view = pool[16 + mis:16 + mis + arr.size].view(arr.shape)
        view.copy_(torch.from_numpy(arr).to(dev))
        assert view.data_ptr() % 16 == mis
        pools.append(pool)
        views.append(view)
    A, SA, B, SB = views
    C = torch.full((a.shape[0], b.shape[0]), float("nan"), dtype=torch.bfloat16, device=dev)
    ws = None
    if workspace:
        need = hk.tk_kernel.mxfp4_gemm_workspace_bytes(a.shape[0], b.shape[0], a.shape[1] * 2)
        assert need > 0
        ws = torch.empty(need, dtype=torch.uint8, device=dev)
    hk.tk_kernel.dispatch_mxfp4_gemm(A, SA, B, SB, C, variant=variant, workspace=ws)
    torch.cuda.synchronize()
    return C.view(torch.int16).cpu().numpy().view(np.uint16)


# K / 32 scale bytes per row, dense rows: 90 (the GPT-OSS hidden size, tail fetched 2 bytes early), and one case
# for each remainder of K / 32 modulo 4 and for rows of whole and broken groups of 16 (more than 64 rows of A: with fewer
# the library picks the skinny kernel, tests/test_gemm_skinny_gpu.py)
DENSE_RAGGED = [(512, 2880, 2880), (300, 200, 2880), (130, 520, 32 * 17), (257, 255, 32 * 19), (72, 384, 32 * 20),
                (96, 80, 32 * 47), (256, 256, 32 * 33), (200, 136, 32 * 18)]


@pytest.mark.parametrize("variant", [1, 2, 3, -1])
@pytest.mark.parametrize("shape", DENSE_RAGGED)
def test_mxfp4_gemm_dense_scale_rows_any_k_on_the_tile_kernels(hk, shape, variant):
    """Dense [rows, K / 32] scale rows with K / 32 not a multiple of 8 (rows of any byte alignment) run on every
    tile kernel: same bits as the call with rows padded to a multiple of 8 bytes, oracle-close, and nothing past
    the arrays is fetched."""
    M, N, K = shape
    print(f"mxfp4_gemm dense ragged shape={shape} variant={variant}", flush=True)
    rng = np.random.default_rng(3 + M + N + K)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    ref = G.mxfp4_gemm(a, sa, b, sb)
    for mis in (0, 1, 3):
        bits = _run_in_pool(hk, a, sa, b, sb, variant, mis)
        out = F.bf16_to_f32(bits)
        assert np.isfinite(out).all(), (shape, variant, mis)
        assert G.rel_fro_error(out, ref) <= 5e-3, (shape, variant, mis)
        if mis == 0:
            first = bits
        assert np.array_equal(bits, first), (shape, variant, mis)
    pitch = (K // 32 + 7) // 8 * 8
    padded = _run(hk, a, _pad_rows(rng, sa, pitch), b, _pad_rows(rng, sb, pitch))   # picks the same tile
    if variant == -1:
        assert np.array_equal(first, padded)
        # ... and it is the tile kernel of the library's choice of tile, not the portable kernel
        forced = {256: 1, 128: 2, 64: 3}[hk.tk_kernel.gemm_tile_choice("mxfp4", M, N, K)]
        assert np.array_equal(first, _run_in_pool(hk, a, sa, b, sb, forced, 0))


def test_mxfp4_gemm_dense_scale_rows_split_k(hk):
    """The split-K path on dense scale rows whose last pair of K-steps is fetched early (K / 32 = 263)."""
    M, N, K = 16, 1024, 32 * 263
    rng = np.random.default_rng(21)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    out = F.bf16_to_f32(_run_in_pool(hk, a, sa, b, sb, -1, 1, workspace=True))
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.mxfp4_gemm(a, sa, b, sb)) <= 5e-3


@pytest.mark.parametrize("variant", [0, 1])
def test_mxfp4_gemm_exact_small_integers(hk, variant):
    """Elements in {-2,-1,0,1,2} with power-of-two block scales: every product and partial sum
    is exact in fp32, so the result must equal the exact value rounded once to bf16."""
    M, N, K = 256, 512, 512
    rng = np.random.default_rng(21)
    codes = np.array([0, 2, 4, 10, 12], dtype=np.uint8)  # e2m1 codes of 0, 1, 2, -1, -2

    def make(rows):
        c = codes[rng.integers(0, 5, size=(rows, K))]
        packed = (c[:, 0::2] | (c[:, 1::2] << 4)).astype(np.uint8)
        scales = rng.integers(125, 130, size=(rows, K // 32)).astype(np.uint8)
        return packed, scales

    (a, sa), (b, sb) = make(M), make(N)
    out = _run(hk, a, sa, b, sb, variant)
    exact = F.dequantize_mxfp4(a, sa).astype(np.float64) @ F.dequantize_mxfp4(b, sb).astype(np.float64).T
    assert np.array_equal(out, F.bf16_round(exact.astype(np.float32)))


def test_mxfp4_gemm_scale_byte_positions(hk):
    """One nonzero block per row pair: catches a scale applied to the wrong 32-block."""
    M = N = 256
    K = 512
    a = np.zeros((M, K // 2), np.uint8); b = np.zeros((N, K // 2), np.uint8)
    sa = np.full((M, K // 32), 127, np.uint8); sb = np.full((N, K // 32), 127, np.uint8)
    rng = np.random.default_rng(2)
    blk_a = rng.integers(0, K // 32, size=M)
    for i in range(M):
        a[i, blk_a[i] * 16:(blk_a[i] + 1) * 16] = 0x22  # all ones in that block
        sa[i, :] = rng.integers(120, 134, size=K // 32)
    b[:] = 0x22
    sb[:] = rng.integers(120, 134, size=(N, K // 32))
    out = _run(hk, a, sa, b, sb, 1)
    exact = F.dequantize_mxfp4(a, sa).astype(np.float64) @ F.dequantize_mxfp4(b, sb).astype(np.float64).T
    assert np.array_equal(out, F.bf16_round(exact.astype(np.float32)))


def test_mxfp4_gemm_device_quantizer_matches_oracle(hk):
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((128, 256)) * np.exp2(rng.integers(-20, 20, size=(128, 1)))).astype(np.float32)
    x[3, :32] = 0.0
    p, s = hk.quant.quantize_mxfp4(torch.from_numpy(x).to(dev))
    po, so = F.quantize_mxfp4(x)
    assert np.array_equal(p.cpu().numpy(), po) and np.array_equal(s.cpu().numpy(), so)


def _pad_rows(rng, s, pitch):
    """Scale rows widened to `pitch` bytes; the padding holds arbitrary bytes other than 0xFF."""
    out = rng.integers(0, 255, size=(s.shape[0], pitch), dtype=np.uint8)
    out[:, :s.shape[1]] = s
    return out


PITCHED = [(2048, 2304, 2880, 96, 96), (16, 2880, 2880, 96, 96), (256, 256, 2880, 96, 96), (300, 520, 2880, 96, 104), (512, 384, 160, 8, 8), (128, 640, 1056, 40, 40),
           (256, 256, 512, 24, 16), (200, 264, 96, 8, 16), (96, 80, 2880, 91, 96)]


@pytest.mark.parametrize("case", PITCHED)
def test_mxfp4_gemm_padded_scale_rows_and_k_tails(hk, case):
    """Scale rows padded to a pitch (a multiple of 8 bytes keeps any K % 32 == 0 on the tile kernel:
    the last K-step's bytes past the row end are not fetched; the operand buffers sit at the end of
    a pool filled with 0xFF so that a fetch past the row would show). The last case has a pitch that
    is not a multiple of 8: its last pair of K-steps is fetched two bytes early."""
    M, N, K, pa, pb = case
    print(f"mxfp4_gemm pitched case={case}", flush=True)
    rng = np.random.default_rng(11 + M + N + K)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    dev = torch.device("cuda:0")
    pool = torch.full((2 * (a.size + b.size),), 0xFF, dtype=torch.uint8, device=dev)
    A = pool[pool.numel() - a.size:].view(M, K // 2)
    B = pool[pool.numel() - a.size - b.size:pool.numel() - a.size].view(N, K // 2)
    A.copy_(torch.from_numpy(a).to(dev))
    B.copy_(torch.from_numpy(b).to(dev))
    SA = torch.from_numpy(_pad_rows(rng, sa, pa)).to(dev)
    SB = torch.from_numpy(_pad_rows(rng, sb, pb)).to(dev)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    hk.tk_kernel.dispatch_mxfp4_gemm(A, SA, B, SB, C)
    torch.cuda.synchronize()
    out = C.float().cpu().numpy()
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.mxfp4_gemm(a, sa, b, sb)) <= 5e-3


def test_mxfp4_gemm_padded_rows_equal_dense_rows_bit_for_bit(hk):
    M, N, K = 512, 768, 1024
    rng = np.random.default_rng(5)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    dense = _run(hk, a, sa, b, sb)
    padded = _run(hk, a, _pad_rows(rng, sa, 40), b, _pad_rows(rng, sb, 48))
    assert np.array_equal(dense, padded)


SPLITK = [(16, 1024, 8192, 0), (1, 512, 8192, 0), (100, 200, 4128, 136), (128, 1000, 6176, 200), (64, 64, 16384, 0)]


@pytest.mark.parametrize("case", SPLITK)
def test_mxfp4_gemm_split_k_matches_oracle(hk, case):
    """Decode-like shapes with a workspace: K split over several workgroups per tile (ranges of an even
    number of K-steps; the last range of two cases ends in a partial K-step), fp32 partial sums added
    in a fixed order. The workspace starts as NaNs, so a partial sum that is read but was not written
    would show; with a workspace that is too small the call must give the plain kernel's result."""
    M, N, K, pitch = case
    print(f"mxfp4_gemm split-k case={case}", flush=True)
    need = hk.tk_kernel.mxfp4_gemm_workspace_bytes(M, N, K)
    assert need > 0, "these shapes are meant to take the split path"
    assert hk.tk_kernel.mxfp4_gemm_workspace_bytes(1024, 1024, 8192) == 0    # enough tiles
    assert hk.tk_kernel.mxfp4_gemm_workspace_bytes(16, 2880, 2880) == 0      # K too short
    assert hk.tk_kernel.mxfp4_gemm_workspace_bytes(128, 4096, 4096) == 0     # partial sums cost more than they save
    rng = np.random.default_rng(3 + M + N + K)
    (a, sa), (b, sb) = _rand_mx(rng, M, K), _rand_mx(rng, N, K)
    ref = G.mxfp4_gemm(a, sa, b, sb)
    if pitch:
        sa, sb = _pad_rows(rng, sa, pitch), _pad_rows(rng, sb, pitch)
    dev = torch.device("cuda:0")
    t = [torch.from_numpy(x).to(dev) for x in (a, sa, b, sb)]
    ws = torch.full((need,), 0xFF, dtype=torch.uint8, device=dev)
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
    hk.tk_kernel.dispatch_mxfp4_gemm(*t, C, workspace=ws)
    torch.cuda.synchronize()
    out = C.float().cpu().numpy()
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, ref) <= 5e-3
    plain = torch.empty_like(C)
    hk.tk_kernel.dispatch_mxfp4_gemm(*t, plain)
    small = torch.empty_like(C)
    hk.tk_kernel.dispatch_mxfp4_gemm(*t, small, workspace=ws[:need - 16])
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), small.view(torch.int16))
