"""FP8 GEMM: HIP path (through the C ABI) against the CPU oracle.

Tolerance: relative Frobenius error <= 1e-2 (the north-star bound; the metric is the
reference's l2_error, kernels/attn/gqa/test_python.py:55). The oracle accumulates in fp32
like the MFMA; differences come from accumulation order and the single bf16 rounding, so
observed errors are ~2e-3. Exactly representable cases are checked bit for bit.
"""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as G

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _run(hk, a_codes, b_codes, sa=1.0, sb=1.0, variant=-1):
    dev = torch.device("cuda:0")
    A = torch.from_numpy(a_codes).to(dev).view(torch.float8_e4m3fn)
    B = torch.from_numpy(b_codes).to(dev).view(torch.float8_e4m3fn)
    C = torch.full((A.shape[0], B.shape[0]), float("nan"), dtype=torch.bfloat16, device=dev)
    hk.tk_kernel.dispatch_fp8_gemm(A, B, C, sa, sb, variant=variant)
    torch.cuda.synchronize()
    return C.view(torch.int16).cpu().numpy().view(np.uint16)


def _random_codes(rng, rows, K):
    x = rng.standard_normal((rows, K)).astype(np.float32)
    return F.quantize_e4m3_per_tensor(x)


SHAPES = [(256, 256, 256), (256, 256, 128), (512, 768, 384), (1024, 1024, 1024), (256, 512, 2048)]
RAGGED = [(300, 200, 256), (257, 255, 128), (64, 72, 640), (1000, 1000, 512), (1, 200, 512), (5, 7, 256)]


@pytest.mark.parametrize("variant", [0, 1, 4, 5, 6, 7, -1])
@pytest.mark.parametrize("shape", SHAPES + RAGGED)
def test_fp8_gemm_matches_oracle(hk, shape, variant):
    M, N, K = shape
    print(f"fp8_gemm shape={shape} variant={variant}", flush=True)
    rng = np.random.default_rng(1234 + M + N + K)
    (a, sa), (b, sb) = _random_codes(rng, M, K), _random_codes(rng, N, K)
    out = F.bf16_to_f32(_run(hk, a, b, float(sa), float(sb), variant))
    ref = G.fp8_gemm(a, b, sa, sb)
    assert np.isfinite(out).all()
    err = G.rel_fro_error(out, ref)
    assert err <= TOL, (shape, variant, err)
    assert err <= 5e-3  # expected level; a layout bug gives O(1)


K_TAIL = [(96, 80, 208), (256, 256, 16), (256, 256, 144), (300, 520, 272), (512, 384, 2880), (128, 128, 112)]


@pytest.mark.parametrize("variant", [0, 1, 4, 5, 6, 7, -1])
@pytest.mark.parametrize("shape", K_TAIL)
def test_fp8_gemm_k_tail(hk, shape, variant):
    """K % 16 == 0 but K % 128 != 0 (2880 is the hidden size of the MoE models): the ring and
    128x128- / 64x64-tile kernels zero-fill the last K-step. The buffers are carved out of a larger one
    filled with NaN codes, so a read past a row's end would show in the result."""
    M, N, K = shape
    print(f"fp8_gemm k-tail shape={shape} variant={variant}", flush=True)
    rng = np.random.default_rng(7 + K)
    (a, sa), (b, sb) = _random_codes(rng, M, K), _random_codes(rng, N, K)
    out = F.bf16_to_f32(_run(hk, a, b, float(sa), float(sb), variant))
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.fp8_gemm(a, b, sa, sb)) <= 5e-3


def test_fp8_gemm_k_tail_last_row_does_not_read_past_the_buffer(hk):
    """The last row's tail chunks lie past the end of the allocation: with A and B placed at the
    very end of a NaN-filled pool, a kernel that fetched them would return NaN."""
    M, N, K = 256, 256, 208
    rng = np.random.default_rng(99)
    (a, sa), (b, sb) = _random_codes(rng, M, K), _random_codes(rng, N, K)
    dev = torch.device("cuda:0")
    for variant in (1, 4, 5, 6, 7):
        pool = torch.full((4 * M * K,), 0x7F, dtype=torch.uint8, device=dev)  # e4m3fn NaN code
        A = pool[M * K:2 * M * K].view(M, K)
        B = pool[2 * M * K:3 * M * K].view(N, K)
        A.copy_(torch.from_numpy(a).to(dev))
        B.copy_(torch.from_numpy(b).to(dev))
        C = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
        hk.tk_kernel.dispatch_fp8_gemm(A.view(torch.float8_e4m3fn), B.view(torch.float8_e4m3fn), C,
                                       float(sa), float(sb), variant=variant)
        torch.cuda.synchronize()
        out = C.float().cpu().numpy()
        assert np.isfinite(out).all(), variant
        assert G.rel_fro_error(out, G.fp8_gemm(a, b, sa, sb)) <= 5e-3


SPLITK = [(16, 1024, 8192), (64, 512, 8192), (100, 520, 6160), (128, 1024, 6144), (1, 128, 8192), (33, 200, 12288)]


@pytest.mark.parametrize("shape", SPLITK)
def test_fp8_gemm_split_k_matches_oracle(hk, shape):
    """Decode-like shapes with a workspace: K split over several workgroups per tile, partial sums
    added in a fixed order. Checked against the oracle and for run-to-run bit identity."""
    M, N, K = shape
    print(f"fp8_gemm split-k shape={shape}", flush=True)
    need = hk.tk_kernel.fp8_gemm_workspace_bytes(M, N, K)
    assert need > 0, "these shapes are meant to take the split path"
    rng = np.random.default_rng(3 + M + N + K)
    (a, sa), (b, sb) = _random_codes(rng, M, K), _random_codes(rng, N, K)
    dev = torch.device("cuda:0")
    A = torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn)
    B = torch.from_numpy(b).to(dev).view(torch.float8_e4m3fn)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    outs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        ws.fill_(0xFF)  # NaN patterns: every partial sum that is read must have been written
        hk.tk_kernel.dispatch_fp8_gemm(A, B, C, float(sa), float(sb), workspace=ws)
        torch.cuda.synchronize()
        outs.append(C.view(torch.int16).cpu().numpy().view(np.uint16))
    assert np.array_equal(outs[0], outs[1])
    out = F.bf16_to_f32(outs[0])
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.fp8_gemm(a, b, sa, sb)) <= 5e-3


def test_fp8_gemm_workspace_is_optional(hk):
    # shapes that are not split (enough tiles, or a short K): zero bytes, and a workspace changes nothing
    assert hk.tk_kernel.fp8_gemm_workspace_bytes(2048, 2048, 1024) == 0
    assert hk.tk_kernel.fp8_gemm_workspace_bytes(1024, 1024, 1024) == 0
    rng = np.random.default_rng(5)
    (a, sa), (b, sb) = _random_codes(rng, 256, 256), _random_codes(rng, 256, 256)
    base = _run(hk, a, b, float(sa), float(sb), -1)
    dev = torch.device("cuda:0")
    C = torch.zeros((256, 256), dtype=torch.bfloat16, device=dev)
    hk.tk_kernel.dispatch_fp8_gemm(torch.from_numpy(a).to(dev).view(torch.float8_e4m3fn),
                                   torch.from_numpy(b).to(dev).view(torch.float8_e4m3fn), C, float(sa), float(sb),
                                   workspace=torch.empty(16, dtype=torch.uint8, device=dev))
    torch.cuda.synchronize()
    assert np.array_equal(C.view(torch.int16).cpu().numpy().view(np.uint16), base)


@pytest.mark.parametrize("variant", [2, 3, 9])
def test_fp8_gemm_rejects_unknown_variants(hk, variant):
    rng = np.random.default_rng(7)
    (a, _), (b, _) = _random_codes(rng, 256, 256), _random_codes(rng, 256, 256)
    with pytest.raises(RuntimeError):
        _run(hk, a, b, 1.0, 1.0, variant)


@pytest.mark.parametrize("variant", [0, 1, 4, 5, 6, 7])
def test_fp8_gemm_identity_is_bit_exact(hk, variant):
    """A = I (K = M): C = bf16(B^T) exactly; every e4m3 value is a bf16 value."""
    n = 256
    a = np.zeros((n, n), dtype=np.uint8)
    a[np.arange(n), np.arange(n)] = 0x38  # 1.0
    rng = np.random.default_rng(3)
    b = rng.integers(0, 256, size=(512, n), dtype=np.uint8)
    b[(b & 0x7F) == 0x7F] = 0x00  # no NaN
    out = _run(hk, a, b, 1.0, 1.0, variant)
    expect = F.bf16_round(F.e4m3_decode(b).T)
    # -0.0 * 1.0 summed with +0.0 terms gives +0.0: compare values, not sign of zero
    assert np.array_equal(F.bf16_to_f32(out), F.bf16_to_f32(expect))


@pytest.mark.parametrize("variant", [1, 4, 5, 6, 7])
def test_fp8_gemm_small_integers_exact(hk, variant):
    """Operands in {-2..2}: all products and partial sums are exact in fp32, so the result is
    order independent and must equal the integer matmul, rounded once to bf16."""
    M, N, K = 512, 256, 384
    rng = np.random.default_rng(11)
    ai = rng.integers(-2, 3, size=(M, K))
    bi = rng.integers(-2, 3, size=(N, K))
    a, b = F.e4m3_encode(ai.astype(np.float32)), F.e4m3_encode(bi.astype(np.float32))
    out = _run(hk, a, b, 0.5, 4.0, variant)
    expect = F.bf16_round((ai @ bi.T).astype(np.float32) * np.float32(2.0))
    assert np.array_equal(out, expect)


def test_fp8_gemm_scale_linearity(hk):
    rng = np.random.default_rng(5)
    (a, _), (b, _) = _random_codes(rng, 256, 256), _random_codes(rng, 256, 256)
    c1 = F.bf16_to_f32(_run(hk, a, b, 1.0, 1.0))
    c2 = F.bf16_to_f32(_run(hk, a, b, 2.0, 4.0))
    assert np.array_equal(c1 * 8.0, c2)  # power-of-two scaling commutes with rounding


def test_fp8_gemm_reference_style_inputs(hk):
    """The reference executable's own inputs: mt19937(42), U(-1,1), unit scales
    (kernels/gemm/fp8fp32/profile_utils.cpp:35-45), at a reduced size."""
    a, b = F.reference_random_init(512, 512, 512)
    out = F.bf16_to_f32(_run(hk, a, b))
    assert G.rel_fro_error(out, G.fp8_gemm(a, b)) <= 5e-3


def test_fp8_gemm_8192_against_portable_and_sampled_oracle(hk):
    """Full headline size: tile kernel vs portable kernel (both on the GPU) everywhere, and
    vs the CPU oracle on a sample of rows."""
    n = 8192
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)
    A = torch.randn(n, n, device=dev, generator=g)
    B = torch.randn(n, n, device=dev, generator=g)
    Aq, sa = hk.quant.quantize_fp8_per_tensor(A)
    Bq, sb = hk.quant.quantize_fp8_per_tensor(B)
    del A, B
    C = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    C0 = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
    hk.tk_kernel.dispatch_fp8_gemm(Aq, Bq, C, sa, sb)
    hk.tk_kernel.dispatch_fp8_gemm(Aq, Bq, C0, sa, sb, variant=0)
    torch.cuda.synchronize()
    diff = (C.float() - C0.float()).norm() / C0.float().norm()
    assert diff.item() <= 5e-3
    rows = np.arange(0, n, 257)
    a = Aq.view(torch.uint8)[torch.from_numpy(rows).to(dev)].cpu().numpy()
    b = Bq.view(torch.uint8).cpu().numpy()
    ref = G.fp8_gemm(a, b, sa, sb)
    out = C[torch.from_numpy(rows).to(dev)].float().cpu().numpy()
    assert G.rel_fro_error(out, ref) <= 5e-3
