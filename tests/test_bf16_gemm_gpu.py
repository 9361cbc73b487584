"""BF16 GEMM: HIP path (through the C ABI) against the CPU oracle (fp32 matmul of the bf16 values,
the check of the reference's kernels/gemm/bf16fp32/mi350x/test_python.py:17,32,105-117).

Tolerance: relative Frobenius error <= 1e-2 on the bf16 output (north-star bound; ~2e-3 observed:
accumulation order and the final bf16 rounding are the only differences). Exact cases: identity
and small integers (every product and partial sum is representable).
"""
import numpy as np
import pytest
import torch

from oracle import formats as F
from oracle import gemm as G

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2


def _bits(a):
    return F.bf16_round(np.asarray(a, dtype=np.float32))


def _run(hk, a_bits, b_bits, variant=-1):
    A = torch.from_numpy(a_bits.view(np.int16)).view(torch.bfloat16).to(DEV)
    B = torch.from_numpy(b_bits.view(np.int16)).view(torch.bfloat16).to(DEV)
    C = torch.full((a_bits.shape[0], b_bits.shape[0]), float("nan"), dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_bf16_gemm(A, B, C, variant=variant)
    torch.cuda.synchronize()
    return C.view(torch.int16).cpu().numpy().view(np.uint16)


SHAPES = [(256, 256, 64), (256, 256, 128), (256, 256, 192), (512, 768, 1024), (1024, 1024, 2048)]
RAGGED = [(300, 200, 256), (257, 255, 512), (64, 72, 768), (1000, 520, 320), (1, 200, 512), (5, 7, 128)]


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, -1])
@pytest.mark.parametrize("shape", SHAPES + RAGGED)
def test_bf16_gemm_matches_oracle(hk, shape, variant):
    M, N, K = shape
    print(f"bf16_gemm shape={shape} variant={variant}", flush=True)
    rng = np.random.default_rng(M + 3 * N + 7 * K)
    a, b = _bits(rng.standard_normal((M, K))), _bits(rng.standard_normal((N, K)))
    out = F.bf16_to_f32(_run(hk, a, b, variant))
    ref = G.bf16_gemm(a, b)
    assert np.isfinite(out).all()
    err = G.rel_fro_error(out, ref)
    assert err <= TOL, (shape, variant, err)
    assert err <= 5e-3  # expected level; a layout bug gives O(1)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, -1])
@pytest.mark.parametrize("shape", [(96, 80, 104), (256, 256, 8), (300, 264, 200), (256, 384, 2880)])
def test_bf16_gemm_k_not_multiple_of_64(hk, shape, variant):
    """K % 8 == 0 only: the tile kernel zero-fills the last K-step."""
    M, N, K = shape
    print(f"bf16_gemm k-tail shape={shape} variant={variant}", flush=True)
    rng = np.random.default_rng(11 + K)
    a, b = _bits(rng.standard_normal((M, K))), _bits(rng.standard_normal((N, K)))
    out = F.bf16_to_f32(_run(hk, a, b, variant))
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, G.bf16_gemm(a, b)) <= 5e-3


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5])
def test_bf16_gemm_identity_is_bit_exact(hk, variant):
    # A = I (K = M): C = bf16(B)^T exactly, whatever the accumulation order
    n = 256
    rng = np.random.default_rng(3)
    a = _bits(np.eye(n, dtype=np.float32))
    b = _bits(rng.standard_normal((384, n)))
    out = _run(hk, a, b, variant)
    assert np.array_equal(out, b.T)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5])
def test_bf16_gemm_small_integers_exact(hk, variant):
    # integer operands in [-4, 4], K = 512: all partial sums are integers < 2^14, exact in fp32;
    # the result is rounded to bf16 once, like the oracle's
    rng = np.random.default_rng(5)
    a = _bits(rng.integers(-4, 5, size=(300, 512)))
    b = _bits(rng.integers(-4, 5, size=(260, 512)))
    out = _run(hk, a, b, variant)
    assert np.array_equal(out, F.bf16_round(G.bf16_gemm(a, b)))


def test_bf16_gemm_dispatch_micro_and_torch(hk):
    # the reference's entry point name, against torch's own matmul
    torch.manual_seed(0)
    A = torch.randn(512, 1024, device=DEV).to(torch.bfloat16)
    B = torch.randn(768, 1024, device=DEV).to(torch.bfloat16)
    C = torch.zeros(512, 768, dtype=torch.bfloat16, device=DEV)
    hk.tk_kernel.dispatch_micro(A, B, C)
    torch.cuda.synchronize()
    ref = A.float() @ B.float().t()
    err = ((C.float() - ref).norm() / ref.norm()).item()
    assert err <= 5e-3, err


def test_bf16_gemm_rejects_bad_arguments(hk):
    A = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    C = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_bf16_gemm(A, A.float(), C)          # wrong dtype
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_bf16_gemm(A, A[:, :32], C)          # non-contiguous / K mismatch
    with pytest.raises(RuntimeError):
        hk.tk_kernel.dispatch_bf16_gemm(A.cpu(), A, C)            # CPU tensor


@pytest.mark.parametrize("shape", [(16, 1024, 4096), (100, 520, 3080), (128, 512, 3072), (1, 128, 8192)])
def test_bf16_gemm_split_k_matches_oracle(hk, shape):
    """Decode-like shapes with a workspace: K split over several workgroups per tile, partial sums
    added in a fixed order; checked against the oracle and for run-to-run bit identity."""
    M, N, K = shape
    print(f"bf16_gemm split-k shape={shape}", flush=True)
    need = hk.tk_kernel.bf16_gemm_workspace_bytes(M, N, K)
    assert need > 0, "these shapes are meant to take the split path"
    assert hk.tk_kernel.bf16_gemm_workspace_bytes(1024, 1024, 1024) == 0
    rng = np.random.default_rng(3 + M + N + K)
    a = F.bf16_round(rng.standard_normal((M, K)).astype(np.float32))
    b = F.bf16_round(rng.standard_normal((N, K)).astype(np.float32))
    dev = torch.device("cuda:0")
    A = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).to(dev)
    B = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).to(dev)
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    outs = []
    for _ in range(2):
        C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=dev)
        ws.fill_(0xFF)  # NaN patterns: every partial sum that is read must have been written
        hk.tk_kernel.dispatch_bf16_gemm(A, B, C, workspace=ws)
        torch.cuda.synchronize()
        outs.append(C.view(torch.int16).cpu().numpy().view(np.uint16))
    assert np.array_equal(outs[0], outs[1])
    out = F.bf16_to_f32(outs[0])
    ref = F.bf16_to_f32(a).astype(np.float64) @ F.bf16_to_f32(b).astype(np.float64).T
    assert np.isfinite(out).all()
    assert G.rel_fro_error(out, ref) <= 5e-3
