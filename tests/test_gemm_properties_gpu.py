"""Properties of the GEMMs that hold at any size: the tile a problem is given (chosen by its size)
does not change a result bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_tile_sizes_give_identical_bits(hk):
    """256x256, 128x128 and 64x64 tiles walk K in the same order with the same MFMA, so the choice of
    tile (made by problem size) never changes a result bit: FP8, BF16 and MXFP4, with ragged edges and
    a K tail."""
    print("tile sizes bit identity", flush=True)
    g = torch.Generator(device=DEV).manual_seed(9)
    M, N, K = 520, 392, 1296
    A = torch.randn(M, K, device=DEV, generator=g)
    B = torch.randn(N, K, device=DEV, generator=g)

    def run(fn, variants):
        outs = []
        for v in variants:
            C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
            fn(C, v)
            torch.cuda.synchronize()
            outs.append(C.view(torch.int16).clone())
        for o in outs[1:]:
            assert torch.equal(outs[0], o)

    A8, B8 = A.to(torch.float8_e4m3fn), B.to(torch.float8_e4m3fn)
    run(lambda C, v: hk.tk_kernel.dispatch_fp8_gemm(A8, B8, C, 0.5, 2.0, variant=v), [4, 5, 6])
    Ab, Bb = A.to(torch.bfloat16), B.to(torch.bfloat16)
    run(lambda C, v: hk.tk_kernel.dispatch_bf16_gemm(Ab, Bb, C, variant=v), [1, 2, 3])
    K4 = 1280  # dense scale rows: K % 256 == 0
    Ap, As = hk.quant.quantize_mxfp4(A[:, :K4].contiguous())
    Bp, Bs = hk.quant.quantize_mxfp4(B[:, :K4].contiguous())
    run(lambda C, v: hk.tk_kernel.dispatch_mxfp4_gemm(Ap, As, Bp, Bs, C, variant=v), [1, 2, 3])
