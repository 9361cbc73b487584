"""Properties of the GEMMs that hold at any size: the tile a problem is given (chosen by its size)
does not change a result bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_tile_sizes_give_identical_bits(hk):
    """256x256 (4-wave interleaved and 8-wave ping-pong schedules), 128x128 and 64x64 tiles walk K in the
    same order with the same MFMA, so the choice of tile and schedule never changes a result bit: FP8,
    BF16 and MXFP4, with ragged edges and a K tail."""
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
    run(lambda C, v: hk.tk_kernel.dispatch_fp8_gemm(A8, B8, C, 0.5, 2.0, variant=v), [4, 5, 6, 1, 7])
    Ab, Bb = A.to(torch.bfloat16), B.to(torch.bfloat16)
    run(lambda C, v: hk.tk_kernel.dispatch_bf16_gemm(Ab, Bb, C, variant=v), [1, 2, 3, 4, 5])
    K4 = 1280  # dense scale rows: K % 256 == 0
    Ap, As = hk.quant.quantize_mxfp4(A[:, :K4].contiguous())
    Bp, Bs = hk.quant.quantize_mxfp4(B[:, :K4].contiguous())
    run(lambda C, v: hk.tk_kernel.dispatch_mxfp4_gemm(Ap, As, Bp, Bs, C, variant=v), [1, 2, 3, 4, 5])


@pytest.mark.parametrize("kind", ["fp8", "bf16"])
def test_banded_tile_order_covers_every_tile(hk, kind):
    """Operands of more than 320 MB are walked in bands of 16 tile columns (ragged last band, ragged
    edges here): every tile must still be computed exactly once. Checked against the 128x128-tile
    kernel, which uses the plain order and gives the same bits."""
    M, N = 10000 + 200, 16384 + 8 * 256 + 40      # 40 x 73 tiles: four bands of 16 and one of 9
    K = 13312 if kind == "fp8" else 6656
    print(f"banded raster {kind} {M}x{N}x{K}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(3)
    dt = torch.float8_e4m3fn if kind == "fp8" else torch.bfloat16
    A = torch.randn(M, K, device=DEV, generator=g).to(dt)
    B = torch.randn(N, K, device=DEV, generator=g).to(dt)
    assert (M + N) * K * A.element_size() > 320 << 20
    C = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    C0 = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    if kind == "fp8":
        hk.tk_kernel.dispatch_fp8_gemm(A, B, C, 1.0, 1.0, variant=4)
        hk.tk_kernel.dispatch_fp8_gemm(A, B, C0, 1.0, 1.0, variant=5)
    else:
        hk.tk_kernel.dispatch_bf16_gemm(A, B, C, variant=1)
        hk.tk_kernel.dispatch_bf16_gemm(A, B, C0, variant=2)
    torch.cuda.synchronize()
    assert torch.equal(C.view(torch.int16), C0.view(torch.int16))
    assert torch.isfinite(C.float()).all()
