"""Every entry point can be recorded into a HIP graph (no allocation, no memset node, no host
synchronisation inside the library): a graph of several launches is replayed three times, with
eager work of the program and synchronisations between the replays, and every replay must
reproduce the eager result bit for bit (all kernels here are deterministic).
"""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _replay_and_compare(fn, outs, scratch_fn=None):
    """fn() writes `outs` (tensors). Eager once, then captured twice in a row, replayed three times."""
    fn()
    torch.cuda.synchronize()
    want = [o.clone() for o in outs]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn()
        fn()
    for rep in range(3):
        for o in outs:
            o.zero_()              # a fill kernel of the program between the replays
        if scratch_fn is not None:
            scratch_fn()           # eager work that dirties the library's workspace
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for o, w in zip(outs, want):
            assert torch.equal(o.view(torch.uint8), w.view(torch.uint8)), f"replay {rep} differs from the eager call"


@pytest.mark.parametrize("shape", [(1024, 1024, 1024), (300, 520, 272), (2048, 2048, 512), (256, 4096, 4096)])
def test_fp8_gemm_in_a_graph(hk, shape):
    M, N, K = shape
    print(f"graph fp8_gemm shape={shape}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(M + N + K)
    A = torch.randn(M, K, device=DEV, generator=g).to(torch.float8_e4m3fn)
    B = torch.randn(N, K, device=DEV, generator=g).to(torch.float8_e4m3fn)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    _replay_and_compare(lambda: hk.tk_kernel.dispatch_fp8_gemm(A, B, C, 0.5, 2.0), [C])


@pytest.mark.parametrize("M", [16, 128])   # the skinny kernel / split-K and its reduction
def test_fp8_split_k_in_a_graph(hk, M):
    N, K = 1024, 8192
    print(f"graph fp8_gemm with workspace M={M}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(1)
    A = torch.randn(M, K, device=DEV, generator=g).to(torch.float8_e4m3fn)
    B = torch.randn(N, K, device=DEV, generator=g).to(torch.float8_e4m3fn)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    need = hk.tk_kernel.fp8_gemm_workspace_bytes(M, N, K)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    _replay_and_compare(lambda: hk.tk_kernel.dispatch_fp8_gemm(A, B, C, 1.0, 1.0, workspace=ws), [C],
                        scratch_fn=lambda: ws.fill_(0xFF))


@pytest.mark.parametrize("M", [16, 128])   # the skinny kernel / split-K and its reduction
def test_mxfp4_split_k_in_a_graph(hk, M):
    N, K = 1024, 8192
    print(f"graph mxfp4_gemm with workspace M={M}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(5)
    Ap, As = hk.quant.quantize_mxfp4(torch.randn(M, K, device=DEV, generator=g))
    Bp, Bs = hk.quant.quantize_mxfp4(torch.randn(N, K, device=DEV, generator=g))
    C = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    need = hk.tk_kernel.mxfp4_gemm_workspace_bytes(M, N, K)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    _replay_and_compare(lambda: hk.tk_kernel.dispatch_mxfp4_gemm(Ap, As, Bp, Bs, C, workspace=ws), [C],
                        scratch_fn=lambda: ws.fill_(0xFF))


def test_bf16_and_mxfp4_gemm_in_a_graph(hk):
    print("graph bf16 / mxfp4 gemm", flush=True)
    g = torch.Generator(device=DEV).manual_seed(2)
    M, N, K = 512, 768, 1024
    A = torch.randn(M, K, device=DEV, generator=g).to(torch.bfloat16)
    B = torch.randn(N, K, device=DEV, generator=g).to(torch.bfloat16)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    Ap, As = hk.quant.quantize_mxfp4(A)
    Bp, Bs = hk.quant.quantize_mxfp4(B)
    C4 = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)

    def fn():
        hk.tk_kernel.dispatch_bf16_gemm(A, B, C)
        hk.tk_kernel.dispatch_mxfp4_gemm(Ap, As, Bp, Bs, C4)

    _replay_and_compare(fn, [C, C4])


def test_moe_mxfp4_layer_in_a_graph(hk):
    T, E, k, H, I = 512, 16, 4, 256, 192
    print("graph moe_mxfp4 layer", flush=True)
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn(T, H, device=DEV, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, device=DEV, generator=g)
    q13 = [hk.quant.quantize_mxfp4(torch.randn(2 * I, H, device=DEV, generator=g) * 0.1) for _ in range(E)]
    q2 = [hk.quant.quantize_mxfp4(torch.randn(H, I, device=DEV, generator=g) * 0.1) for _ in range(E)]
    W = hk.tk_kernel.MoeMxfp4ShuffledWeights.from_plain(
        torch.stack([a for a, _ in q13]), torch.stack([hk.quant.pad_scales(s) for _, s in q13]),
        torch.stack([a for a, _ in q2]), torch.stack([hk.quant.pad_scales(s) for _, s in q2]))
    ws = torch.empty(hk.tk_kernel.moe_mxfp4_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
    _replay_and_compare(lambda: hk.tk_kernel.dispatch_moe_mxfp4(x, logits, W, None, None, None, y, k, ws), [y],
                        scratch_fn=lambda: ws.fill_(0xA5))


def test_moe_fp8blk_layer_in_a_graph(hk):
    T, E, k, H, I, G, KG = 300, 16, 4, 256, 128, 4, 2
    print("graph moe_fp8blk layer", flush=True)
    g = torch.Generator(device=DEV).manual_seed(4)
    xq, xs = hk.quant.quantize_fp8_blocks(torch.randn(T, H, device=DEV, generator=g), 1, 128)
    logits = torch.randn(T, E, device=DEV, generator=g)
    w13q = torch.empty((E, 2 * I, H), dtype=torch.float8_e4m3fn, device=DEV)
    w13s = torch.empty((E, 2 * I // 128, H // 128), dtype=torch.float32, device=DEV)
    w2q = torch.empty((E, H, I), dtype=torch.float8_e4m3fn, device=DEV)
    w2s = torch.empty((E, H // 128, I // 128), dtype=torch.float32, device=DEV)
    for e in range(E):
        w13q[e], w13s[e] = hk.quant.quantize_fp8_blocks(torch.randn(2 * I, H, device=DEV, generator=g) * 0.1, 128, 128)
        w2q[e], w2s[e] = hk.quant.quantize_fp8_blocks(torch.randn(H, I, device=DEV, generator=g) * 0.1, 128, 128)
    ws = torch.empty(hk.tk_kernel.moe_fp8blk_workspace_bytes(T, H, I, E, k), dtype=torch.uint8, device=DEV)
    y = torch.empty((T, H), dtype=torch.bfloat16, device=DEV)
    _replay_and_compare(lambda: hk.tk_kernel.dispatch_moe_fp8blk(xq, xs, logits, None, w13q, w13s, w2q, w2s, y,
                                                                  k, G, KG, 2.5, ws), [y],
                        scratch_fn=lambda: ws.fill_(0xA5))

