"""The split-K FP8 GEMM entry point that allocates nothing (hk_fp8_gemm_static_ws: partial sums in a
device array inside the library) against hk_fp8_gemm_ws with a caller workspace, through the C ABI
(ctypes on libhk355.so): identical bits, on calls in a row that share the array, the later ones
smaller than the first, with device memory unchanged across the calls; and the same calls recorded
under HIP graph capture (where an allocation inside the library would fail the capture), replayed
against the oracle-tested sibling's bits."""
import ctypes

import numpy as np
import pytest
import torch

from hipkittens_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _operands(M, N, K, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    A = torch.randn(M, K, device=DEV, generator=g).to(torch.float8_e4m3fn)
    B = torch.randn(N, K, device=DEV, generator=g).to(torch.float8_e4m3fn)
    return A, B


def test_fp8_gemm_static_ws_matches_caller_workspace_entry_point():
    lib = _lib.load_library()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    cap = lib.hk_fp8_gemm_static_ws_max_bytes()
    assert cap == 8 << 20
    # first the largest split-K shape (fills the array), then smaller ones (the third and fourth run on the skinny
    # kernel, which needs no partial sums), then one that is not split
    shapes = [(128, 4096, 8192), (100, 520, 6160), (16, 1024, 8192), (1, 128, 8192), (512, 512, 512)]
    cases = []
    for i, (M, N, K) in enumerate(shapes):   # all tensors exist before the first call
        A, B = _operands(M, N, K, 10 + i)
        need = lib.hk_fp8_gemm_workspace_bytes(M, N, K)
        assert need <= cap
        ws = torch.full((max(need, 16),), 0xFF, dtype=torch.uint8, device=DEV)
        want = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        cases.append((M, N, K, A, B, ws, need, want, got))
    assert cases[0][6] == cap and cases[1][6] > 0 and cases[-1][6] == 0
    for (M, N, K, A, B, ws, need, want, got) in cases:
        rc = lib.hk_fp8_gemm_ws(A.data_ptr(), B.data_ptr(), want.data_ptr(), M, N, K, 0.5, 2.0, ws.data_ptr(),
                                ws.numel(), stream)
        assert rc == 0
    torch.cuda.synchronize()
    # set-up call (looks the array's address up on this device), then nothing may be allocated
    M, N, K, A, B, ws, need, want, got = cases[1]
    assert lib.hk_fp8_gemm_static_ws(A.data_ptr(), B.data_ptr(), got.data_ptr(), M, N, K, 0.5, 2.0, stream) == 0
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    for (M, N, K, A, B, ws, need, want, got) in cases:
        print(f"static_ws M={M} N={N} K={K} need={need}", flush=True)
        rc = lib.hk_fp8_gemm_static_ws(A.data_ptr(), B.data_ptr(), got.data_ptr(), M, N, K, 0.5, 2.0, stream)
        assert rc == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0, "device memory changed across calls that must not allocate"
    for (M, N, K, A, B, ws, need, want, got) in cases:
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, N, K)
    # the same argument checks as the entry point it is a variant of
    a, b, c = cases[1][3], cases[1][4], cases[1][8]
    assert lib.hk_fp8_gemm_static_ws(None, b.data_ptr(), c.data_ptr(), 16, 1024, 8192, 1.0, 1.0, stream) == -1
    assert lib.hk_fp8_gemm_static_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), 0, 1024, 8192, 1.0, 1.0, stream) == -2
    assert lib.hk_fp8_gemm_static_ws(a.data_ptr(), b.data_ptr(), c.data_ptr(), 16, 1024, 8190, 1.0, 1.0, stream) == -2


def test_fp8_gemm_static_ws_records_into_a_graph():
    """Stream capture refuses hipMalloc / hipFree: a capture of the entry point that succeeds shows that the
    call path allocates nothing. Replays (with eager work of the program that dirties the shared array in
    between) must reproduce hk_fp8_gemm_ws's bits, the second call of the graph on a smaller shape."""
    lib = _lib.load_library()
    shapes = [(128, 2048, 8192), (100, 520, 6160)]
    cases = []
    for i, (M, N, K) in enumerate(shapes):
        A, B = _operands(M, N, K, 30 + i)
        need = lib.hk_fp8_gemm_workspace_bytes(M, N, K)
        assert 0 < need <= lib.hk_fp8_gemm_static_ws_max_bytes()
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        want = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        got = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        rc = lib.hk_fp8_gemm_ws(A.data_ptr(), B.data_ptr(), want.data_ptr(), M, N, K, 0.5, 2.0, ws.data_ptr(), ws.numel(),
                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0
        cases.append((M, N, K, A, B, want, got))
    # set-up call outside the capture (the per-device address look-up happens on a device's first call)
    M, N, K, A, B, want, got = cases[1]
    assert lib.hk_fp8_gemm_static_ws(A.data_ptr(), B.data_ptr(), got.data_ptr(), M, N, K, 0.5, 2.0,
                                     ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        for (M, N, K, A, B, want, got) in cases:
            assert lib.hk_fp8_gemm_static_ws(A.data_ptr(), B.data_ptr(), got.data_ptr(), M, N, K, 0.5, 2.0, stream) == 0
    big = _operands(128, 4096, 8192, 99)
    sink = torch.empty((128, 4096), dtype=torch.bfloat16, device=DEV)
    for rep in range(3):
        for c in cases:
            c[6].fill_(float("nan"))
        # an eager call on the largest shape overwrites the whole shared array between the replays
        assert lib.hk_fp8_gemm_static_ws(big[0].data_ptr(), big[1].data_ptr(), sink.data_ptr(), 128, 4096, 8192, 1.0, 1.0,
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)) == 0
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for (M, N, K, A, B, want, got) in cases:
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (rep, M, N, K)
