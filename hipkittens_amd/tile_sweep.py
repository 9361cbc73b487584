"""Times every tile kernel of one GEMM format against the kernel the library picks, on a grid of shapes.

    python -m hipkittens_amd.tile_sweep fp8|bf16|mxfp4

For each shape it prints the GPU time (a HIP graph of 20 launches between two events, best of three
replays) of the default choice (variant -1), of the 256x256, 128x128 and 64x64 tile kernels, and of the
split-K path where the library would use one, and marks the shapes where the default is more than 5 %
behind the best tile kernel. The thresholds of `pick_tile` (csrc/gemm_small_tile.h) were set from
this output on an MI355X; run it again after changing a tile kernel or on another device.
"""
import sys

import torch

from . import tk_kernel as tk

M_GRID = (16, 128, 256, 512, 768, 1024, 1536, 2048, 3072, 4096, 8192)
NK_GRID = ((1024, 1024), (2048, 2048), (4096, 4096), (8192, 8192), (4096, 14336), (14336, 4096),
           (2880, 2880), (7168, 2048), (2048, 7168), (5120, 5120))


def _time_us(fn, iters=20):
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        fn()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(iters):
                fn()
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) / iters)
    return best * 1000.0


def _problem(fmt, M, N, K, dev):
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    if fmt == "fp8":
        A = torch.randn(M, K, device=dev).to(torch.float8_e4m3fn)
        B = torch.randn(N, K, device=dev).to(torch.float8_e4m3fn)
        return (lambda v, ws=None: tk.dispatch_fp8_gemm(A, B, C, 1.0, 1.0, variant=v, workspace=ws),
                tk.fp8_gemm_workspace_bytes(M, N, K))
    if fmt == "bf16":
        A = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
        B = torch.randn(N, K, device=dev, dtype=torch.bfloat16)
        return (lambda v, ws=None: tk.dispatch_bf16_gemm(A, B, C, variant=v, workspace=ws),
                tk.bf16_gemm_workspace_bytes(M, N, K))
    A = torch.randint(0, 256, (M, K // 2), dtype=torch.uint8, device=dev)
    B = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device=dev)
    As = torch.randint(120, 130, (M, K // 32), dtype=torch.uint8, device=dev)
    Bs = torch.randint(120, 130, (N, K // 32), dtype=torch.uint8, device=dev)
    return (lambda v, ws=None: tk.dispatch_mxfp4_gemm(A, As, B, Bs, C, variant=v, workspace=ws),
            tk.mxfp4_gemm_workspace_bytes(M, N, K))


def main(argv):
    if len(argv) != 2 or argv[1] not in ("fp8", "bf16", "mxfp4"):
        print(__doc__)
        return 2
    if not torch.cuda.is_available():
        raise RuntimeError("tile_sweep needs a GPU")
    fmt, dev = argv[1], "cuda:0"
    tiles = {"fp8": (4, 5, 6), "bf16": (1, 2, 3), "mxfp4": (1, 2, 3)}[fmt]   # 256, 128, 64
    behind = total = 0
    for M in M_GRID:
        for N, K in NK_GRID:
            if fmt == "mxfp4":
                K = (K + 255) // 256 * 256
            run, ws_bytes = _problem(fmt, M, N, K, dev)
            t = {v: _time_us(lambda: run(v)) for v in (-1,) + tiles}
            line = (f"M={M} N={N} K={K}: default {t[-1]:.1f} us | 256x256 {t[tiles[0]]:.1f}  128x128 "
                    f"{t[tiles[1]]:.1f}  64x64 {t[tiles[2]]:.1f}")
            if ws_bytes:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
                line += f" | split-K {_time_us(lambda: run(-1, ws)):.1f}"
            best = min(t[v] for v in tiles)
            total += 1
            if t[-1] > 1.05 * best:
                behind += 1
                line += "  <-- default more than 5 % behind"
            print(line, flush=True)
    print(f"default more than 5 % behind the best tile kernel on {behind} of {total} shapes")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
