"""Times every tile kernel of one GEMM format against the kernel the library picks, on a grid of shapes,
and writes the per-shape table that the library's choice of tile consults.

    python -m hipkittens_amd.tile_sweep fp8|bf16|mxfp4            report on the 110-shape grid
    python -m hipkittens_amd.tile_sweep fp8|bf16|mxfp4 --emit     sweep the larger grid, rewrite the format's
                                                                  entries of csrc/tile_table.inc, then rebuild

For each shape it prints the GPU time (a HIP graph of 20 launches between two events, the launches rotating
over copies of B that exceed the memory-side cache, as a model's weights do; best of three replays, in two passes over the kernels, forwards and backwards) of the default choice (variant -1; with at
most 64 rows of A that can be the skinny kernel, csrc/gemm_skinny.h, instead of a tile kernel), of the 256x256,
128x128 and 64x64 tile kernels, and of the call with a workspace where the library would split K without the
skinny kernel, and marks the shapes where the default is more than 5 % behind the best tile kernel.

The choice of tile (`pick_tile`, csrc/gemm_small_tile.h) is a rule plus a generated table of exceptions,
the counterpart of the reference's tuned.yaml (analysis/baselines/gemm/utils/tuned.yaml: one tuned solution
per shape). `--emit` measures the three tile kernels on every shape of the larger grid and records the
shapes where the rule's choice (`hk_gemm_tile_choice(..., consult_table=0)`) is more than 3 % slower than
the fastest tile, keyed as the library looks them up: format, ceil(M / 64), ceil(N / 64), K-steps. The
table applies on devices with the CU count it was measured on; run it again after changing a tile kernel
or on another device, and rebuild the library.
"""
import re
import sys
from pathlib import Path

import torch

from . import _lib
from . import tk_kernel as tk

M_GRID = (16, 128, 256, 512, 768, 1024, 1536, 2048, 3072, 4096, 8192)
NK_GRID = ((1024, 1024), (2048, 2048), (4096, 4096), (8192, 8192), (4096, 14336), (14336, 4096),
           (2880, 2880), (7168, 2048), (2048, 7168), (5120, 5120))
# the grid of --emit: the report's grid and the shapes between its points
M_GRID_EMIT = (16, 64, 128, 192, 256, 384, 512, 640, 768, 1024, 1280, 1536, 2048, 2560, 3072, 4096, 6144, 8192)
NK_GRID_EMIT = NK_GRID + ((1536, 1536), (3072, 3072), (6144, 6144), (5760, 2880), (2880, 5760), (4096, 7168),
                          (7168, 4096), (1024, 8192), (8192, 1024), (2560, 10240),
                          (28672, 4096), (32768, 8192), (65536, 2880))   # (wide outputs: vocabulary projections)
FORMATS = {"fp8": 0, "bf16": 1, "mxfp4": 2}
TABLE_PATH = Path(__file__).resolve().parent / "csrc" / "tile_table.inc"
EMIT_MARGIN = 1.03


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


# B is the weight matrix of a layer: in a model it comes from HBM every time, because between two uses of it the
# other layers' weights have passed through the 256 MB memory-side cache. Timing one and the same B again and again
# would find it in that cache whenever it fits, and would tune the choice of tile for a case that does not occur.
# The calls therefore rotate over copies of B that together exceed the cache more than four times (A, the
# activations, stays).
ROTATE_BYTES = 1.2e9
ROTATE_MAX = 32


def _copies(b_bytes):
    return 1 if b_bytes >= 256e6 else min(ROTATE_MAX, int(ROTATE_BYTES // b_bytes) + 1)


def _problem(fmt, M, N, K, dev):
    C = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    turn = [0]

    def rotating(items):
        def nxt():
            turn[0] = (turn[0] + 1) % len(items)
            return items[turn[0]]
        return nxt

    if fmt == "fp8":
        A = torch.randn(M, K, device=dev).to(torch.float8_e4m3fn)
        B = rotating([torch.randn(N, K, device=dev).to(torch.float8_e4m3fn) for _ in range(_copies(N * K))])
        return (lambda v, ws=None: tk.dispatch_fp8_gemm(A, B(), C, 1.0, 1.0, variant=v, workspace=ws),
                tk.fp8_gemm_workspace_bytes(M, N, K))
    if fmt == "bf16":
        A = torch.randn(M, K, device=dev, dtype=torch.bfloat16)
        B = rotating([torch.randn(N, K, device=dev, dtype=torch.bfloat16) for _ in range(_copies(2 * N * K))])
        return (lambda v, ws=None: tk.dispatch_bf16_gemm(A, B(), C, variant=v, workspace=ws),
                tk.bf16_gemm_workspace_bytes(M, N, K))
    A = torch.randint(0, 256, (M, K // 2), dtype=torch.uint8, device=dev)
    As = torch.randint(120, 130, (M, K // 32), dtype=torch.uint8, device=dev)
    B = rotating([(torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device=dev),
                   torch.randint(120, 130, (N, K // 32), dtype=torch.uint8, device=dev))
                  for _ in range(_copies(N * (K // 2 + K // 32)))])

    def run(v, ws=None):
        b, bs = B()
        tk.dispatch_mxfp4_gemm(A, As, b, bs, C, variant=v, workspace=ws)

    return run, tk.mxfp4_gemm_workspace_bytes(M, N, K)


def _k_steps(fmt, K):
    row_bytes = {"fp8": K, "bf16": 2 * K, "mxfp4": K // 2}[fmt]
    return (row_bytes + 127) // 128


def _write_table(fmt, entries, cus):
    """Replaces the entries of `fmt` in csrc/tile_table.inc; the other formats' entries stay."""
    code = FORMATS[fmt]
    kept = []
    for m in re.finditer(r"\{(\d+), (\d+), (\d+), (\d+), (\d+)\},", TABLE_PATH.read_text()):
        e = tuple(int(x) for x in m.groups())
        if e[0] != code and e[0] != 255:
            kept.append(e)
    rows = sorted(set(kept) | {(code,) + e for e in entries})
    lines = [
        "// Generated by `python -m hipkittens_amd.tile_sweep FORMAT --emit` (one run per format; each run rewrites its",
        "// format's entries). Shapes on which the rule of pick_tile (gemm_small_tile.h) was measured more than 3 % behind",
        "// another tile kernel: {format, ceil(M / 64), ceil(N / 64), K-steps, tile}.",
        f"constexpr int kTileTableCus = {cus};   // CU count of the device the sweeps ran on",
        "static const TileTableEntry kTileTable[] = {",
        "    {255, 0, 0, 0, 0},   // (keeps the array non-empty)",
    ]
    lines += [f"    {{{e[0]}, {e[1]}, {e[2]}, {e[3]}, {e[4]}}}," for e in rows]
    lines.append("};")
    TABLE_PATH.write_text("\n".join(lines) + "\n")
    return len(rows)


def main(argv):
    args = [a for a in argv[1:] if not a.startswith("--")]
    flags = [a for a in argv[1:] if a.startswith("--")]
    if len(args) != 1 or args[0] not in FORMATS or any(f != "--emit" for f in flags):
        print(__doc__)
        return 2
    if not torch.cuda.is_available():
        raise RuntimeError("tile_sweep needs a GPU")
    fmt, dev, emit = args[0], "cuda:0", "--emit" in flags
    lib = _lib.load_library()
    tiles = {"fp8": (4, 5, 6), "bf16": (1, 2, 3), "mxfp4": (1, 2, 3)}[fmt]   # 256, 128, 64
    size_of = dict(zip(tiles, (256, 128, 64)))
    behind = total = 0
    entries = set()
    for M in (M_GRID_EMIT if emit else M_GRID):
        for N, K in (NK_GRID_EMIT if emit else NK_GRID):
            run, ws_bytes = _problem(fmt, M, N, K, dev)
            # every kernel is timed in two passes, the second in reverse order, and the faster one counts: single
            # timings of one and the same kernel differ by 2-6 % with their position in the sequence (cold operands
            # first, a warm chip last)
            order = tiles + ((-1,) if not emit else ())
            t = {v: _time_us(lambda: run(v)) for v in order}
            for v in reversed(order):
                t[v] = min(t[v], _time_us(lambda: run(v)))
            best_v = min(tiles, key=lambda v: t[v])
            if emit:
                rule = int(lib.hk_gemm_tile_choice(FORMATS[fmt], M, N, K, 0))
                t_rule = t[[v for v in tiles if size_of[v] == rule][0]]
                line = (f"M={M} N={N} K={K}: rule {rule} {t_rule:.1f} us | 256x256 {t[tiles[0]]:.1f}  128x128 "
                        f"{t[tiles[1]]:.1f}  64x64 {t[tiles[2]]:.1f}")
                if t_rule > EMIT_MARGIN * t[best_v]:
                    entries.add(((M + 63) // 64, (N + 63) // 64, _k_steps(fmt, K), size_of[best_v]))
                    line += f"  -> table: {size_of[best_v]}"
                print(line, flush=True)
                continue
            line = (f"M={M} N={N} K={K}: default {t[-1]:.1f} us | 256x256 {t[tiles[0]]:.1f}  128x128 "
                    f"{t[tiles[1]]:.1f}  64x64 {t[tiles[2]]:.1f}")
            if ws_bytes:
                ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
                line += f" | split-K {_time_us(lambda: run(-1, ws)):.1f}"
            total += 1
            if t[-1] > 1.05 * t[best_v]:
                behind += 1
                line += "  <-- default more than 5 % behind"
            print(line, flush=True)
    if emit:
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        n = _write_table(fmt, entries, cus)
        print(f"{len(entries)} entries for {fmt}; {TABLE_PATH} now holds {n}: rebuild the library "
              f"(python -m hipkittens_amd.build)")
    else:
        print(f"default more than 5 % behind the best tile kernel on {behind} of {total} shapes")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
