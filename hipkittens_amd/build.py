"""Build libhk355.so (the C-ABI library) from hipkittens_amd/csrc/*.hip with hipcc for gfx950.

Each .hip file is compiled to an object in parallel and the objects are linked
into one shared library that sits next to this file, so that it travels with the
source tree.
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
BUILD_DIR = PKG_DIR / "csrc" / "build"
LIB_PATH = PKG_DIR / "libhk355.so"
# bench-only tooling (csrc/bench/*.hip: a register-only MFMA rate probe). A library of its own so that
# nothing of it is exported by, or linked into, the product library; only bench.py loads it.
BENCH_LIB_PATH = PKG_DIR / "libhk355_bench.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",
    # packed-fp32 VALU forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# Files whose arithmetic is specified operation by operation (bit-exact against the CPU oracle)
# are built without fused multiply-add contraction.
PER_FILE_FLAGS = {
    "moe_routing.hip": ["-ffp-contract=off"],
}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; cannot build libhk355.so")
    return exe


def _compile_one(src: Path, extra: list[str]) -> Path:
    obj = BUILD_DIR / (("bench_" if src.parent.name == "bench" else "") + src.stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_FILE_FLAGS.get(src.name, []), *extra, "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stdout}\n{res.stderr}")
    return obj


def build(verbose: bool = True, extra_flags: list[str] | None = None, jobs: int = 8, check: bool = True) -> Path:
    """Compile every csrc/*.hip and link libhk355.so. Always recompiles.

    check: also scan the kernels' assembly for the wait states the compiler does not provide around
    inline assembly (isa_check) and refuse a library with findings: a kernel whose register allocation
    puts a spill restore next to a hand-written load reads from a wild address on the GPU."""
    extra = list(extra_flags or [])
    BUILD_DIR.mkdir(parents=True, exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    bench_sources = sorted((CSRC / "bench").glob("*.hip"))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        all_objs = list(pool.map(lambda s: _compile_one(s, extra), sources + bench_sources))
    objs, bench_objs = all_objs[:len(sources)], all_objs[len(sources):]
    _link(objs, LIB_PATH)
    if bench_objs:
        _link(bench_objs, BENCH_LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} from {len(sources)} sources", file=sys.stderr)
    if check and not extra:
        from . import isa_check

        findings = isa_check.check_sources(sources + bench_sources, jobs=jobs)
        if findings:
            LIB_PATH.unlink(missing_ok=True)
            raise RuntimeError("isa_check: the built kernels break wait-state rules around inline assembly; "
                               "library removed:\n" + "\n".join(str(f) for f in findings))
        if verbose:
            print("isa_check: 0 findings", file=sys.stderr)
    return LIB_PATH


def _link(objs: list[Path], out: Path) -> None:
    tmp = out.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link of {out.name} failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, out)


if __name__ == "__main__":
    build(check="--no-check" not in sys.argv[1:])
