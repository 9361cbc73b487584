"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol declared in
include/hk355.h, and rejects bad arguments with the documented status codes before anything
touches a GPU. The Python shim's checks mirror the reference's binding
(include/pyutils/pyutils.cuh:14-47: Tensor, contiguous, not on the CPU) and raise RuntimeError."""
import ctypes
import os
import re

import pytest
import torch

import hipkittens_amd as hk
from hipkittens_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hk355.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = hk.load_library()
    names = _declared_symbols()
    assert "hk_fp8_gemm" in names and "hk_mxfp4_gemm" in names and "hk_moe_sort" in names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/hk355.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert lib.hk_version() >= 100
    assert lib.hk_status_string(0) == b"ok" and lib.hk_status_string(-2) == b"bad shape"


def test_product_library_exports_nothing_but_the_declared_abi():
    """Every exported hk* function is declared in include/hk355.h: bench-only tooling (the MFMA rate
    probe) lives in a library of its own and is not part of the product's ABI."""
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", str(_lib.lib_path())], capture_output=True, text=True,
                         check=True).stdout
    exported = sorted({ln.split()[-1] for ln in out.splitlines() if " T " in ln and ln.split()[-1].startswith("hk")})
    assert exported == _declared_symbols()


def test_c_entry_points_reject_bad_arguments_without_a_gpu():
    lib = hk.load_library()
    buf = ctypes.create_string_buffer(4096 + 64)
    p = (ctypes.addressof(buf) + 63) & ~63  # aligned host pointer; never dereferenced on this path
    assert lib.hk_fp8_gemm(None, p, p, 256, 256, 256, 1.0, 1.0, None) == -1
    assert lib.hk_fp8_gemm(p, p, p, 0, 256, 256, 1.0, 1.0, None) == -2
    assert lib.hk_fp8_gemm(p, p, p, 256, 256, 250, 1.0, 1.0, None) == -2      # K % 16
    assert lib.hk_fp8_gemm(p + 1, p, p, 256, 256, 256, 1.0, 1.0, None) == -3
    assert lib.hk_fp8_gemm_variant(p, p, p, 256, 256, 256, 1.0, 1.0, 2, None) == -6  # a variant that no longer exists
    assert lib.hk_fp8_gemm_variant(p, p, p, 256, 256, 256, 1.0, 1.0, 9, None) == -6
    assert lib.hk_mxfp4_gemm(p, None, p, p, p, 64, 64, 64, None) == -1
    assert lib.hk_mxfp4_gemm(p, p, p, p, p, 64, 64, 48, None) == -2           # K % 32
    assert lib.hk_mxfp4_gemm_variant(p, p, p, p, p, 64, 64, 64, 1, None) == -2  # K % 256 for the tile kernel
    assert lib.hk_moe_topk_softmax(p, 4, 1024, 2, p, p, None) == -2           # E > 512
    assert lib.hk_moe_topk_softmax(p, 4, 16, 17, p, p, None) == -2            # k > E
    assert lib.hk_moe_topk_grouped_sigmoid(p, None, 4, 30, 2, 4, 2, 1.0, p, p, None) == -2
    assert lib.hk_moe_sort(p, 4, 2, 8, p, p, None, None, 0, None) == -4       # no workspace
    assert lib.hk_moe_sort(p, 4, 2, 8, p, p, None, p, 4, None) == -4          # workspace too small
    assert lib.hk_moe_sort_workspace_bytes(4096, 4, 128) == 17 * 128 * 4
    # split-K entry point: the same argument checks; the workspace is optional
    assert lib.hk_fp8_gemm_ws(p, p, p, 0, 256, 256, 1.0, 1.0, None, 0, None) == -2
    assert lib.hk_fp8_gemm_ws(None, p, p, 16, 4096, 4096, 1.0, 1.0, p, 1 << 40, None) == -1
    assert lib.hk_fp8_gemm_ws(p, p, p, 16, 4096, 4090, 1.0, 1.0, p, 1 << 40, None) == -2
    assert lib.hk_fp8_gemm_workspace_bytes(8192, 8192, 8192) == 0
    assert lib.hk_fp8_gemm_workspace_bytes(16, 8192, 8192) % (16 * 8192 * 4) == 0
    assert lib.hk_fp8_gemm_workspace_bytes(16, 8192, 8192) > 0
    assert lib.hk_bf16_gemm(p, p, p, 64, 64, 60, None) == -2                  # K % 8
    assert lib.hk_bf16_gemm_ws(p, p, p, 16, 1024, 4092, p, 1 << 40, None) == -2          # K % 8, split path
    assert lib.hk_bf16_gemm_ws(p, p, p, 0, 256, 256, None, 0, None) == -2
    assert lib.hk_bf16_gemm_workspace_bytes(8192, 8192, 8192) == 0
    assert lib.hk_bf16_gemm_workspace_bytes(16, 8192, 4096) == lib.hk_fp8_gemm_workspace_bytes(16, 8192, 8192)
    assert lib.hk_mxfp4_gemm_pitched(p, p, 88, p, p, 96, p, 64, 64, 2880, None) == -2    # pitch < K / 32
    assert lib.hk_mxfp4_gemm_pitched(p, None, 96, p, p, 96, p, 64, 64, 2880, None) == -1
    assert lib.hk_mxfp4_gemm_pitched(p, p, 96, p, p, 96, p, 64, 64, 2872, None) == -2    # K % 32
    assert lib.hk_mxfp4_gemm_ws(p, p, 256, p, p, 256, p, 0, 64, 8192, None, 0, None) == -2
    assert lib.hk_mxfp4_gemm_ws(p, p, 256, p, p, 256, p, 16, 1024, 8176, p, 1 << 40, None) == -2     # K % 32
    assert lib.hk_mxfp4_gemm_ws(None, p, 256, p, p, 256, p, 16, 1024, 8192, p, 1 << 40, None) == -1  # split path
    assert lib.hk_mxfp4_gemm_ws(p, p, 256, p, p, 256, p, 16, 1024, 8192, p + 4, 1 << 40, None) == -3
    assert lib.hk_mxfp4_gemm_ws(p, p, 255, p, p, 256, p, 16, 1024, 8192, p, 1 << 40, None) == -2     # pitch < K / 32
    assert lib.hk_mxfp4_gemm_workspace_bytes(16, 1024, 8192) % (16 * 1024 * 4) == 0
    assert lib.hk_mxfp4_gemm_workspace_bytes(16, 1024, 8192) > 0
    assert lib.hk_mxfp4_gemm_workspace_bytes(8192, 8192, 8192) == 0
    # dimensions beyond the launchers' 32-bit arithmetic are refused before anything is computed from them
    imax = 2**31 - 1
    for M, N, K in ((imax, 64, 128), (64, imax, 128), (64, 64, imax - 15), (1 << 24, 1 << 24, 128)):
        assert lib.hk_fp8_gemm(p, p, p, M, N, K & ~15, 1.0, 1.0, None) == -2
        assert lib.hk_fp8_gemm_ws(p, p, p, M, N, K & ~15, 1.0, 1.0, p, 1 << 40, None) == -2
        assert lib.hk_fp8_gemm_static_ws(p, p, p, M, N, K & ~15, 1.0, 1.0, None) == -2
        assert lib.hk_bf16_gemm(p, p, p, M, N, K & ~7, None) == -2
        assert lib.hk_bf16_gemm_ws(p, p, p, M, N, K & ~7, p, 1 << 40, None) == -2
        assert lib.hk_mxfp4_gemm(p, p, p, p, p, M, N, K & ~31, None) == -2
        assert lib.hk_fp8_gemm_workspace_bytes(M, N, K) == 0
        assert lib.hk_bf16_gemm_workspace_bytes(M, N, K) == 0
        assert lib.hk_mxfp4_gemm_workspace_bytes(M, N, K) == 0
    assert lib.hk_moe_mxfp4_workspace_bytes(16, 64, 32, imax, 2) == 0       # shapes the entry points refuse
    assert lib.hk_moe_mxfp4_workspace_bytes(16, 64, 32, 4, 8) == 0          # k > E
    assert lib.hk_moe_fp8blk_workspace_bytes(16, 128, 128, 513, 2) == 0
    assert lib.hk_moe_topk_softmax(p, imax, 128, 4, p, p, None) == -2
    assert lib.hk_moe_sort(p, imax, 8, 128, p, p, None, p, 1 << 40, None) == -2
    # extended MoE entry points: option checks come before anything touches memory
    args = (p, p, p, 8, p, p, 8, p, p, p, p, p, 16, 64, 32, 4, 2, 0)
    assert lib.hk_moe_mxfp4_experts_ex(*args, None, None, 7, 1.702, 7.0, 0, p, 1 << 30, None) == -6   # activation
    assert lib.hk_moe_mxfp4_experts_ex(*args, None, None, 1, 1.702, 0.0, 0, p, 1 << 30, None) == -2   # limit <= 0
    assert lib.hk_moe_mxfp4_experts_ex(*args, p + 4, None, 0, 0.0, 0.0, 0, p, 1 << 30, None) == -3    # bias alignment
    assert lib.hk_moe_mxfp4_experts_ex(*args, None, None, 0, 0.0, 0.0, 0, None, 0, None) == -4        # workspace
    # a bias array of 4 GiB or more cannot be addressed by the kernels' 32-bit offsets (512 x 2 x 2^20 floats)
    huge = (p, p, p, 8, p, p, 32768, p, p, p, p, p, 1, 32, 1 << 20, 512, 1, 0)
    assert lib.hk_moe_mxfp4_experts_ex(*huge, p, None, 0, 0.0, 0.0, 0, p, 1 << 40, None) == -2
    # MXFP8-activation entry points (pre-shuffled weights only): same option and workspace checks
    a8 = (p, p, p, p, p, p, p, p, p, p, 16, 64, 32, 4, 2)
    assert lib.hk_moe_mxfp4_a8_experts(*a8, None, None, 7, 1.702, 7.0, 0, p, 1 << 30, None) == -6
    assert lib.hk_moe_mxfp4_a8_experts(*a8, None, None, 0, 0.0, 0.0, 0, None, 0, None) == -4
    assert lib.hk_moe_mxfp4_a8_experts(None, *a8[1:], None, None, 0, 0.0, 0.0, 0, p, 1 << 30, None) == -1
    assert lib.hk_moe_mxfp4_a8_experts(*a8[:10], 16, 60, 32, 4, 2, None, None, 0, 0.0, 0.0, 0, p, 1 << 30, None) == -2  # H % 32
    assert lib.hk_moe_mxfp4_a8_forward(p, None, p, p, p, p, p, 16, 64, 32, 4, 2, None, None, 0, 0.0, 0.0, 0, p, 1 << 30, None) == -1
    # 1 M rows x 2880: the MXFP4 tiles fit 32-bit offsets, the MXFP8 ones do not
    big = (p, p, p, p, p, p, p, p, p, p, 250000, 2880, 2880, 128, 4)
    assert lib.hk_moe_mxfp4_a8_experts(*big, None, None, 0, 0.0, 0.0, 0, p, 1 << 50, None) == -2
    assert lib.hk_moe_mxfp4_a8_workspace_bytes(16, 64, 32, 4, 2) > lib.hk_moe_mxfp4_workspace_bytes(16, 64, 32, 4, 2)
    assert lib.hk_moe_mxfp4_a8_workspace_bytes(0, 64, 32, 4, 2) == 0
    # a layer of one token: its regions, each rounded up to 256 bytes, and nothing behind them
    assert 1 * 32 * 2 <= lib.hk_moe_mxfp4_workspace_bytes(1, 32, 32, 1, 1) < 16384
    assert 1 * 128 * 2 <= lib.hk_moe_fp8blk_workspace_bytes(1, 128, 128, 1, 1) < 16384
    assert lib.hk_mxfp8_quantize_rows(p, 4, 48, p, p, 8, None) == -2          # cols % 32
    assert lib.hk_mxfp8_quantize_rows(p, 4, 64, None, p, 8, None) == -1
    assert lib.hk_mxfp8_quantize_rows(p, 4, 64, p, p, 4, None) == -2          # scale pitch % 8
    assert lib.hk_moe_unpermute_add(p, p, p, 4, 2, 60, None, p, None) == -2                            # H % 8
    assert lib.hk_moe_unpermute_add(p, p, p, 4, 2, 64, p + 2, p, None) == -3


def test_python_boundary_rejects_like_the_reference():
    A = torch.zeros((256, 256), dtype=torch.uint8)
    C = torch.zeros((256, 256), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        hk.tk_kernel.dispatch_fp8_gemm(A, A, C)                 # CPU tensors
    with pytest.raises(RuntimeError, match="contiguous"):
        hk.tk_kernel.dispatch_fp8_gemm(A.t(), A, C)
    with pytest.raises(RuntimeError, match="Tensor"):
        hk.tk_kernel.dispatch_fp8_gemm([1, 2], A, C)
    with pytest.raises(RuntimeError, match="GPU"):
        hk.tk_kernel.dispatch_micro(A, A, C)


def test_device_independent_quantizers_match_oracle_on_cpu():
    import numpy as np

    from oracle import formats as F

    rng = np.random.default_rng(0)
    x = (rng.standard_normal((64, 256)) * np.exp2(rng.integers(-10, 10, size=(64, 1)))).astype(np.float32)
    p, s = hk.quant.quantize_mxfp4(torch.from_numpy(x))
    po, so = F.quantize_mxfp4(x)
    assert np.array_equal(p.numpy(), po) and np.array_equal(s.numpy(), so)
    q, sc = hk.quant.quantize_fp8_per_tensor(torch.from_numpy(x))
    qo, sco = F.quantize_e4m3_per_tensor(x)
    assert np.float32(sc) == sco and np.array_equal(q.view(torch.uint8).numpy(), qo)


def test_tile_choice_rule_and_generated_table():
    """The choice of GEMM tile (no GPU needed: without a device the library assumes 256 CUs, the count the
    committed table was measured on): the rule's landmarks (rounds of workgroups over the CUs times a cost per
    round), and every entry of csrc/tile_table.inc is what the default entry points would pick for a shape with
    the entry's key."""
    tk = hk.tk_kernel
    for fmt in ("fp8", "bf16", "mxfp4"):
        assert tk.gemm_tile_choice(fmt, 8192, 8192, 8192, False) == 256     # 1024 large tiles: four full rounds
        assert tk.gemm_tile_choice(fmt, 1024, 1024, 1024, False) == 64      # one round with any tile: the cheapest
        assert tk.gemm_tile_choice(fmt, 2048, 4096, 1024, False) == 128     # 128 large tiles, short K
        assert tk.gemm_tile_choice(fmt, 16, 8192, 8192, False) == 64
        # 64 large tiles = one round of 256 small ones doing a quarter of the work each
        assert tk.gemm_tile_choice(fmt, 1024, 4096, 4096, False) == 128
    # 72 / 80 large tiles are one round where their 288 / 320 tiles of 128 x 128 are two: the large tile from a
    # long K on (MXFP4, whose 64 x 64 kernel costs more per K-step, already here)
    assert tk.gemm_tile_choice("mxfp4", 768, 6144, 6144, False) == 256
    assert tk.gemm_tile_choice("mxfp4", 2048, 2560, 16384, False) == 256
    assert tk.gemm_tile_choice("fp8", 2048, 2560, 16384, False) in (256, 64)
    assert tk.gemm_tile_choice("fp8", 2048, 2560, 16384, False) != 128
    with pytest.raises(RuntimeError):
        tk.gemm_tile_choice("fp8", 0, 8, 8)
    text = open(os.path.join(ROOT, "hipkittens_amd", "csrc", "tile_table.inc")).read()
    assert re.search(r"kTileTableCus = 256;", text)
    entries = [tuple(int(x) for x in m.groups()) for m in re.finditer(r"\{(\d+), (\d+), (\d+), (\d+), (\d+)\},", text)]
    entries = [e for e in entries if e[0] != 255]
    assert entries and len(set(e[:4] for e in entries)) == len(entries)     # one tile per key
    k_per_step = {0: 128, 1: 64, 2: 256}
    for code, m64, n64, nk, tile in entries:
        assert tile in (256, 128, 64)
        fmt = ("fp8", "bf16", "mxfp4")[code]
        M, N, K = 64 * m64 - 5, 64 * n64, nk * k_per_step[code]
        assert tk.gemm_tile_choice(fmt, M, N, K) == tile
        assert tk.gemm_tile_choice(fmt, M, N, K, False) != tile             # an entry that repeats the rule is noise
