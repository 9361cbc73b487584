"""Host logic of bench.py and tile_sweep.py that needs no GPU: the refusal of more than one GPU, the
collection of the traffic figures from rocprofv3 counter files, every bench leg's traffic coming from the one
tracked file, and the rewriting of one format's entries in the generated tile table."""
import csv
import importlib.util
import json
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def _load_bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode == 2
    assert "exactly one GPU" in res.stderr and res.stdout.strip() == ""


def _write_run(root, run, counter, rows):
    d = root / f"{run}_{counter}" / "host" / "x"
    d.mkdir(parents=True)
    with open(d / "123_counter_collection.csv", "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["Kernel_Name", "Counter_Name", "Counter_Value"])
        w.writeheader()
        for kernel, value in rows:
            w.writerow({"Kernel_Name": kernel, "Counter_Name": counter, "Counter_Value": value})


def test_collect_traffic_scales_by_the_calibration_copy(tmp_path, monkeypatch):
    bench = _load_bench()
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(tmp_path / "traffic.json"))
    monkeypatch.setattr(bench, "TRAFFIC_LEGS", {"fp8_gemm_8192": ("calibration", ["fp8_gemm_4wave_ring_kernel<false>"]),
                                                "toy": ("toy", ["toy_kernel<1>", "other_kernel"])})
    full = "void hk::fp8_gemm_4wave_ring_kernel<false>(unsigned char const*, int)"
    # FETCH_SIZE reads half of the KiB moved (factor 2), WRITE_SIZE all of them (factor 1); small copies ride along
    _write_run(tmp_path, "calibration", "FETCH_SIZE", [("__amd_rocclr_copyBuffer", 524288.0), ("__amd_rocclr_copyBuffer", 16.0),
                                                       (full, 1000.0), (full, 3000.0)])
    _write_run(tmp_path, "calibration", "WRITE_SIZE", [("__amd_rocclr_copyBuffer", 1048576.0), (full, 500.0)])
    _write_run(tmp_path, "toy", "FETCH_SIZE", [("void hk::toy_kernel<1>(int)", 10.0), ("hk::other_kernel(int)", 1.0),
                                               ("void hk::toy_kernel<2>(int)", 99.0)])
    _write_run(tmp_path, "toy", "WRITE_SIZE", [("void hk::toy_kernel<1>(int)", 4.0), ("hk::other_kernel(int)", 2.0)])
    out = bench.collect_traffic(str(tmp_path))
    assert out["calibration_factor"] == {"FETCH_SIZE": 2.0, "WRITE_SIZE": 1.0}
    assert out["legs"]["fp8_gemm_8192"]["read_bytes"] == round(2000.0 * 2.0 * 1024)       # mean of the dispatches
    assert out["legs"]["fp8_gemm_8192"]["written_bytes"] == 500 * 1024
    toy = out["legs"]["toy"]
    assert toy["kernels"]["toy_kernel<1>"] == {"read_bytes": 20 * 1024, "written_bytes": 4 * 1024}
    assert toy["total_bytes"] == (20 + 2 + 4 + 2) * 1024
    assert json.load(open(tmp_path / "traffic.json")) == out
    # a kernel of a leg that no longer appears (or appears twice) is an error, not a silent zero
    monkeypatch.setattr(bench, "TRAFFIC_LEGS", {"toy": ("toy", ["toy_kernel"])})
    with pytest.raises(RuntimeError, match="2 kernels match"):
        bench.collect_traffic(str(tmp_path))
    monkeypatch.setattr(bench, "TRAFFIC_LEGS", {"toy": ("toy", ["gone_kernel"])})
    with pytest.raises(RuntimeError, match="0 kernels match"):
        bench.collect_traffic(str(tmp_path))


def test_every_traffic_leg_of_bench_is_in_the_tracked_file():
    bench = _load_bench()
    tracked = json.load(open(ROOT / "profiles" / "traffic.json"))
    assert set(tracked["legs"]) == set(bench.TRAFFIC_LEGS)
    for key, (_, kernels) in bench.TRAFFIC_LEGS.items():
        leg = tracked["legs"][key]
        assert set(leg["kernels"]) == set(kernels), key
        assert leg["total_bytes"] == leg["read_bytes"] + leg["written_bytes"] > 0
        assert bench._traffic(key) == leg["total_bytes"]
    assert bench._traffic("no_such_leg") is None


def test_tile_table_rewrite_keeps_the_other_formats(tmp_path, monkeypatch):
    from hipkittens_amd import tile_sweep

    table = tmp_path / "tile_table.inc"
    table.write_text("constexpr int kTileTableCus = 256;\nstatic const TileTableEntry kTileTable[] = {\n"
                     "    {255, 0, 0, 0, 0},\n    {0, 4, 16, 8, 64},\n    {1, 2, 2, 2, 128},\n    {2, 9, 9, 9, 256},\n};\n")
    monkeypatch.setattr(tile_sweep, "TABLE_PATH", table)
    n = tile_sweep._write_table("bf16", {(12, 45, 23, 64), (3, 3, 3, 256)}, 304)
    text = table.read_text()
    assert n == 4 and "kTileTableCus = 304" in text
    rows = [ln.strip() for ln in text.splitlines() if ln.strip().startswith("{")]
    assert rows == ["{255, 0, 0, 0, 0},   // (keeps the array non-empty)", "{0, 4, 16, 8, 64},", "{1, 3, 3, 3, 256},",
                    "{1, 12, 45, 23, 64},", "{2, 9, 9, 9, 256},"]
    assert tile_sweep._k_steps("fp8", 8192) == 64 and tile_sweep._k_steps("bf16", 8192) == 128
    assert tile_sweep._k_steps("mxfp4", 2880) == 12
