"""bench.py contract pieces that can be checked without a GPU, and the JSON line on one."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                       stderr=subprocess.PIPE, text=True, timeout=120)
    assert p.returncode == 2
    assert "one GPU" in p.stderr and p.stdout.strip() == ""


def test_traffic_table_names_existing_profiles():
    t = json.load(open(os.path.join(ROOT, "profiles", "traffic.json")))
    assert "fem_banded_K32_f32" in t                      # the bench default
    for key, rec in t.items():
        if key.startswith("_"):
            continue
        assert rec["bytes_per_launch"] == rec["fetch_bytes"] + rec["write_bytes"]


@pytest.mark.gpu
def test_json_line_on_a_small_run():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--size", "small", "--steps", "5", "--warmup", "2",
                        "--per-config", "small", "--fused"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=280)
    assert p.returncode == 0, p.stderr
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["unit"] == "GFLOP/s"
    assert d["dtype"] == "f32" and d["data"] == "synthetic" and d["vs_baseline"] is None
    assert d["config"]["workload"] == "fem_banded" and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12
    # compulsory bytes over launch time: a fraction of the peak, whatever the kernel reuses
    assert 0 < r["frac"] <= 1.0 and r["gathered_equiv_gbs"] >= r["achieved_llc"]
    # the HBM figure is the one of the cold launches; the loop's is reported apart
    assert r["achieved"] == pytest.approx(d["bytes_compulsory"] / (d["kernel_ms"]["cold_p50"] * 1e-3) / 1e9)
    assert r["achieved_llc"] == pytest.approx(d["bytes_compulsory"] / (d["kernel_ms"]["avg"] * 1e-3) / 1e9)
    assert r["launches"].startswith("cold")
    c = d["cpu_baseline"]
    assert c["kind"] in ("reference", "port") and c["cores"] == 1 and c["value"] > 0 and c["sample"]
    assert d["validated"]["entries"] == d["config"]["nnz"]
    f = d["fused"]
    assert f["ms_p50"] >= f["ms_min"] > 0 and f["kernels_launched"] >= 1
    assert f["validated"]["elements"] == d["config"]["M"] * d["config"]["K"] and f["validated"]["worst_over_tol"] <= 1.0
    # the sweep over the five shapes: AUTO next to every fixed strategy, all validated
    pc = d["per_config"]
    assert [(x["workload"], x["K"]) for x in pc] == [
        ("small_uniform", 32), ("fem_banded", 32), ("fem_banded", 128), ("power_law", 32), ("mixed_density", 32),
        ("mixed_density", 64), ("mixed_density", 256), ("dense_tiles", 128), ("dense_tiles", 512)]
    for x in pc:
        assert 0 < x["frac"] <= 1.0 and 0 < x["frac_llc"] <= 1.0
        assert x["frac"] == pytest.approx(x["bytes_compulsory"] / (x["auto_cold_us"] * 1e-6) / 1e9 / 8000.0)
        assert x["auto_us"] > 0 and x["best_fixed"] in x["fixed_us"]
        assert x["best_single_kernel"] in ("FLAT", "ROW_WAVE", "SHORT_ROWS")
        assert x["auto_over_best_single_kernel"] == pytest.approx(x["best_single_kernel_us"] / x["auto_us"])
        assert x["validated"]["entries"] == x["nnz"] and x["validated"]["worst_over_tol"] <= 1.0
        assert x["cpu_1core_gflops"] > 0
        assert x["dtype"] == ("bf16" if x["workload"] == "dense_tiles" else "f32")
