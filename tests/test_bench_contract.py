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
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--size", "small", "--steps", "5", "--warmup", "2"],
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
    c = d["cpu_baseline"]
    assert c["kind"] in ("reference", "port") and c["cores"] == 1 and c["value"] > 0 and c["sample"]
    assert d["validated"]["entries"] == d["config"]["nnz"]
