"""Runs the C++ host-layer test program (tests/host/test_host.cpp): the reference's
own test cases against this repository's containers and GPUAmd competitor, and --
when it was built next to the reference tree -- the adapter compiled against the
reference's real headers (oracle/_ref/ref_adapter_check)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host", "test_host")
REF_BIN = os.path.join(ROOT, "oracle", "_ref", "ref_adapter_check")


def _run(args, timeout):
    p = subprocess.run(args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=timeout, text=True)
    print(p.stdout, flush=True)
    return p


def _binary():
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-C", os.path.dirname(BIN)])
    return BIN


def test_containers_and_partition_cpu():
    p = _run([_binary(), "cpu"], 300)
    assert p.returncode == 0, p.stdout
    assert " 0 failed" in p.stdout


@pytest.mark.gpu
def test_competitor_runs_the_reference_test_cases():
    p = _run([_binary(), "gpu"], 110)
    assert p.returncode == 0, p.stdout
    assert " 0 failed" in p.stdout


@pytest.mark.gpu
@pytest.mark.skipif(not os.path.exists(REF_BIN), reason="oracle/_ref/ref_adapter_check not built (reference tree absent)")
def test_adapter_against_reference_headers_and_cpu_basic():
    p = _run([REF_BIN], 110)
    assert p.returncode == 0, p.stdout
    assert "0 failure(s)" in p.stdout


DRIVER = os.path.join(ROOT, "dphpc_amd", "lib", "sddmm_driver")
CSV_COLUMNS = ("competitor,dataset,mat_repr,M,N,K,NZ,total_ns,init_ns,comp_ns,cleanup_ns,correctness,"
               "num_thread_blocks,num_threads_per_block")


def _csv_rows(text):
    lines = [l for l in text.splitlines() if l.count(",") == 13]
    assert lines and lines[0] == CSV_COLUMNS      # the reference's schema (src/main.cpp:356-358)
    return [dict(zip(CSV_COLUMNS.split(","), l.split(","))) for l in lines[1:]]


@pytest.mark.gpu
def test_driver_prints_reference_csv_and_all_runs_are_correct():
    assert os.path.exists(DRIVER), "driver not built: run __graft_entry__.build()"
    p = _run([DRIVER, "--scale", "0.05", "--num_runs", "2", "--K", "32"], 110)
    assert p.returncode == 0, p.stdout
    rows = _csv_rows(p.stdout)
    assert {r["dataset"] for r in rows} == {"small_uniform", "fem_banded", "power_law", "mixed_density", "dense_tiles"}
    # competitors[0] is the host loop, the expected result of every other row
    # (src/benchmark/benchmark.hpp:50-61, src/main.cpp:18-22)
    assert rows[0]["competitor"] == "CPU-Basic"
    assert {r["competitor"] for r in rows} == {"CPU-Basic", "GPU-AMD-Exact", "GPU-AMD-Dynamic", "GPU-AMD-Flat", "GPU-AMD-RowWave",
                                               "GPU-AMD-ShortRows", "GPU-AMD-Tiled", "GPU-AMD-MFMA"}
    assert {r["mat_repr"] for r in rows} == {"CSR", "COO"}
    for r in rows:
        assert r["correctness"] == "1", r
        assert int(r["comp_ns"]) > 0 and int(r["total_ns"]) >= int(r["init_ns"])
        assert r["num_threads_per_block"] == ("1" if r["competitor"] == "CPU-Basic" else "256")


@pytest.mark.gpu
def test_driver_reads_matrix_market_like_the_reference(tmp_path):
    # symmetric qualifier is not expanded and |v| < 1e-7 is dropped
    # (src/benchmark/dataset.hpp:159-175)
    mtx = tmp_path / "tiny.mtx"
    mtx.write_text("%%MatrixMarket matrix coordinate real symmetric\n% comment\n4 5 5\n"
                   "1 1 2.5\n2 1 -1.0\n4 5 3.0\n3 2 1e-9\n2 4 0.5\n")
    p = _run([DRIVER, "--dataset", str(mtx), "--num_runs", "1", "--K", "8"], 60)
    assert p.returncode == 0, p.stdout
    rows = _csv_rows(p.stdout)
    assert rows and all(r["M"] == "4" and r["N"] == "5" and r["NZ"] == "4" and r["correctness"] == "1" for r in rows)
    bad = tmp_path / "bad.mtx"
    bad.write_text("%%MatrixMarket matrix coordinate real general\n2 2 2\n1 1 1.0\n")
    p = _run([DRIVER, "--dataset", str(bad)], 60)
    assert p.returncode == 1 and "ends before" in p.stdout


@pytest.mark.gpu
def test_driver_reads_snap_edge_list_like_the_reference(tmp_path):
    # four '#' header lines, TAB-separated 0-based pairs, value 1, fixed square
    # dimension (src/benchmark/dataset.hpp:271-313)
    import random
    rnd = random.Random(5)
    edges = {(rnd.randrange(300), rnd.randrange(300)) for _ in range(4000)}
    txt = tmp_path / "edges.txt"
    txt.write_text("# Directed graph\n# test\n# Nodes: 300 Edges: %d\n# FromNodeId\tToNodeId\n" % len(edges)
                   + "".join("%d\t%d\n" % e for e in sorted(edges)))
    p = _run([DRIVER, "--dataset", str(txt), "--dim", "320", "--num_runs", "1", "--K", "32"], 60)
    assert p.returncode == 0, p.stdout
    rows = _csv_rows(p.stdout)
    assert rows and all(r["M"] == "320" and r["N"] == "320" and r["NZ"] == str(len(edges)) and r["correctness"] == "1"
                        for r in rows)
    p = _run([DRIVER, "--dataset", str(txt), "--dim", "100"], 60)
    assert p.returncode == 1 and "dimension" in p.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("name,nz", [("latin_hypercube", 5000), ("unbalanced", 49 * 496)])
def test_driver_runs_the_reference_latin_and_unbalanced_shapes(name, nz):
    # one entry per row and column; a block of completely filled leading rows
    # (src/benchmark/dataset.hpp:358-412); scale 0.05: 5000 x 5000 and 992 x 496 with 49 full rows
    p = _run([DRIVER, "--dataset", name, "--scale", "0.05", "--num_runs", "1", "--K", "32"], 60)
    assert p.returncode == 0, p.stdout
    rows = _csv_rows(p.stdout)
    assert len(rows) == 16 and rows[0]["competitor"] == "CPU-Basic" and all(r["dataset"] == name and r["NZ"] == str(nz) and r["correctness"] == "1" for r in rows)
