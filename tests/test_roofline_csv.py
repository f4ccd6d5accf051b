"""The roofline summary of a benchmark CSV: the reference's quantities
(plots/plot_roofline.py:29-30) on rows in the reference's schema (src/main.cpp:356-358)."""
import importlib.util
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("roofline_csv", os.path.join(ROOT, "dphpc_amd", "host", "roofline_csv.py"))
R = importlib.util.module_from_spec(spec)
spec.loader.exec_module(R)

HEADER = ("competitor,dataset,mat_repr,M,N,K,NZ,total_ns,init_ns,comp_ns,cleanup_ns,correctness,"
          "num_thread_blocks,num_threads_per_block")


def test_points_and_table(tmp_path, capsys):
    lines = [HEADER,
             "GPU-AMD-Dynamic,fem,CSR,1000,2000,32,50000,900,100,400,400,1,0,256",
             "GPU-AMD-Dynamic,fem,CSR,1000,2000,32,50000,900,100,200,400,1,0,256",
             "GPU-AMD-Dynamic,fem,CSR,1000,2000,32,50000,900,100,600,400,1,0,256",
             "GPU-AMD-Dynamic,fem,CSR,1000,2000,32,50000,900,100,1,400,0,0,256",     # failed run: ignored
             "GPU-AMD-Flat,fem,COO,1000,2000,32,50000,900,100,1000,400,1,0,256",
             "some stderr-like noise"]
    p = tmp_path / "r.csv"
    p.write_text("\n".join(lines) + "\n")
    pts = R.points(R.read_csv(str(p)))
    a = pts[("fem", "GPU-AMD-Dynamic", "CSR", 32)]
    assert a["runs"] == 3 and a["ns"] == 400.0
    assert a["flops"] == 2 * 32 * 50000 + 50000                      # plot_roofline.py:29
    assert a["bytes"] == (1000 * 32 + 2000 * 32) * 4 + 50000 * 4     # plot_roofline.py:30
    assert abs(a["performance"] - a["flops"] / 400e-9) < 1e-3 * a["performance"]
    assert abs(a["op_intensity"] - a["flops"] / a["bytes"]) < 1e-12
    assert a["roof"] == min(R.PEAK_FLOPS, R.PEAK_BYTES * a["op_intensity"])
    b = pts[("fem", "GPU-AMD-Flat", "COO", 32)]
    assert b["ns"] == 1000.0 and len(pts) == 2
    assert R.points(R.read_csv(str(p)), percentile=1.0)[("fem", "GPU-AMD-Dynamic", "CSR", 32)]["ns"] == 600.0
    assert R.main([str(p), "--png", str(tmp_path / "r.png")]) == 0
    out = capsys.readouterr().out
    assert "GPU-AMD-Dynamic" in out and "GPU-AMD-Flat" in out
    assert (tmp_path / "r.png").stat().st_size > 1000
