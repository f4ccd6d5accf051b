#!/usr/bin/env python3
"""Roofline figures from a benchmark CSV in the reference's 14-column schema
(src/main.cpp:356-358), as written by dphpc_amd/lib/sddmm_driver.

    python dphpc_amd/host/roofline_csv.py results.csv [--percentile 0.5] [--png roofline.png]

The quantities are the ones of the reference's plots/plot_roofline.py:29-30 --
flops = 2*K*NZ + NZ, bytes = 4*(M*K + N*K) + 4*NZ (each operand once, P not
counted), performance = flops / comp time, operational intensity = flops / bytes
-- with seconds = ns / 1e9 (the reference divides by 10e9 and scales its peaks by
the same factor of ten, plot_roofline.py:18-21,93) against the MI355X roofs.
"""
import argparse
import csv
import sys
from collections import defaultdict

PEAK_FLOPS = 157.3e12      # MI355X fp32 (vector and matrix), FLOP/s
PEAK_BYTES = 8.0e12        # MI355X HBM3E, B/s


def flops(nz, k):
    return 2.0 * k * nz + nz


def trans_bytes(m, n, k, nz):
    return (m * k + n * k) * 4.0 + nz * 4.0


def quantile(values, q):
    v = sorted(values)
    if not v:
        return float("nan")
    pos = q * (len(v) - 1)
    lo = int(pos)
    hi = min(lo + 1, len(v) - 1)
    return v[lo] + (v[hi] - v[lo]) * (pos - lo)


def points(rows, percentile=0.5, field="comp_ns"):
    """{(dataset, competitor, mat_repr, K): dict} from CSV rows (dicts); runs flagged
    incorrect (correctness != 1) are left out, as a failed run has no meaningful time."""
    groups = defaultdict(list)
    shape = {}
    for r in rows:
        if str(r.get("correctness", "1")).strip() != "1":
            continue
        key = (r["dataset"], r["competitor"], r["mat_repr"], int(r["K"]))
        groups[key].append(float(r[field]))
        shape[key] = (int(r["M"]), int(r["N"]), int(r["K"]), int(r["NZ"]))
    out = {}
    for key, times in groups.items():
        m, n, k, nz = shape[key]
        ns = quantile(times, percentile)
        f, b = flops(nz, k), trans_bytes(m, n, k, nz)
        perf = f / (ns / 1e9) if ns > 0 else float("nan")
        oi = f / b
        out[key] = {"ns": ns, "flops": f, "bytes": b, "performance": perf, "op_intensity": oi,
                    "roof": min(PEAK_FLOPS, PEAK_BYTES * oi), "runs": len(times)}
    return out


def read_csv(path):
    with open(path, newline="") as fh:
        lines = [l for l in fh if l.count(",") == 13]     # the driver prints its errors to stderr only
    return list(csv.DictReader(lines))


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("csv")
    ap.add_argument("--percentile", type=float, default=0.5)
    ap.add_argument("--field", default="comp_ns", choices=["total_ns", "init_ns", "comp_ns", "cleanup_ns"])
    ap.add_argument("--png", help="write a log-log roofline plot (needs matplotlib)")
    args = ap.parse_args(argv)
    pts = points(read_csv(args.csv), args.percentile, args.field)
    print("%-16s %-20s %-4s %5s %12s %14s %10s %9s" % ("dataset", "competitor", "repr", "K", "time [us]", "GFLOP/s",
                                                       "flop/byte", "of roof"))
    for key in sorted(pts):
        p = pts[key]
        print("%-16s %-20s %-4s %5d %12.1f %14.1f %10.3f %8.1f%%" % (key[0], key[1], key[2], key[3], p["ns"] / 1e3,
                                                                     p["performance"] / 1e9, p["op_intensity"],
                                                                     100.0 * p["performance"] / p["roof"]))
    if args.png:
        import matplotlib
        matplotlib.use("Agg")
        import matplotlib.pyplot as plt
        fig, ax = plt.subplots(figsize=(10, 8))
        xs = [2.0 ** (e / 4.0) for e in range(-16, 41)]
        ax.plot(xs, [min(PEAK_FLOPS, PEAK_BYTES * x) for x in xs], color="black")
        markers = "osD^vP*X<>"
        comps = sorted({k[1] + " - " + k[2] for k in pts})
        sets = sorted({k[0] for k in pts})
        for key, p in pts.items():
            ax.scatter(p["op_intensity"], p["performance"], marker=markers[comps.index(key[1] + " - " + key[2]) % len(markers)],
                       color="C%d" % (sets.index(key[0]) % 10), s=60)
        for i, s in enumerate(sets):
            ax.scatter([], [], color="C%d" % (i % 10), label=s)
        for i, c in enumerate(comps):
            ax.scatter([], [], color="grey", marker=markers[i % len(markers)], label=c)
        ax.set_xscale("log"); ax.set_yscale("log")
        ax.set_xlabel("Operational Intensity [Flops/byte]"); ax.set_ylabel("Performance [Flops/s]")
        ax.set_title("SDDMM roofline, MI355X (fp32 peak 157.3 TFLOP/s, HBM 8 TB/s)")
        ax.legend(loc="upper center", bbox_to_anchor=(0.5, -0.1), ncol=4, fontsize="small")
        fig.tight_layout()
        fig.savefig(args.png)
    return 0


if __name__ == "__main__":
    sys.exit(main())
