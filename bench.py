#!/usr/bin/env python3
"""SDDMM benchmark on one MI355X: GFLOP/s (2*nnz*K) on the FEM-banded fp32 K=32 shape.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--K K] [--strategy S]
                    [--per-config full|small|none] [--no-cpu]

A step is one SDDMM over the whole sampling matrix with every operand already
resident in HBM.  Prints ONE JSON line.  The headline (`value`, `roofline`) is the
workload named on the command line (default: fem_banded, K=32, AUTO); `per_config`
repeats the measurement for every benchmark shape at full size with its K sweep:
AUTO and every fixed strategy, launches in a loop ("warm") and launches that follow a
1 GiB copy through the caches ("cold"), each result read back AFTER its timed
launches and validated against the CPU oracle, with the reference's CPU loop timed on
the host cores of the same box beside it.

Roofline figures divide the COMPULSORY bytes of a launch (every operand byte once:
4(M+1) + 12 nnz + e K (rows_nonempty + columns_touched)) by the launch duration, so a
kernel that reuses gathered rows cannot exceed the 8 TB/s peak by counting bytes it
never moved; the gathered-bytes model (one B row per stored entry) is reported apart
as `gathered_equiv_gbs`.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0

# the five benchmark shapes with their K sweeps
PER_CONFIG = [("small_uniform", 32), ("fem_banded", 32), ("fem_banded", 128), ("power_law", 32),
              ("mixed_density", 32), ("mixed_density", 64), ("mixed_density", 256),
              ("dense_tiles", 128), ("dense_tiles", 512)]
FIXED = ["FLAT", "ROW_WAVE", "SHORT_ROWS", "LDS_TILED", "MFMA_TILE"]


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# --------------------------------------------------------------------------- CPU side
def cpu_baseline(w, budget_s=20.0, reps=3):
    """Reference CPU loop (1 thread, as the reference is serial) on the same inputs.
    The whole workload is one sample when a run fits the budget, else a leading
    block of rows.  Returns the dict for the JSON line plus an all-cores figure."""
    from oracle import oracle as O
    rowptr, col, sval = w.rowptr, w.col, w.sval
    est = w.flops() / 1.0e9          # seconds at ~1 GFLOP/s, conservative
    rows = w.M
    if est > budget_s:
        target = int(w.nnz * budget_s / est)
        rows = max(1, int(np.searchsorted(rowptr, target)))
    rp = np.ascontiguousarray(rowptr[: rows + 1])
    nn = int(rp[-1])
    cc, sv = np.ascontiguousarray(col[:nn]), np.ascontiguousarray(sval[:nn])
    flops = 2.0 * nn * w.K
    sample = "rows [0,%d) of %d: %d of %d entries, best of %d" % (rows, w.M, nn, w.nnz, reps)
    kind = "port"
    best = None
    if O.Ref.available():
        # the reference's own CPUBasic<float>::run_csr compiled from its headers
        kind = "reference"
        coo_r = np.repeat(np.arange(rows, dtype=np.int32), np.diff(rp)).astype(np.int32)
        best, _ = O.Ref().cpu_basic_csr_seconds(rows, w.N, coo_r, cc, sv, w.A[:rows], w.B, reps=reps)
    else:
        for _ in range(reps):
            t0 = time.perf_counter()
            O.sddmm_csr(rp, cc, sv, w.A, w.B, threads=1)
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
    threads = O.max_threads()
    allc = None
    for _ in range(reps):
        t0 = time.perf_counter()
        O.sddmm_csr(rp, cc, sv, w.A, w.B, threads=threads)
        dt = time.perf_counter() - t0
        allc = dt if allc is None else min(allc, dt)
    return ({"value": flops / best / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": kind, "sample": sample},
            {"value": flops / allc / 1e9, "unit": "GFLOP/s", "cores": threads, "kind": "port",
             "sample": sample})


class Checker:
    """The CPU oracle's result for one workload, computed once (all host cores)."""

    def __init__(self, w):
        from oracle import oracle as O
        self.O = O
        self.ref = O.sddmm_csr(w.rowptr, w.col, w.sval, w.A, w.B, threads=0)
        _, self.mag = O.sddmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)

    def check(self, got, rtol):
        ok, worst, i = self.O.check_values_fast(got, self.ref, mag=self.mag, rtol=rtol)
        return ok, worst, i


def load_traffic(key, field="bytes_per_launch"):
    """HBM bytes per launch (or another recorded field: `l2_hit`, `bound`) from an
    earlier rocprofv3 --pmc pair of runs (FETCH_SIZE, WRITE_SIZE), recorded by hand in
    profiles/traffic.json: a constant of the repository, NOT measured by this run;
    None when there is no record."""
    p = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(p):
        return None
    try:
        return json.load(open(p)).get(key, {}).get(field)
    except Exception:
        return None


TRAFFIC_SOURCE = ("profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (and TCC hits / requests) of an "
                  "earlier run of this command, recorded constants, not measured by this run")
SINGLE_KERNEL = ["FLAT", "ROW_WAVE", "SHORT_ROWS"]     # strategies that are one gather kernel, none of AUTO's parts


# --------------------------------------------------------------------------- GPU side
class CacheFlusher:
    """Two 512 MiB device buffers: copying one onto the other (1 GiB through the
    caches; the last-level cache holds 256 MB) leaves nothing of the SDDMM operands
    in any cache level."""

    def __init__(self):
        self.ok = False
        try:
            self.hip = C.CDLL("libamdhip64.so")
        except OSError:
            return
        self.hip.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.hip.hipFree.argtypes = [C.c_void_p]
        self.n = 512 << 20
        self.a, self.b = C.c_void_p(), C.c_void_p()
        if self.hip.hipMalloc(C.byref(self.a), self.n) != 0:
            return
        if self.hip.hipMalloc(C.byref(self.b), self.n) != 0:
            self.hip.hipFree(self.a)
            return
        self.ok = True

    def cold_launches(self, engine, reps):
        """Median device time (ms) of a launch right after the flush; None when unavailable."""
        if not self.ok:
            return None
        times = []
        for _ in range(reps):
            if self.hip.hipMemcpy(self.b, self.a, self.n, 3) != 0:      # device to device, returns when done
                break
            self.hip.hipDeviceSynchronize()
            times.append(float(engine.time_runs(0, 1)[0]))
        return float(np.median(times)) if times else None

    def close(self):
        if self.ok:
            self.hip.hipFree(self.a)
            self.hip.hipFree(self.b)
            self.ok = False


def upload(e, w, capi):
    if w.dtype != "f32":
        e.set_dense(w.A_bits, w.B_bits, capi.BF16 if w.dtype == "bf16" else capi.F16)
    else:
        e.set_dense(w.A, w.B, capi.F32)


def rtol_for(w, strategy_name):
    # 16-bit operands on the tile path are allowed 1e-2 (fp32 accumulation of exact products
    # lands far inside it); everything else is held to 1e-5
    return 1e-2 if w.dtype != "f32" and strategy_name == "MFMA_TILE" else 1e-5


def time_strategy(e, w, capi, name, steps, warmup, flusher, checker, cold_reps=6):
    """Plan `name`, run warm and cold launches, then read P back and validate it.
    The pattern is set again first, which clears P: what is validated is what the
    timed launches wrote.  Returns a dict, or {"error": ...} when the strategy does not
    apply to this input."""
    strategy = capi.STRATEGY_NAMES.index(name)
    try:
        e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
        e.plan(strategy)
        e.plan(strategy)                         # the second plan of a pattern: no allocation left to pay for
        st = e.stats()
        plan_ms = st.plan_ms
        for _ in range(warmup):
            e.launch()
        e.synchronize()
        region = min(e.time_region(steps) for _ in range(3))
        warm_ms = region / steps
        cold_ms = flusher.cold_launches(e, cold_reps) if flusher is not None else None
        st = e.stats()
        out = {"us": warm_ms * 1e3, "cold_us": None if cold_ms is None else cold_ms * 1e3,
               "plan_us": plan_ms * 1e3, "resolved": capi.STRATEGY_NAMES[st.strategy_used],
               "launches": st.kernels_launched or 1}
        if checker is not None:
            got = e.values()
            ok, worst, i = checker.check(got, rtol_for(w, name))
            if not ok:
                log("VALIDATION FAILED: %s K=%d %s entry %d got %r ref %r (%.2f x tolerance)" % (
                    w.name, w.K, name, i, got[i], checker.ref[i], worst))
                sys.exit(1)
            out["validated"] = {"entries": int(len(got)), "worst_over_tol": round(worst, 4)}
        if name == "AUTO":
            out["classes"] = {"rows_short": st.rows_short, "rows_medium": st.rows_medium, "rows_long": st.rows_long,
                              "panels": st.panels, "nnz_panel": st.nnz_panel, "mfma_tiles": st.mfma_tiles,
                              "nnz_mfma": st.nnz_mfma}
        return out
    except capi.SddmmError as ex:
        if ex.code == capi.ERR_UNSUPPORTED:
            return {"error": "unsupported"}
        raise


def fused_leg(e, w, capi, reps, check):
    """O = P * B after the SDDMM, in the same pass (sddmm_run_fused): device time per call between
    the library's own events (the memset of O included), 4*nnz*K flops."""
    e.plan(capi.AUTO)
    times = []
    for _ in range(reps):
        e.run_fused(fetch=False)
        times.append(e.stats().run_ms)
    launches = e.stats().kernels_launched
    t = float(np.median(times))
    res = {"ms_p50": t, "ms_min": float(min(times)), "gflops": 4.0 * w.nnz * w.K / (t * 1e-3) / 1e9,
           "kernels_launched": launches, "validated": None}
    if check:
        from oracle import oracle as O
        got = e.run_fused()
        ref_p, ref_o = O.fusedmm_csr(w.rowptr, w.col, w.sval, w.A, w.B)
        _, mag_o = O.fusedmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
        ok, worst, i = O.check_values_fast(got[:w.M].ravel(), ref_o.ravel(), mag=mag_o.ravel(), rtol=rtol_for(w, "AUTO"))
        if not ok:
            log("VALIDATION FAILED (fused): element %d got %r (%.2f x tolerance)" % (i, got[:w.M].ravel()[i], worst))
            sys.exit(1)
        res["validated"] = {"elements": int(w.M * w.K), "worst_over_tol": round(worst, 4)}
    if w.dtype == "f32" and w.K % 8 == 0:
        res["bf16_operands"] = fused_bf16_leg(w, capi, reps, check)
    return res


def fused_bf16_leg(w, capi, reps, check):
    """The same fused call with A and B stored as bfloat16 (P and O stay fp32), validated
    against the fp32 oracle on the rounded operands."""
    Ab, Bb = capi.to_bf16(w.A).reshape(w.A.shape), capi.to_bf16(w.B).reshape(w.B.shape)
    e = capi.Engine(0)
    e.set_dense(Ab, Bb, capi.BF16)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    e.plan(capi.AUTO)
    times = []
    for _ in range(reps):
        e.run_fused(fetch=False)
        times.append(e.stats().run_ms)
    t = float(np.median(times))
    res = {"ms_p50": t, "ms_min": float(min(times)), "gflops": 4.0 * w.nnz * w.K / (t * 1e-3) / 1e9,
           "kernels_launched": e.stats().kernels_launched, "validated": None}
    if check:
        from oracle import oracle as O
        got = e.run_fused()
        Ar, Br = capi.from_bf16(Ab).reshape(w.A.shape), capi.from_bf16(Bb).reshape(w.B.shape)
        _, ref_o = O.fusedmm_csr(w.rowptr, w.col, w.sval, Ar, Br)
        _, mag_o = O.fusedmm_csr_f64(w.rowptr, w.col, w.sval, Ar, Br)
        ok, worst, i = O.check_values_fast(got[:w.M].ravel(), ref_o.ravel(), mag=mag_o.ravel(), rtol=1e-5)
        if not ok:
            log("VALIDATION FAILED (fused, bf16 operands): element %d got %r (%.2f x tolerance)" % (i, got[:w.M].ravel()[i], worst))
            sys.exit(1)
        res["validated"] = {"elements": int(w.M * w.K), "worst_over_tol": round(worst, 4)}
    e.close()
    return res


def fractions(w, us, cold_us):
    """Compulsory bytes over launch time against the HBM peak.  `frac` is taken from the
    cold launches, the only ones whose operands come from HBM; `frac_llc` from the
    launches of a loop, which find a working set below 256 MB in the last-level cache.
    Also the recorded counter figures of the shape (traffic against the peak, L2 hit
    rate, what bounds it) and, for 16-bit operands, the flops against the bf16 MFMA peak."""
    comp = w.bytes_compulsory()
    d = {"frac": None if not cold_us else comp / (cold_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
         "frac_llc": comp / (us * 1e-6) / 1e9 / HBM_PEAK_GBS}
    key = "%s_K%d_%s" % (w.name, w.K, w.dtype)
    traffic = load_traffic(key)
    d["traffic"] = traffic
    d["traffic_frac"] = None if not (traffic and cold_us) else traffic / (cold_us * 1e-6) / 1e9 / HBM_PEAK_GBS
    d["traffic_frac_llc"] = None if not traffic else traffic / (us * 1e-6) / 1e9 / HBM_PEAK_GBS
    d["l2_hit"] = load_traffic(key, "l2_hit")
    d["bound"] = load_traffic(key, "bound")
    if w.dtype != "f32":
        d["mfma_frac"] = w.flops() / (us * 1e-6) / 1e12 / MFMA_BF16_PEAK_TFLOPS
    return d


def per_config_entry(name, K, capi, workloads, steps, warmup, flusher, no_cpu, size="full"):
    t0 = time.time()
    w = workloads.make(name, size, K=K)
    checker = Checker(w)
    e = capi.Engine(0)
    upload(e, w, capi)
    auto = time_strategy(e, w, capi, "AUTO", steps, warmup, flusher, checker)
    fixed = {s: time_strategy(e, w, capi, s, steps, warmup, flusher, checker) for s in FIXED}
    e.close()
    ran = {s: r for s, r in fixed.items() if "us" in r}
    best = min(ran, key=lambda s: ran[s]["us"])
    best_cold = min(ran, key=lambda s: ran[s]["cold_us"] or float("inf"))
    single = [s for s in SINGLE_KERNEL if s in ran]
    best_single = min(single, key=lambda s: ran[s]["us"])
    entry = {
        "workload": w.name, "K": w.K, "dtype": w.dtype, "M": w.M, "N": w.N, "nnz": w.nnz,
        "auto_us": auto["us"], "auto_cold_us": auto["cold_us"], "auto_resolved": auto["resolved"],
        "plan_us": auto["plan_us"], "launches": auto["launches"],
        "best_fixed": best, "best_fixed_us": ran[best]["us"],
        "best_fixed_cold": best_cold, "best_fixed_cold_us": ran[best_cold]["cold_us"],
        "auto_over_best_fixed": ran[best]["us"] / auto["us"],
        "best_single_kernel": best_single, "best_single_kernel_us": ran[best_single]["us"],
        "auto_over_best_single_kernel": ran[best_single]["us"] / auto["us"],
        "fixed_us": {s: (round(r["us"], 2) if "us" in r else r["error"]) for s, r in fixed.items()},
        "gflops": w.flops() / (auto["us"] * 1e-6) / 1e9,
        "bytes_compulsory": w.bytes_compulsory(),
        "compulsory_gbs": w.bytes_compulsory() / (auto["us"] * 1e-6) / 1e9,
        "gathered_equiv_gbs": w.bytes_gathered() / (auto["us"] * 1e-6) / 1e9,
        "classes": auto.get("classes"),
        "validated": {"strategies": 1 + len(ran), "entries": w.nnz,
                      "worst_over_tol": max([auto["validated"]["worst_over_tol"]] +
                                            [r["validated"]["worst_over_tol"] for r in ran.values()])},
    }
    entry.update(fractions(w, auto["us"], auto["cold_us"]))
    if not no_cpu:
        base, allc = cpu_baseline(w, budget_s=1.5, reps=2)
        entry["cpu_1core_gflops"] = round(base["value"], 3)
        entry["cpu_1core_kind"] = base["kind"]
        entry["cpu_allcores_gflops"] = round(allc["value"], 2)
        entry["cpu_cores"] = allc["cores"]
        entry["cpu_sample"] = base["sample"]
    log("per_config %s K=%d: AUTO %.1f us (cold %s), plan %.0f us, best fixed %s %.1f us, best single kernel %s %.1f us, "
        "frac %s (llc %.3f)  [%.1fs]" % (
            w.name, w.K, auto["us"], "%.1f" % auto["cold_us"] if auto["cold_us"] else "-", auto["plan_us"], best,
            ran[best]["us"], best_single, ran[best_single]["us"],
            "%.3f" % entry["frac"] if entry["frac"] else "-", entry["frac_llc"], time.time() - t0))
    return entry


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="fem_banded")
    ap.add_argument("--size", default="full", choices=["full", "small"])
    ap.add_argument("--K", type=int, default=32)
    ap.add_argument("--strategy", default="AUTO")
    ap.add_argument("--include-plan", action="store_true", help="re-run the classifier inside every timed step")
    ap.add_argument("--f16", action="store_true", help="dense_tiles: IEEE half operands instead of bf16")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline legs")
    ap.add_argument("--no-check", action="store_true", help="skip validation of the headline against the oracle")
    ap.add_argument("--per-config", default=None, choices=["full", "small", "none"],
                    help="size of the per_config sweep (default: full with --size full, none otherwise)")
    ap.add_argument("--no-per-config", action="store_true", help="headline only (e.g. under a profiler)")
    ap.add_argument("--fused", action="store_true",
                    help="also time SDDMM followed by SpMM over the same pattern (sddmm_run_fused) and add it as `fused`")
    args = ap.parse_args()

    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        log("bench.py measures one GPU: SDDMM row panels are independent, there is no multi-GPU path "
            "in this build (requested --gpus %d, WORLD_SIZE %d)." % (args.gpus, world))
        sys.exit(2)

    from dphpc_amd import capi, workloads

    t0 = time.time()
    extra = {"f16": True} if args.f16 and args.workload == "dense_tiles" else {}
    w = workloads.make(args.workload, args.size, K=args.K, **extra)
    log("workload %s: M=%d N=%d K=%d nnz=%d (%.1fs to generate)" % (w.name, w.M, w.N, w.K, w.nnz, time.time() - t0))
    strategy = capi.STRATEGY_NAMES.index(args.strategy.upper())

    e = capi.Engine(0)
    upload(e, w, capi)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)      # P starts at zero
    e.plan(strategy)
    plan_first_ms = e.stats().plan_ms        # the first plan of the process also pays for allocations and code loading
    plans = []
    for _ in range(5):
        e.plan(strategy)
        plans.append(e.stats().plan_ms)
    plan_ms = float(np.median(plans))

    # ---- timed region: W warm-up steps, then exactly K steps --------------------
    for _ in range(args.warmup):
        if args.include_plan:
            e.plan(strategy)
        e.launch()
    e.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        if args.include_plan:
            e.plan(strategy)
        e.launch()
    e.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # ---- validate what the timed launches left in P ------------------------------
    validated = None
    if not args.no_check:
        got = e.values()
        ok, worst, i = Checker(w).check(got, rtol_for(w, args.strategy.upper()))
        if not ok:
            log("VALIDATION FAILED: entry %d got %r (%.2f x tolerance)" % (i, got[i], worst))
            sys.exit(1)
        validated = {"entries": int(len(got)), "worst_over_tol": round(worst, 4), "when": "after the timed steps"}
        log("validated %d entries against the CPU oracle (worst %.3f of tolerance)" % (len(got), worst))

    # ---- device time from HIP events on the launch stream ------------------------
    # average launch duration: the same K steps between one pair of events (best of 3
    # regions; what a kernel trace of this loop reports per launch); `isolated` is
    # each launch between its own events with a wait in between, i.e. with the idle
    # gap a lone launch pays; `cold` is a launch that follows a 1 GiB device copy
    region = min(e.time_region(args.steps, include_plan=args.include_plan) for _ in range(3))
    ev_avg = region / args.steps
    ev = e.time_runs(2, max(args.steps, 20), include_plan=args.include_plan)
    ev_p50, ev_min = float(np.median(ev)), float(ev.min())
    flusher = CacheFlusher()
    ev_cold = None if args.include_plan else flusher.cold_launches(e, 10)
    # classifier + run in one timed region, for the record (the classifier belongs to
    # the init phase, as the reference's preprocessing does: benchmark.hpp:148-190
    # times init_csr apart from run_csr)
    ev_plan = e.time_runs(1, 5, include_plan=True)
    st = e.stats()
    flops, gathered, compulsory = w.flops(), w.bytes_gathered(), w.bytes_compulsory()
    # The HBM figure comes from the cold launches: in the loop a working set below 256 MB is
    # served by the last-level cache, which `achieved_llc` / `frac_llc` report apart.  Only
    # with --include-plan (no cold launches are timed then) does the loop stand in.
    achieved_llc = compulsory / (ev_avg * 1e-3) / 1e9
    hbm_ms = ev_cold if ev_cold else ev_avg
    achieved = compulsory / (hbm_ms * 1e-3) / 1e9
    key = "%s_K%d_%s" % (w.name, w.K, w.dtype)
    traffic = load_traffic(key)
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS,
                "launches": "cold: each follows a 1 GiB device copy, operands come from HBM" if ev_cold else
                "in a loop (no cold launches were timed): the last-level cache may serve them",
                "bytes": "compulsory: every operand byte once per launch",
                "achieved_llc": achieved_llc,
                "frac_llc": achieved_llc / HBM_PEAK_GBS,
                "gathered_equiv_gbs": gathered / (ev_avg * 1e-3) / 1e9,
                "traffic": traffic,
                "traffic_source": None if traffic is None else TRAFFIC_SOURCE,
                "l2_hit": load_traffic(key, "l2_hit"),
                "limit": load_traffic(key, "bound")}
    if traffic:
        roofline["traffic_frac"] = traffic / (hbm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS
        roofline["traffic_frac_llc"] = traffic / (ev_avg * 1e-3) / 1e9 / HBM_PEAK_GBS
    if w.dtype != "f32":
        roofline["mfma_frac"] = flops / (ev_avg * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS

    out = {
        "metric": "SDDMM GFLOP/s (2*nnz*K), 1 MI355X, K=%d" % w.K,
        "value": flops / (ms_per_step * 1e-3) / 1e9,
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.dtype,
        "data": "synthetic",
        "config": {"workload": w.name, "size": args.size, "M": w.M, "N": w.N, "K": w.K, "nnz": w.nnz,
                   "strategy": capi.STRATEGY_NAMES[st.strategy_used], "requested": args.strategy.upper(),
                   "plan_in_step": bool(args.include_plan)},
        "roofline": roofline,
        "kernel_ms": {"avg": ev_avg, "isolated_p50": ev_p50, "isolated_min": ev_min, "cold_p50": ev_cold,
                      "launches_per_step": st.kernels_launched or 1},
        "gflops_kernel": flops / (ev_avg * 1e-3) / 1e9,
        "gflops_kernel_cold": None if not ev_cold else flops / (ev_cold * 1e-3) / 1e9,
        "bytes_gathered": gathered,
        "bytes_compulsory": compulsory,
        "plan_ms": plan_ms,
        "plan_first_ms": plan_first_ms,
        "plan_plus_run_ms": float(np.median(ev_plan)),
        "classes": {"rows_short": st.rows_short, "rows_medium": st.rows_medium, "rows_long": st.rows_long,
                    "panels": st.panels, "nnz_panel": st.nnz_panel, "mfma_tiles": st.mfma_tiles,
                    "nnz_mfma": st.nnz_mfma},
        "validated": validated,
    }
    if args.fused:
        out["fused"] = fused_leg(e, w, capi, max(args.steps, 20), not args.no_check)
    e.close()
    if not args.no_cpu:
        base, allc = cpu_baseline(w)
        out["cpu_baseline"] = base
        out["cpu_allcores"] = allc
    sweep = args.per_config or ("full" if args.size == "full" else "none")
    if not args.no_per_config and sweep != "none":
        t0 = time.time()
        out["per_config_size"] = sweep
        out["per_config"] = [per_config_entry(n, k, capi, workloads, max(20, min(args.steps, 50)), 3, flusher,
                                              args.no_cpu, sweep) for n, k in PER_CONFIG]
        log("per_config: %d entries in %.0f s" % (len(out["per_config"]), time.time() - t0))
    flusher.close()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
