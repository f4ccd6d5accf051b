"""Parity of the HIP path (through the C ABI) with the CPU oracle.  All GPU.

Bar: pattern and entry order bit-exact (P is returned in the caller's order by
construction, checked through per-entry comparison); fp32 values within
1e-5 * max(|ref|, 0.25 * |S| sum_k |a_k b_k|) of the oracle's fp32 k-ascending
result (the floor covers entries whose terms cancel: both summation orders are
equally accurate there and the pure relative error is unbounded); the EXACT
strategy must be bit-identical to the oracle; bf16 inputs within 1e-2 on the
same scale, the oracle consuming the bf16-rounded inputs.
"""
import sys

import numpy as np
import pytest

from dphpc_amd import capi, workloads as W
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32

FP32_STRATEGIES = [capi.AUTO, capi.FLAT, capi.ROW_WAVE, capi.SHORT_ROWS, capi.LDS_TILED, capi.MFMA_TILE, capi.EXACT]


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def run_csr(make, rowptr, col, sval, A, B, N, strategy, dtype=capi.F32):
    e = make()
    try:
        e.set_dense(A, B, dtype)
        e.set_csr(len(rowptr) - 1, N, rowptr, col, sval)
        e.plan(strategy)
        e.run()
        return e.values(), e.stats()
    finally:
        e.close()


def assert_parity(got, rowptr, col, sval, A, B, rtol=1e-5, exact=False, what=""):
    ref = O.sddmm_csr(rowptr, col, sval, A, B, threads=0)
    if exact:
        bad = np.nonzero(got.view(np.uint32) != ref.view(np.uint32))[0]
        assert len(bad) == 0, "%s: %d entries differ bitwise, first %d: %r vs %r" % (
            what, len(bad), bad[0], got[bad[0]], ref[bad[0]])
        return
    _, mag = O.sddmm_csr_f64(rowptr, col, sval, A, B)
    ok, worst, i = O.check_values(got, ref, mag=mag, rtol=rtol)
    assert ok, "%s: entry %d got %r ref %r (%.2f x tolerance)" % (what, i, got[i], ref[i], worst)


# ---- the reference's hand-checkable cases (tests/matrix_test.cc:124-182) -------
KATS = {
    "sddmm_coo1": ([[1, 2], [3, 4]], [[-1, 2], [-3, 4]], [(0, 0, 1), (0, 1, 1), (1, 0, 1), (1, 1, 1)], 2, 2, [3, 5, 5, 7]),
    "sddmm_coo2": ([[1, 2, 3], [4, 5, 6]], [[-1, -3, 5], [2, 4, -6]], [(0, 0, 1), (1, 0, 1), (1, 1, 1)], 2, 2, [8, 11, -8]),
    "sddmm_coo3": ([[1, 2, 3], [4, 5, 6]], [[-1, -3, 5]], [(0, 0, 1), (1, 0, -1)], 2, 1, [8, -11]),
    "sddmm_coo4": ([[1, 2], [3, 4], [5, 6]], [[-1, -3], [2, 2], [3, 1]], [(0, 0, 1), (1, 0, -1), (2, 0, 1), (2, 2, 1)], 3, 3, [-7, 15, -23, 21]),
    "dummy": ([[1, 1], [1, 1]], [[1, 1], [1, 1]], [(0, 0, 1), (0, 1, 1), (1, 0, 1), (1, 1, 1)], 2, 2, [2, 2, 2, 2]),
}


@pytest.mark.parametrize("name", list(KATS))
@pytest.mark.parametrize("strategy", FP32_STRATEGIES)
def test_reference_kats_csr_and_coo(engine_factory, name, strategy):
    A, B, trip, M, N, exp = KATS[name]
    A, B = np.array(A, f32), np.array(B, f32)
    r = np.array([t[0] for t in trip], np.int32)
    c = np.array([t[1] for t in trip], np.int32)
    v = np.array([t[2] for t in trip], f32)
    _say("KAT", name, capi.STRATEGY_NAMES[strategy])
    rowptr, col, val = O.csr_from_triplets(M, r, c, v)
    got, _ = run_csr(engine_factory, rowptr, col, val, A, B, N, strategy)
    np.testing.assert_array_equal(got, np.array(exp, f32))       # small integers: exact in every order
    e = engine_factory()
    e.set_dense(A, B)
    e.set_coo(M, N, r, c, v)
    e.plan(strategy)
    e.run()
    np.testing.assert_array_equal(e.values(), np.array(exp, f32))
    e.close()


def _random_case(rng, M, N, K, density, lo=-1.0):
    mask = rng.random((M, N)) < density
    r, c = np.nonzero(mask)
    v = rng.uniform(lo, 1.0, len(r)).astype(f32)
    A = rng.uniform(lo, 1.0, (M, K)).astype(f32)
    B = rng.uniform(lo, 1.0, (N, K)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
    return rowptr, col, val, A, B


# the reference's randomized cross-checks (tests/matrix_test.cc:184-246), seeded here
RANDOM_CASES = [(500, 500, 32, 0.3), (250, 250, 32, 0.7), (10000, 10000, 32, 0.001)]


@pytest.mark.parametrize("case", RANDOM_CASES)
@pytest.mark.parametrize("strategy", FP32_STRATEGIES)
def test_random_matrices_like_the_reference_tests(engine_factory, case, strategy):
    M, N, K, d = case
    rng = np.random.default_rng(M + int(d * 1000))
    rowptr, col, val, A, B = _random_case(rng, M, N, K, d)
    _say("random", case, capi.STRATEGY_NAMES[strategy], "nnz", len(col))
    got, st = run_csr(engine_factory, rowptr, col, val, A, B, N, strategy)
    assert st.nnz == len(col)
    assert_parity(got, rowptr, col, val, A, B, exact=(strategy == capi.EXACT), what=str(case))


# every K from 1 up, powers of two, multiples of 4 that are not powers of two,
# odd K (scalar pieces) and K beyond one piece per lane
KS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 24, 31, 32, 33, 48, 64, 96, 100, 128, 160, 256, 260, 300, 512, 1024, 2048, 4097]


@pytest.mark.parametrize("K", KS)
def test_any_k(engine_factory, K):
    rng = np.random.default_rng(K)
    rowptr, col, val, A, B = _random_case(rng, 150, 130, K, 0.25)
    for strategy in (capi.FLAT, capi.ROW_WAVE, capi.SHORT_ROWS, capi.AUTO, capi.EXACT):
        _say("K", K, capi.STRATEGY_NAMES[strategy])
        got, _ = run_csr(engine_factory, rowptr, col, val, A, B, 130, strategy)
        assert_parity(got, rowptr, col, val, A, B, exact=(strategy == capi.EXACT), what="K=%d" % K)


def test_strategies_agree_bitwise(engine_factory):
    # same per-entry arithmetic in every gather kernel (density below the tile
    # path's threshold, so that AUTO is made of gather kernels only)
    rng = np.random.default_rng(77)
    for K in (32, 64, 20, 7, 128):
        rowptr, col, val, A, B = _random_case(rng, 400, 300, K, 0.08)
        a, _ = run_csr(engine_factory, rowptr, col, val, A, B, 300, capi.FLAT)
        b, _ = run_csr(engine_factory, rowptr, col, val, A, B, 300, capi.ROW_WAVE)
        c, st = run_csr(engine_factory, rowptr, col, val, A, B, 300, capi.AUTO)
        assert st.mfma_tiles == 0
        d, _ = run_csr(engine_factory, rowptr, col, val, A, B, 300, capi.SHORT_ROWS)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
        np.testing.assert_array_equal(a.view(np.uint32), c.view(np.uint32))
        np.testing.assert_array_equal(a.view(np.uint32), d.view(np.uint32))


def test_edge_shapes(engine_factory):
    rng = np.random.default_rng(5)
    K = 32
    A = rng.uniform(-1, 1, (70, K)).astype(f32)
    B = rng.uniform(-1, 1, (90, K)).astype(f32)
    cases = {}
    # empty matrix
    cases["empty"] = (np.zeros(71, np.int32), np.zeros(0, np.int32), np.zeros(0, f32))
    # single entry in the last row / last column
    rp = np.zeros(71, np.int32); rp[70] = 1
    cases["last"] = (rp, np.array([89], np.int32), np.array([2.0], f32))
    # mostly empty rows, one full row, ragged lengths 0..69
    lens = np.arange(70) % 7 == 0
    lens = np.where(lens, np.arange(70), 0); lens[33] = 90
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(90, l, replace=False)) for l in lens]).astype(np.int32)
    cases["ragged"] = (rp, col, rng.uniform(-1, 1, len(col)).astype(f32))
    # explicit zeros in S stay stored and give exact zeros
    rp = np.array([0] + [3] * 70, np.int32)
    cases["zeros"] = (rp, np.array([1, 5, 9], np.int32), np.array([0.0, 1.0, -0.0], f32))
    for name, (rowptr, col, val) in cases.items():
        for strategy in FP32_STRATEGIES:
            _say("edge", name, capi.STRATEGY_NAMES[strategy])
            got, st = run_csr(engine_factory, rowptr, col, val, A, B, 90, strategy)
            assert got.shape == (len(col),)
            if len(col):
                assert_parity(got, rowptr, col, val, A, B, exact=(strategy == capi.EXACT), what=name)
    got, _ = run_csr(engine_factory, *cases["zeros"], A, B, 90, capi.AUTO)
    assert got[0] == 0 and got[2] == 0


def test_unsorted_columns_and_duplicates_keep_entry_order(engine_factory):
    rng = np.random.default_rng(9)
    K = 16
    A = rng.uniform(-1, 1, (5, K)).astype(f32)
    B = rng.uniform(-1, 1, (6, K)).astype(f32)
    rowptr = np.array([0, 4, 4, 7, 8, 8], np.int32)
    col = np.array([5, 0, 3, 0, 2, 2, 1, 4], np.int32)   # unsorted, duplicates
    val = rng.uniform(-1, 1, 8).astype(f32)
    for strategy in FP32_STRATEGIES:
        got, _ = run_csr(engine_factory, rowptr, col, val, A, B, 6, strategy)
        assert_parity(got, rowptr, col, val, A, B, exact=(strategy == capi.EXACT))
    assert got[1] / val[1] == pytest.approx(got[3] / val[3], rel=1e-6)


def test_coo_sorted_and_unsorted(engine_factory):
    rng = np.random.default_rng(10)
    rowptr, col, val, A, B = _random_case(rng, 300, 200, 32, 0.1)
    rows = O.coo_rows_from_csr(rowptr)
    ref = O.sddmm_coo(rows, col, val, A, B)
    np.testing.assert_array_equal(ref, O.sddmm_csr(rowptr, col, val, A, B))
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    for strategy in FP32_STRATEGIES:
        e = engine_factory()
        e.set_dense(A, B)
        e.set_coo(300, 200, rows, col, val)
        e.plan(strategy)
        e.run()
        got = e.values()
        e.close()
        if strategy == capi.EXACT:
            np.testing.assert_array_equal(got.view(np.uint32), ref.view(np.uint32))
        else:
            assert O.check_values(got, ref, mag=mag)[0]
    # shuffled entries: output follows the caller's order
    p = rng.permutation(len(col))
    for strategy in (capi.AUTO, capi.FLAT, capi.EXACT):
        e = engine_factory()
        e.set_dense(A, B)
        e.set_coo(300, 200, rows[p], col[p], val[p])
        e.plan(strategy)
        e.run()
        got = e.values()
        e.close()
        assert O.check_values(got, ref[p], mag=mag[p])[0]
    e = engine_factory()
    e.set_dense(A, B)
    e.set_coo(300, 200, rows[p], col[p], val[p])
    for st in (capi.ROW_WAVE, capi.SHORT_ROWS):
        with pytest.raises(capi.SddmmError) as ei:
            e.plan(st)
        assert ei.value.code == capi.ERR_UNSUPPORTED
    e.close()


def test_error_paths_on_device(engine_factory):
    e = engine_factory()
    with pytest.raises(capi.SddmmError) as ei:
        e.run()
    assert ei.value.code == capi.ERR_STATE
    A = np.ones((4, 8), f32); B = np.ones((5, 8), f32)
    e.set_dense(A, B)
    for rowptr, col, N in [
        ([0, 2, 1, 3, 3], [0, 1, 2], 5),          # decreasing row pointer
        ([1, 2, 3, 3, 3], [0, 1, 2], 5),          # does not start at 0
        ([0, 1, 2, 3, 2], [0, 1, 2], 5),          # rowptr[M] != nnz
        ([0, 1, 2, 3, 3], [0, 1, 5], 5),          # column out of range
        ([0, 1, 2, 3, 3], [0, -1, 2], 5),
    ]:
        with pytest.raises(capi.SddmmError) as ei:
            e.set_csr(4, N, np.array(rowptr, np.int32), np.array(col, np.int32), np.ones(len(col), f32))
        assert ei.value.code == capi.ERR_PATTERN
    with pytest.raises(capi.SddmmError) as ei:
        e.set_coo(4, 5, np.array([0, 4], np.int32), np.array([0, 0], np.int32), np.ones(2, f32))
    assert ei.value.code == capi.ERR_PATTERN
    # more entries than 32-bit positions (with look-ahead room) hold: refused before any array is read
    tiny = np.zeros(8, np.int32)
    assert e.L.sddmm_set_csr(e.h, 4, 5, 2 ** 31 - 1000, capi._ptr(tiny), capi._ptr(tiny),
                             capi._ptr(tiny.view(f32))) == capi.ERR_INVALID
    # S larger than the dense operands
    e.set_csr(6, 5, np.zeros(7, np.int32), np.zeros(0, np.int32), np.zeros(0, f32))
    with pytest.raises(capi.SddmmError) as ei:
        e.plan(capi.AUTO)
    assert ei.value.code == capi.ERR_INVALID
    with pytest.raises(capi.SddmmError) as ei:
        e.set_dense(np.ones((4, 12), np.uint16), np.ones((5, 12), np.uint16), capi.BF16)
    assert ei.value.code == capi.ERR_INVALID
    # a context stays usable after errors
    e.set_dense(A, B)
    e.set_csr(4, 5, np.array([0, 1, 1, 1, 2], np.int32), np.array([0, 4], np.int32), np.array([2, 3], f32))
    e.run()
    np.testing.assert_array_equal(e.values(), np.array([16, 24], f32))
    e.close()


def test_context_reuse_and_update_values(engine_factory):
    # the harness reuses one competitor object for many runs and datasets
    rng = np.random.default_rng(12)
    e = engine_factory()
    for M, N, K in [(100, 80, 32), (30, 200, 8), (100, 80, 32)]:
        rowptr, col, val, A, B = _random_case(rng, M, N, K, 0.2)
        e.set_dense(A, B)
        e.set_csr(M, N, rowptr, col, val)
        e.plan(capi.AUTO)
        e.run()
        assert_parity(e.values(), rowptr, col, val, A, B)
        e.run()                                       # idempotent
        assert_parity(e.values(), rowptr, col, val, A, B)
        val2 = (val * f32(2)).astype(f32)
        p1 = e.values()
        e.update_values(val2)
        e.run()
        np.testing.assert_array_equal(e.values(), p1 * f32(2))   # linear in S, exactly for a factor 2
    e.close()


def test_one_context_across_patterns_of_different_sizes(engine_factory):
    """One context, as the harness keeps one competitor object: patterns with more and fewer
    rows, entries, tiles and panels in turn.  The plan's work arrays are sized for the largest
    pattern seen; a smaller one after a larger one must not see what the larger one left."""
    e = engine_factory()
    order = ["mixed_density", "small_uniform", "fem_banded", "dense_tiles", "small_uniform", "mixed_density",
             "power_law", "fem_banded"]
    for name in order:
        w = W.make(name, "small", K=32)
        e.set_dense(w.A, w.B)
        e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
        for strategy in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
            e.plan(strategy)
            e.run()
            st = e.stats()
            assert_parity(e.values(), w.rowptr, w.col, w.sval, w.A, w.B, what="%s after others" % name)
            if st.strategy_used in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
                assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == w.nnz
        e.plan(capi.AUTO)
        got_o = e.run_fused()
        ref_p, ref_o = O.fusedmm_csr(w.rowptr, w.col, w.sval, w.A, w.B)
        _, mag_o = O.fusedmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
        ok, worst, i = O.check_values(got_o[:w.M].ravel(), ref_o.ravel(), mag=mag_o.ravel())
        assert ok, (name, i, worst)
    e.close()


@pytest.mark.parametrize("name", ["fem_banded", "mixed_density", "similar_rows"])
def test_non_finite_operands_stay_in_their_own_entries(engine_factory, name):
    """A NaN in one B row and an infinity in one A row: exactly the entries that involve
    them are non-finite, as in the CPU loop; the matrix-core paths compute whole tiles and
    panels, and nothing of a poisoned row or column may leak into its neighbours."""
    w = W.make(name, "small", K=32)
    A, B = w.A.copy(), w.B.copy()
    rows_of = np.repeat(np.arange(w.M), np.diff(w.rowptr))
    bad_col = int(w.col[len(w.col) // 2])
    bad_row = int(rows_of[len(w.col) // 3])
    B[bad_col, 5] = np.nan
    A[bad_row, 7] = np.inf
    with np.errstate(all="ignore"):
        ref = O.sddmm_csr(w.rowptr, w.col, w.sval, A, B, threads=0)
    poisoned = (w.col == bad_col) | (rows_of == bad_row)
    assert poisoned.any() and np.array_equal(~np.isfinite(ref), poisoned)
    clean = ~poisoned
    _, mag = O.sddmm_csr_f64(w.rowptr[:], w.col, np.where(clean, w.sval, 0).astype(f32), w.A, w.B)
    for strategy in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED, capi.FLAT, capi.ROW_WAVE):
        got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, A, B, w.N, strategy)
        what = "%s %s" % (name, capi.STRATEGY_NAMES[strategy])
        assert np.array_equal(~np.isfinite(got), poisoned), what
        assert np.array_equal(np.isnan(got), np.isnan(ref)), what
        ok, worst, i = O.check_values(got[clean], ref[clean], mag=mag[clean])
        assert ok, (what, i, worst)


@pytest.mark.parametrize("name", ["fem_banded", "mixed_density"])
def test_denormal_results_are_not_flushed(engine_factory, name):
    """Operands of magnitude 1e-20: every product and every result is a denormal fp32
    number.  The CPU loop keeps them; so must the vector and the matrix-core paths.
    Sums of denormals are exact, so the only differences allowed are the roundings of
    the K products (one step of 2^-149 each, fused or not)."""
    K = 32
    w = W.make(name, "small", K=K)
    A = (w.A * f32(1e-20)).astype(f32)
    B = (w.B * f32(1e-20)).astype(f32)
    ref = O.sddmm_csr(w.rowptr, w.col, w.sval, A, B, threads=0)
    assert 0 < float(np.abs(ref).max()) < 1.17e-38 and np.count_nonzero(ref) > 0.99 * len(ref)
    for strategy in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED, capi.FLAT, capi.EXACT):
        got, _ = run_csr(engine_factory, w.rowptr, w.col, w.sval, A, B, w.N, strategy)
        what = "%s %s" % (name, capi.STRATEGY_NAMES[strategy])
        assert np.count_nonzero(got) >= np.count_nonzero(ref) - 5, what
        assert float(np.abs(got.astype(np.float64) - ref).max()) <= (K + 1) * 2.0 ** -149, what


def test_replaced_operands_are_planned_again_as_last_asked(engine_factory):
    rng = np.random.default_rng(14)
    e = engine_factory()
    rowptr, col, val, A, B = _random_case(rng, 200, 150, 32, 0.3)
    e.set_dense(A, B)
    e.set_csr(200, 150, rowptr, col, val)
    e.run()                                           # never planned: AUTO
    assert e.stats().strategy_used in (capi.AUTO, capi.FLAT)
    assert_parity(e.values(), rowptr, col, val, A, B)
    e.plan(capi.ROW_WAVE)
    for M, N, K in [(90, 300, 16), (400, 60, 32)]:
        rowptr, col, val, A, B = _random_case(rng, M, N, K, 0.25)
        e.set_dense(A, B)
        e.set_csr(M, N, rowptr, col, val)             # drops the plan
        e.launch()
        e.synchronize()
        assert_parity(e.values(), rowptr, col, val, A, B)
        e.run()
        assert e.stats().strategy_used == capi.ROW_WAVE
    e.close()


def test_new_dense_values_of_the_same_shape_keep_the_plan(engine_factory):
    # iterations of a solver: the same S, new A and B every time
    rng = np.random.default_rng(15)
    w = W.make("mixed_density", "small", K=32)
    e = engine_factory()
    e.set_dense(w.A, w.B)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    e.plan(capi.AUTO)
    planned = e.stats().plan_ms
    assert planned > 0
    for it in range(3):
        A = rng.uniform(-1, 1, w.A.shape).astype(f32)
        B = rng.uniform(-1, 1, w.B.shape).astype(f32)
        e.set_dense(A, B)
        e.run()
        assert e.stats().plan_ms == planned                    # no new plan was made
        assert_parity(e.values(), w.rowptr, w.col, w.sval, A, B, what="iteration %d" % it)
    # another width is another plan
    A = rng.uniform(-1, 1, (w.M, 64)).astype(f32)
    B = rng.uniform(-1, 1, (w.N, 64)).astype(f32)
    e.set_dense(A, B)
    e.run()
    assert e.stats().plan_ms != planned
    assert_parity(e.values(), w.rowptr, w.col, w.sval, A, B, what="K=64")
    e.close()


def test_distinct_contexts_on_distinct_threads(engine_factory):
    """A context is single-threaded, but two contexts driven from two host threads at
    once (each on its own stream) must not disturb each other: every result of every
    round is checked, with a different matrix, width and strategy mix per thread."""
    import threading

    cases = {}
    for t, (wl, K) in enumerate([("fem_banded", 32), ("mixed_density", 64), ("similar_rows", 32)]):
        w = W.make(wl, "small", K=K)
        cases[t] = (w, O.sddmm_csr(w.rowptr, w.col, w.sval, w.A, w.B, threads=0),
                    O.sddmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)[1])
    engines = {t: engine_factory() for t in cases}
    errors = []

    def drive(t):
        try:
            w, ref, mag = cases[t]
            e = engines[t]
            for rnd in range(6):
                e.set_dense(w.A, w.B)
                e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
                e.plan([capi.AUTO, capi.FLAT, capi.MFMA_TILE][(rnd + t) % 3])
                e.run()
                ok, worst, i = O.check_values(e.values(), ref, mag=mag, rtol=1e-5)
                if not ok:
                    errors.append("thread %d round %d: entry %d off by %.2f x tolerance" % (t, rnd, i, worst))
                    return
        except Exception as ex:                       # surfaced by the assert below
            errors.append("thread %d: %r" % (t, ex))

    threads = [threading.Thread(target=drive, args=(t,)) for t in cases]
    for th in threads:
        th.start()
    for th in threads:
        th.join(120)
    assert not any(th.is_alive() for th in threads), "a thread did not finish"
    assert not errors, errors


def test_timing_entry_points(engine_factory):
    """Per-launch events and one event pair around a stream of launches: both leave
    the result intact, both report positive times, and a launch inside a stream is
    not slower than a launch that has to start from an idle device."""
    rng = np.random.default_rng(13)
    rowptr, col, val, A, B = _random_case(rng, 600, 500, 32, 0.2)
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(600, 500, rowptr, col, val)
    e.plan(capi.AUTO)
    each = e.time_runs(2, 20)
    assert each.shape == (20,) and (each > 0).all()
    total = min(e.time_region(20) for _ in range(3))
    assert 0 < total / 20 <= float(np.median(each)) * 1.5
    assert e.time_region(3, include_plan=True) > 0
    assert_parity(e.values(), rowptr, col, val, A, B)
    with pytest.raises(capi.SddmmError):
        e.time_region(0)
    e.close()


@pytest.mark.parametrize("name", ["small_uniform", "fem_banded", "power_law", "mixed_density"])
def test_benchmark_shapes_scaled_down(engine_factory, name):
    w = W.make(name, "small")
    for strategy in FP32_STRATEGIES:
        _say("shape", name, capi.STRATEGY_NAMES[strategy], "nnz", w.nnz)
        got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, strategy)
        assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, exact=(strategy == capi.EXACT), what=name)
        assert st.flops == 2.0 * w.nnz * w.K
        assert st.bytes_gathered == w.bytes_gathered()
        if strategy == capi.AUTO and name in ("power_law", "small_uniform"):
            assert st.mfma_tiles == 0          # nothing there is dense enough for the tile path
        if strategy == capi.AUTO and name == "mixed_density":
            # no 16 consecutive rows share tiles, but the near-dense rows gathered by
            # column window do: most of their entries end up on the matrix cores
            dense_nnz = int(np.diff(w.rowptr)[np.diff(w.rowptr) >= 64].sum())
            assert st.mfma_tiles > 0 and st.nnz_mfma > 0.8 * dense_nnz
            assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == w.nnz


@pytest.mark.parametrize("K", [32, 128])
def test_bf16_inputs_gather_path(engine_factory, K):
    w = W.make("dense_tiles", "small", K=K)
    for strategy in (capi.FLAT, capi.ROW_WAVE, capi.SHORT_ROWS, capi.AUTO, capi.EXACT):
        _say("bf16", K, capi.STRATEGY_NAMES[strategy])
        got, _ = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A_bits, w.B_bits, w.N, strategy, capi.BF16)
        # products of bf16 values are exact in fp32, accumulation is fp32: the fp32 bar applies
        assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, rtol=1e-5, exact=(strategy == capi.EXACT), what="bf16")


@pytest.mark.parametrize("K", [8, 32, 128, 512, 1032])
def test_f16_inputs(engine_factory, K):
    """IEEE half inputs with fp32 accumulation on every path (gather kernels with
    v_dot2c_f32_f16, dense tiles on v_mfma_f32_16x16x32_f16).  Products of halves are
    exact in fp32, so the fp32 bar applies; EXACT is bit-identical to the oracle on
    the half-rounded inputs."""
    w = W.make("dense_tiles", "small", K=K, bf16=False)
    Ab, Bb = capi.to_f16(w.A).reshape(w.M, K), capi.to_f16(w.B).reshape(w.N, K)
    A, B = capi.from_f16(Ab).reshape(w.M, K), capi.from_f16(Bb).reshape(w.N, K)
    tiled = (2 * K) % 64 == 0 and 2 * K <= 1024
    for strategy in (capi.FLAT, capi.ROW_WAVE, capi.SHORT_ROWS, capi.AUTO, capi.MFMA_TILE, capi.EXACT):
        _say("f16", K, capi.STRATEGY_NAMES[strategy])
        got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, Ab, Bb, w.N, strategy, capi.F16)
        assert_parity(got, w.rowptr, w.col, w.sval, A, B, rtol=1e-5, exact=(strategy == capi.EXACT), what="f16 K=%d" % K)
        if strategy in (capi.AUTO, capi.MFMA_TILE):
            assert (st.mfma_tiles == w.meta["tiles"]) == tiled and (st.mfma_tiles == 0) == (not tiled)
    # K must be a multiple of 8 for 16-bit operands
    e = engine_factory()
    with pytest.raises(capi.SddmmError):
        e.set_dense(np.zeros((4, 12), np.uint16), np.zeros((4, 12), np.uint16), capi.F16)
    e.close()


def test_auto_resolves_to_flat_when_short_rows_dominate(engine_factory):
    w = W.make("power_law", "small")
    got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.AUTO)
    assert st.strategy_used == capi.FLAT
    flat, _ = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.FLAT)
    np.testing.assert_array_equal(got.view(np.uint32), flat.view(np.uint32))
    assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B)


def test_auto_row_classes_and_segments(engine_factory, monkeypatch):
    """AUTO: rows below the short threshold go to the many-rows kernel, the rest to
    wave-per-segment items; very long rows are cut into several segments."""
    monkeypatch.setenv("SDDMM_FLAT_AVG", "0")            # keep the row split whatever the average row length
    rng = np.random.default_rng(21)
    M, N, K = 1000, 6000, 32
    lens = rng.integers(0, 20, M)
    lens[::50] = rng.integers(30, 300, len(lens[::50]))
    lens[7] = 5000                                       # several segments
    lens[500] = 0
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(N, l, replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    got, st = run_csr(engine_factory, rowptr, col, val, A, B, N, capi.AUTO)
    assert_parity(got, rowptr, col, val, A, B, what="auto classes")
    assert st.strategy_used == capi.AUTO and st.kernels_launched == 1
    ts, seg = 24, 256
    assert st.rows_short == np.count_nonzero((lens > 0) & (lens < ts))
    assert st.nnz_short == lens[lens < ts].sum()
    assert st.rows_long == np.count_nonzero(lens > seg) >= 1
    assert st.rows_medium == np.count_nonzero((lens >= ts) & (lens <= seg))
    assert st.nnz_short + st.nnz_medium + st.nnz_long == len(col)
    assert st.rows_nonempty == np.count_nonzero(lens)
    assert st.mfma_tiles == 0
    ref = run_csr(engine_factory, rowptr, col, val, A, B, N, capi.FLAT)[0]
    np.testing.assert_array_equal(got.view(np.uint32), ref.view(np.uint32))


# ---- dense-tile (MFMA) path ------------------------------------------------------
def _tile_count(rowptr, col, M):
    rows = np.repeat(np.arange(M), np.diff(rowptr))
    return len(np.unique((rows // 16).astype(np.int64) * (1 << 32) + (col // 16)))


@pytest.mark.parametrize("K", [32, 128, 512])
def test_mfma_tiles_bf16(engine_factory, K):
    """bf16 inputs, fully dense 16x16 tiles.  Products of bf16 values are exact in
    fp32 and the accumulator is fp32, so the result is held to the fp32 bar
    (1e-5 with the magnitude floor), well inside the 1e-2 allowed for this path."""
    w = W.make("dense_tiles", "small", K=K)
    for strategy in (capi.AUTO, capi.MFMA_TILE):
        _say("mfma bf16", K, capi.STRATEGY_NAMES[strategy])
        got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A_bits, w.B_bits, w.N, strategy, capi.BF16)
        assert st.mfma_tiles == w.meta["tiles"] and st.nnz_mfma == w.nnz
        assert st.kernels_launched == 1
        assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, rtol=1e-5, what="mfma bf16 K=%d" % K)


@pytest.mark.parametrize("K", [16, 32, 64, 128, 256])
def test_mfma_tiles_fp32(engine_factory, K):
    w = W.make("dense_tiles", "small", K=K, bf16=False)
    for strategy in (capi.AUTO, capi.MFMA_TILE):
        _say("mfma f32", K, capi.STRATEGY_NAMES[strategy])
        got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, strategy)
        assert st.mfma_tiles == w.meta["tiles"] and st.nnz_mfma == w.nnz
        assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, what="mfma f32 K=%d" % K)


def test_tiles_partial_fill_ragged_edges_and_mixed_strips(engine_factory, monkeypatch):
    """Strips of every kind in one matrix: full tiles, partly filled tiles, 8x8
    blocks, strips too sparse for the tile path, an unsorted row (its strip must
    stay on the gather kernels), M and N not multiples of 16."""
    rng = np.random.default_rng(33)
    M, N, K = 16 * 9 + 5, 16 * 13 + 7, 32
    dense = np.zeros((M, N), bool)
    dense[0:16, 32:64] = True                                  # strip 0: two full tiles
    dense[16:32, :] = rng.random((16, N)) < 0.5                # strip 1: half filled everywhere
    for b in range(4):                                         # strip 2: 8x8 blocks
        dense[32 + 8 * (b % 2):40 + 8 * (b % 2), 16 * b + 8 * (b % 2):16 * b + 8 * (b % 2) + 8] = True
    dense[48:64, :] = rng.random((16, N)) < 0.02               # strip 3: sparse -> gather
    dense[64:80, 100:180] = rng.random((16, 80)) < 0.7         # strip 4: unsorted row below
    dense[80:96, N - 7:] = True                                # strip 5: last, partial tile column
    dense[128:, 0:40] = rng.random((M - 128, 40)) < 0.6        # last strip has only 5+16 rows
    r, c = np.nonzero(dense)
    v = rng.uniform(-1, 1, len(r)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
    s, e = rowptr[70], rowptr[71]
    assert e - s >= 2
    col[s], col[s + 1] = col[s + 1], col[s]                    # row 70 no longer sorted
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    for strategy in (capi.AUTO, capi.MFMA_TILE):
        got, st = run_csr(engine_factory, rowptr, col, val, A, B, N, strategy)
        assert_parity(got, rowptr, col, val, A, B, what="mixed strips")
        assert st.mfma_tiles > 0 and 0 < st.nnz_mfma < len(col)
        extra = 1 if st.panels else 0                            # the panel kernel is a launch of its own
        assert st.kernels_launched == 1 + extra                  # tiles and rows share one launch at this row size
        monkeypatch.setenv("SDDMM_FUSE", "0")
        got2, st2 = run_csr(engine_factory, rowptr, col, val, A, B, N, strategy)
        monkeypatch.delenv("SDDMM_FUSE")
        assert st2.kernels_launched == 2 + extra
        np.testing.assert_array_equal(got.view(np.uint32), got2.view(np.uint32))
    rows = np.repeat(np.arange(M), np.diff(rowptr))
    forced = rows // 16 != 4                                   # MFMA_TILE: every strip but the unsorted one
    assert st.nnz_mfma == np.count_nonzero(forced)
    assert st.mfma_tiles == _tile_count(rowptr, col, M) - len(np.unique(col[rows // 16 == 4] // 16))
    # AUTO takes only the strips whose tiles are well filled
    _, st_auto = run_csr(engine_factory, rowptr, col, val, A, B, N, capi.AUTO)
    assert 0 < st_auto.nnz_mfma < st.nnz_mfma
    assert st_auto.nnz_mfma >= np.count_nonzero(rows // 16 == 0)


def test_tile_strips_wider_than_the_classifier_bitmap(engine_factory):
    """A strip whose columns span more than 524288 columns does not fit the
    classifier's per-strip bitmap and is merged row by row instead; strips inside
    the limit in the same matrix take the bitmap route.  Both must describe the same
    tiles the host counts."""
    rng = np.random.default_rng(35)
    M, N, K = 16 * 5, 700_003, 16
    r_list, c_list = [], []
    def block(r0, r1, c0, c1, fill=1.0):
        m = rng.random((r1 - r0, c1 - c0)) < fill
        rr, cc = np.nonzero(m)
        r_list.append(rr + r0); c_list.append(cc + c0)
    block(0, 16, 0, 48); block(0, 16, N - 40, N)              # strip 0: both ends of a 700k-column span
    block(16, 32, 1000, 1064, 0.8)                             # strip 1: narrow
    block(32, 48, 5, 37, 0.9); block(32, 48, 600_000, 600_050, 0.9)   # strip 2: wide, partly filled
    block(48, 64, 0, N, 0.00002)                               # strip 3: scattered -> gather kernels
    block(64, 80, 524_288, 524_288 + 16 * 40, 0.7)             # strip 4: narrow span far from column 0
    r = np.concatenate(r_list).astype(np.int32); c = np.concatenate(c_list).astype(np.int32)
    v = rng.uniform(-1, 1, len(r)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r, c, v)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    rows = np.repeat(np.arange(M), np.diff(rowptr))
    got, st = run_csr(engine_factory, rowptr, col, val, A, B, N, capi.MFMA_TILE)
    assert_parity(got, rowptr, col, val, A, B, what="wide strips, forced")
    assert st.mfma_tiles == _tile_count(rowptr, col, M) and st.nnz_mfma == len(col)
    got, st = run_csr(engine_factory, rowptr, col, val, A, B, N, capi.AUTO)
    assert_parity(got, rowptr, col, val, A, B, what="wide strips, auto")
    keep = rows // 16 != 3
    assert st.nnz_mfma == np.count_nonzero(keep)
    assert st.mfma_tiles == _tile_count(rowptr, col, M) - len(np.unique(col[~keep] // 16))


def test_tile_path_not_applicable_falls_back_to_gather(engine_factory):
    # K*4 not a multiple of 64 bytes, and bf16 with K=8: everything on the gather kernels
    rng = np.random.default_rng(34)
    w = W.make("dense_tiles", "small", K=24, bf16=False)
    got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.MFMA_TILE)
    assert st.mfma_tiles == 0 and st.nnz_mfma == 0
    assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B)


def test_fem_blocks_tiles_and_panels(engine_factory, monkeypatch):
    w = W.make("fem_banded", "small")
    got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.MFMA_TILE)
    assert st.nnz_mfma == w.nnz and st.mfma_tiles == _tile_count(w.rowptr, w.col, w.M)
    assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, what="fem tiles")
    # every block row is an 8-row panel with one column list
    got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.LDS_TILED)
    assert st.panels == w.M // 8 and st.nnz_panel == w.nnz and st.mfma_tiles == 0
    assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, what="fem panels (MFMA kernel)")
    # the VALU panel kernel has the per-entry arithmetic of the gather kernels
    monkeypatch.setenv("SDDMM_PANEL_MFMA", "0")
    got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.LDS_TILED)
    assert st.panels == w.M // 8 and st.nnz_panel == w.nnz
    flat, _ = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.FLAT)
    np.testing.assert_array_equal(got.view(np.uint32), flat.view(np.uint32))
    monkeypatch.delenv("SDDMM_PANEL_MFMA")
    got, st = run_csr(engine_factory, w.rowptr, w.col, w.sval, w.A, w.B, w.N, capi.AUTO)
    assert st.nnz_mfma + st.nnz_panel == w.nnz
    assert_parity(got, w.rowptr, w.col, w.sval, w.A, w.B, what="fem auto")


@pytest.mark.parametrize("K,dtype", [(32, "f32"), (64, "f32"), (128, "f32"), (256, "f32"), (64, "bf16"), (256, "bf16"),
                                     (24, "f32"), (33, "f32"), (32, "f16"), (64, "f16"), (512, "f16")])
def test_row_panels(engine_factory, monkeypatch, K, dtype):
    """Groups of identical rows: aligned 8-row panels are taken, everything else
    (unaligned groups, groups of other sizes, rows with one differing column, short
    lists, the ragged tail) stays on the row kernels."""
    rng = np.random.default_rng(100 + K)
    N = 700
    rows_cols = []

    def add_group(n_rows, length):
        cols = np.sort(rng.choice(N, length, replace=False))
        for _ in range(n_rows):
            rows_cols.append(cols.copy())

    add_group(8, 300)          # rows 0-7    panel (several work items when SDDMM_PANEL_SEG is small)
    add_group(8, 70)           # rows 8-15   panel
    add_group(3, 40)           # rows 16-18  too few rows ...
    add_group(8, 40)           # rows 19-26  ... and this group is not 8-aligned
    add_group(5, 0)            # rows 27-31  empty rows
    add_group(16, 33)          # rows 32-47  two panels
    add_group(8, 50)           # rows 48-55  one row differs in one column below
    add_group(8, 9)            # rows 56-63  shorter than AUTO's minimum (still a panel for LDS_TILED)
    add_group(5, 20)           # rows 64-68  ragged tail
    c = rows_cols[51].copy()
    c[7] = np.setdiff1d(np.arange(N), c)[5]                # a column the group does not have
    rows_cols[51] = np.sort(c)
    M = len(rows_cols)
    lens = np.array([len(x) for x in rows_cols])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows_cols).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    if dtype == "bf16":
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        A, B = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K)
        ops, dt = (Ab, Bb), capi.BF16
    elif dtype == "f16":
        Ab, Bb = capi.to_f16(A).reshape(M, K), capi.to_f16(B).reshape(N, K)
        A, B = capi.from_f16(Ab).reshape(M, K), capi.from_f16(Bb).reshape(N, K)
        ops, dt = (Ab, Bb), capi.F16
    else:
        ops, dt = (A, B), capi.F32
    row_bytes = K * (4 if dtype == "f32" else 2)
    applicable = row_bytes % 64 == 0                                         # the MFMA panel kernel
    valu_applicable = (dtype, K) in (("f32", 32), ("f32", 64), ("bf16", 64), ("f16", 64))  # A rows of a panel fit in registers
    same = len(rows_cols[51]) == 50 and np.array_equal(rows_cols[51], rows_cols[48])
    assert not same
    for strategy, min_len in ((capi.LDS_TILED, 1), (capi.AUTO, 16)):
        _say("panels", K, dtype, capi.STRATEGY_NAMES[strategy])
        got, st = run_csr(engine_factory, rowptr, col, val, *ops, N, strategy, dt)
        assert_parity(got, rowptr, col, val, A, B, what="panels K=%d" % K)
        if strategy == capi.LDS_TILED:
            exp = [(0, 300), (8, 70), (32, 33), (40, 33), (56, 9)] if applicable else []
            assert st.panels == len(exp) and st.nnz_panel == sum(8 * l for _, l in exp)
            assert st.mfma_tiles == 0
            st_lds = st
    # column lists cut into several work items, at boundaries that are and are not multiples of 4
    for seg in ("96", "100", "67"):
        monkeypatch.setenv("SDDMM_PANEL_SEG", seg)
        got, st2 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.LDS_TILED, dt)
        assert_parity(got, rowptr, col, val, A, B, what="panels K=%d in segments of %s" % (K, seg))
        assert st2.panels == st_lds.panels and st2.nnz_panel == st_lds.nnz_panel
    monkeypatch.delenv("SDDMM_PANEL_SEG")
    monkeypatch.setenv("SDDMM_PANEL_MFMA", "0")
    lds, st = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.LDS_TILED, dt)
    assert_parity(lds, rowptr, col, val, A, B, what="VALU panels K=%d" % K)
    assert (st.panels == 5) == valu_applicable and (st.panels == 0) == (not valu_applicable)
    flat, _ = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.FLAT, dt)
    np.testing.assert_array_equal(flat.view(np.uint32), lds.view(np.uint32))


@pytest.mark.parametrize("K,dtype", [(32, "f32"), (128, "f32"), (64, "bf16"), (256, "f16")])
def test_gathered_strips(engine_factory, monkeypatch, K, dtype):
    """Near-dense rows scattered over S: no 16 consecutive rows share tiles, but the
    rows sorted by their first column do.  Ties in the first column, a candidate count
    that is not a multiple of 16, one unsorted candidate and rows too short or too
    spread out to be candidates are all in the mix."""
    rng = np.random.default_rng(400 + K)
    M, N = 1000, 5000
    rows = [np.sort(rng.choice(N, int(rng.integers(1, 12)), replace=False)) for _ in range(M)]
    dense_rows = np.sort(rng.choice(M, 203, replace=False))               # 203 = 12 strips of 16 + 11
    starts = rng.choice([100, 100, 100, 900, 2500, 2500, 4000], len(dense_rows))   # many equal first columns
    for r, s0 in zip(dense_rows, starts):
        c = s0 + np.nonzero(rng.random(400) < 0.6)[0]
        c[0] = s0                                                          # the first column itself: ties
        rows[r] = np.unique(c)
    spread = [int(x) for x in rng.choice(np.setdiff1d(np.arange(M), dense_rows), 20, replace=False)]
    for r in spread:                                                       # long but not compact: no candidates
        rows[r] = np.sort(rng.choice(N, 200, replace=False))
    bad = int(dense_rows[7])
    rows[bad] = np.concatenate([rows[bad][:5], rows[bad][5:7][::-1], rows[bad][7:]])   # one candidate is not sorted
    lens = np.array([len(x) for x in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    if dtype == "bf16":
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        A, B, ops, dt = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K), (Ab, Bb), capi.BF16
    elif dtype == "f16":
        Ab, Bb = capi.to_f16(A).reshape(M, K), capi.to_f16(B).reshape(N, K)
        A, B, ops, dt = capi.from_f16(Ab).reshape(M, K), capi.from_f16(Bb).reshape(N, K), (Ab, Bb), capi.F16
    else:
        ops, dt = (A, B), capi.F32
    got, st = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert_parity(got, rowptr, col, val, A, B, what="gathered strips")
    dense_nnz = int(lens[dense_rows].sum())
    # of the 13 strips, the one with the unsorted row and up to three that straddle two
    # windows (too few entries per tile) may be given up
    assert st.mfma_tiles > 0 and 0.6 * dense_nnz <= st.nnz_mfma <= dense_nnz
    assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == len(col)
    assert st.kernels_launched == 1
    monkeypatch.setenv("SDDMM_FUSE", "0")
    two, st2 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert st2.kernels_launched == 2 and st2.nnz_mfma <= dense_nnz
    assert_parity(two, rowptr, col, val, A, B, what="gathered strips, two launches")
    monkeypatch.setenv("SDDMM_GATHERED", "0")
    off, st3 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert st3.mfma_tiles == 0
    assert_parity(off, rowptr, col, val, A, B, what="gathered strips off")


@pytest.mark.parametrize("K,dtype,n_dense_strips", [(32, "f32", 1), (32, "f32", 2), (64, "f32", 3), (64, "bf16", 2),
                                                    (128, "f32", 1), (256, "f16", 2)])
def test_gathered_pairs_behind_other_tiles(engine_factory, monkeypatch, K, dtype, n_dense_strips):
    """Gathered strips come in pairs that share their B tiles (rows of up to 256 bytes: one
    wavefront per two windows), and their descriptors start a window of their own: with 16-row
    strips of fully dense tiles ahead of them whose tile count is not a multiple of four, the
    window in between is filled with descriptors that stand for nothing.  Candidate counts of 1..3
    strips and a half: a last pair without a second strip, and pairs whose two strips reach over
    different tile columns."""
    rng = np.random.default_rng(900 + K + n_dense_strips)
    M, N = 16 * n_dense_strips + 700, 4000
    rows = [np.sort(rng.choice(N, int(rng.integers(1, 10)), replace=False)) for _ in range(M)]
    n_tiles_dense = 0
    for sidx in range(n_dense_strips):                     # 16-row strips of 1, 2, 3 .. dense tiles: 1, 3, 6 in all
        tcs = np.sort(rng.choice(N // 16, sidx + 1, replace=False))
        cols = np.concatenate([16 * t + np.arange(16) for t in tcs])
        for r in range(16 * sidx, 16 * sidx + 16):
            rows[r] = cols.copy()
        n_tiles_dense += len(tcs)
    assert n_tiles_dense % 4 != 0
    pool = np.arange(16 * n_dense_strips, M)
    dense_rows = np.sort(rng.choice(pool, 16 * 3 + 9 + 32 * (K % 3), replace=False))
    for r in dense_rows:
        s0 = int(rng.choice([200, 1500, 1500, 2600]))
        c = s0 + int(rng.integers(0, 40)) + np.nonzero(rng.random(500) < 0.55)[0]
        rows[r] = np.unique(c)
    lens = np.array([len(x) for x in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    if dtype == "bf16":
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        A, B, ops, dt = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K), (Ab, Bb), capi.BF16
    elif dtype == "f16":
        Ab, Bb = capi.to_f16(A).reshape(M, K), capi.to_f16(B).reshape(N, K)
        A, B, ops, dt = capi.from_f16(Ab).reshape(M, K), capi.from_f16(Bb).reshape(N, K), (Ab, Bb), capi.F16
    else:
        ops, dt = (A, B), capi.F32
    dense_nnz = int(lens[dense_rows].sum())
    strips_nnz = int(lens[:16 * n_dense_strips].sum())
    _say("gathered pairs", K, dtype, n_dense_strips)
    got, st = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert_parity(got, rowptr, col, val, A, B, what="pairs behind %d dense tiles" % n_tiles_dense)
    assert st.nnz_mfma >= strips_nnz + 0.6 * dense_nnz and st.mfma_tiles > n_tiles_dense
    assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == len(col)
    # the same plan, one wavefront per window
    monkeypatch.setenv("SDDMM_PAIRS", "0")
    one, st1 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert st1.mfma_tiles == st.mfma_tiles and st1.nnz_mfma == st.nnz_mfma
    np.testing.assert_array_equal(one.view(np.uint32), got.view(np.uint32))
    # and tile by tile from the descriptors
    monkeypatch.setenv("SDDMM_WINDOW_FILL", "1")
    walk, st2 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert st2.mfma_tiles == st.mfma_tiles
    assert_parity(walk, rowptr, col, val, A, B, what="pairs, tile by tile")
    monkeypatch.delenv("SDDMM_WINDOW_FILL")
    monkeypatch.delenv("SDDMM_PAIRS")
    # the candidates ordered by the library's radix sort instead of by their ranks: the same plan, the same bits
    monkeypatch.setenv("SDDMM_RANK_SORT", "0")
    radix, st3 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert st3.mfma_tiles == st.mfma_tiles and st3.nnz_mfma == st.nnz_mfma
    np.testing.assert_array_equal(radix.view(np.uint32), got.view(np.uint32))


def _host_union_model(M, rowptr, col, min_fill, span_limit=131072):
    """Union strips as the device must find them when no other path owns a row: a
    16-row strip is taken iff its rows are strictly increasing, its column span fits
    the classifier and it holds at least min_fill entries per tile of 16 union columns."""
    tiles = entries = 0
    for s in range((M + 15) // 16):
        lo, hi = rowptr[s * 16], rowptr[min(M, s * 16 + 16)]
        if hi - lo < min_fill:
            continue
        rows = [col[rowptr[r]:rowptr[r + 1]].astype(np.int64) for r in range(s * 16, min(M, s * 16 + 16))]
        if any(len(c) > 1 and (np.diff(c) <= 0).any() for c in rows):
            continue
        u = np.unique(np.concatenate(rows))
        if u[-1] - u[0] + 1 > span_limit:
            continue
        t = (len(u) + 15) // 16
        if hi - lo >= min_fill * t:
            tiles += t
            entries += hi - lo
    return tiles, entries


@pytest.mark.parametrize("K,dtype", [(32, "f32"), (128, "f32"), (64, "bf16")])
def test_union_strips(engine_factory, monkeypatch, K, dtype):
    """Rows that share most of their columns without being identical or aligned to
    16-column blocks: the tiles are cut from the union of the strip's columns."""
    monkeypatch.setenv("SDDMM_GATHERED", "0")
    rng = np.random.default_rng(600 + K)
    M, N = 16 * 40 + 5, 300_000
    rows = []
    for g in range(M // 16 + 1):
        kind = g % 5
        if kind == 0:                                    # 16 similar rows, scattered base
            base = np.sort(rng.choice(60_000, 150, replace=False)) + int(rng.integers(0, N - 60_000))
            grp = [base[rng.random(150) > 0.15] for _ in range(16)]
        elif kind == 1:                                  # two different groups of 8 similar rows
            grp = []
            for _ in range(2):
                base = np.sort(rng.choice(5_000, 120, replace=False)) + int(rng.integers(0, N - 5_000))
                grp += [base[rng.random(120) > 0.1] for _ in range(8)]
        elif kind == 2:                                  # unrelated rows: the union is as large as the strip
            grp = [np.sort(rng.choice(100_000, 40, replace=False)) for _ in range(16)]
        elif kind == 3:                                  # similar rows over a span too wide for the classifier
            base = np.sort(rng.choice(N, 150, replace=False))
            grp = [base[rng.random(150) > 0.1] for _ in range(16)]
        else:                                            # similar rows, one of them not sorted
            base = np.sort(rng.choice(3_000, 100, replace=False))
            grp = [base[rng.random(100) > 0.1] for _ in range(16)]
            grp[3] = np.concatenate([grp[3][:2][::-1], grp[3][2:]])
        rows += grp
    rows = rows[:M]
    lens = np.array([len(x) for x in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    if dtype == "bf16":
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        A, B, ops, dt = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K), (Ab, Bb), capi.BF16
    else:
        ops, dt = (A, B), capi.F32
    fill = 80 if K * (2 if dtype == "bf16" else 4) <= 128 else 56
    got, st = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert_parity(got, rowptr, col, val, A, B, what="union strips")
    want = _host_union_model(M, rowptr, col, fill)
    assert want[0] > 0 and st.panels == 0
    assert (st.mfma_tiles, st.nnz_mfma) == want
    assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == len(col)
    monkeypatch.setenv("SDDMM_UNION", "0")
    off, st0 = run_csr(engine_factory, rowptr, col, val, *ops, N, capi.AUTO, dt)
    assert st0.mfma_tiles == 0
    assert_parity(off, rowptr, col, val, A, B, what="union strips off")


@pytest.mark.parametrize("fill_limit", ["0", "100000"])
@pytest.mark.parametrize("K,dtype", [(32, capi.F32), (64, capi.F32), (128, capi.BF16), (256, capi.F32), (512, capi.BF16)])
def test_tile_windows_and_tile_walk_agree_with_the_oracle(engine_factory, monkeypatch, fill_limit, K, dtype):
    """The tile kernels take four consecutive tiles of a strip either as one batch (the
    entries of a row inside the window read and written as runs; SDDMM_WINDOW_FILL above
    the fill of the tiles) or tile by tile (below it).  Both on strips whose rows hold
    0, 1, 2, 3, 4, 5 and many entries per window, on a strip count that is not a multiple
    of anything, with the last window of a strip shorter than four tiles."""
    monkeypatch.setenv("SDDMM_WINDOW_FILL", fill_limit)
    rng = np.random.default_rng(4100 + K)
    M, N = 16 * 9 + 3, 16 * 41 + 7
    dense = np.zeros((M, N), bool)
    for s in range(M // 16 + 1):
        r0 = 16 * s
        tiles = np.sort(rng.choice(N // 16, int(rng.integers(1, 15)), replace=False))
        for tj in tiles:
            blk = rng.random((16, 16)) < rng.choice([0.08, 0.3, 0.9, 1.0])
            dense[r0:r0 + 16, 16 * tj:16 * tj + 16][: M - r0] |= blk[: M - r0]
        # rows of the strip with very few entries, and empty ones
        for rr, keep in ((1, 1), (2, 2), (3, 3), (5, 4), (6, 5), (7, 0)):
            if r0 + rr < M:
                c = np.nonzero(dense[r0 + rr])[0]
                dense[r0 + rr] = False
                dense[r0 + rr, c[:keep]] = True
    r, c = np.nonzero(dense)
    v = rng.uniform(-1, 1, len(r)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    if dtype == capi.BF16:
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        A, B = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K)
    else:
        Ab, Bb = A, B
    got, st = run_csr(engine_factory, rowptr, col, val, Ab, Bb, N, capi.MFMA_TILE, dtype)
    assert st.nnz_mfma == len(col) and st.mfma_tiles > 0
    assert_parity(got, rowptr, col, val, A, B, what="tiles K=%d limit %s" % (K, fill_limit))


@pytest.mark.parametrize("fill_limit", ["0", "100000"])
@pytest.mark.parametrize("name,K", [("dense_tiles", 128), ("dense_tiles", 512), ("mixed_density", 64)])
def test_windows_taken_block_by_block_over_strips_and_columns(engine_factory, monkeypatch, name, K, fill_limit):
    """The plan may hand the windows to the launch in an order of its own (blocks of strips x tile
    columns, one per XCD, for operands that exceed an L2).  Forced here on small inputs, for the
    batch and the tile-by-tile form of the windows, with and without row kernels in the same
    launch: every entry is still computed exactly once."""
    monkeypatch.setenv("SDDMM_WINDOW_ORDER", "1")
    monkeypatch.setenv("SDDMM_WINDOW_FILL", fill_limit)
    w = W.make(name, "small", K=K)
    bf16 = w.dtype == "bf16"
    e = engine_factory()
    if bf16:
        e.set_dense(w.A_bits, w.B_bits, capi.BF16)
    else:
        e.set_dense(w.A, w.B)
    for strategy in (capi.AUTO, capi.MFMA_TILE):
        e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)      # clears P
        e.plan(strategy)
        e.run()
        st = e.stats()
        assert st.mfma_tiles > 0
        assert_parity(e.values(), w.rowptr, w.col, w.sval, w.A, w.B, what="%s K=%d ordered windows" % (name, K))
        assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == w.nnz
    e.close()
