"""SDDMM followed by SpMM over the same pattern (sddmm_run_fused) against the CPU
oracle: O within 1e-5 of the fp32 storage-order result with the cancellation-free
magnitude as floor, P to the bar of the SDDMM tests."""
import numpy as np
import pytest

from dphpc_amd import capi, workloads as W
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32


def _check(e, rowptr, col, val, A, B, what):
    got_o = e.run_fused()
    got_p = e.values()
    ref_p, ref_o = O.fusedmm_csr(rowptr, col, val, A, B)
    _, mag_p = O.sddmm_csr_f64(rowptr, col, val, A, B)
    ok, worst, i = O.check_values(got_p, ref_p, mag=mag_p)
    assert ok, "%s: P entry %d got %r ref %r (%.2f x tolerance)" % (what, i, got_p[i], ref_p[i], worst)
    _, mag_o = O.fusedmm_csr_f64(rowptr, col, val, A, B)
    M = len(rowptr) - 1
    ok, worst, i = O.check_values(got_o[:M].ravel(), ref_o.ravel(), mag=mag_o.ravel())
    assert ok, "%s: O element %d got %r ref %r (%.2f x tolerance)" % (what, i, got_o[:M].ravel()[i], ref_o.ravel()[i], worst)
    assert not got_o[M:].any()                       # rows of A beyond S's rows stay zero
    return got_o


@pytest.mark.parametrize("K", [4, 8, 32, 48, 100, 128, 256])
def test_fused_random(engine_factory, K):
    rng = np.random.default_rng(900 + K)
    M, N = 300, 260
    dense = rng.random((M, N)) < 0.08
    dense[17] = False
    dense[40, :] = rng.random(N) < 0.9               # a long row
    r, c = np.nonzero(dense)
    v = rng.uniform(-1, 1, len(r)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
    A = rng.uniform(-1, 1, (M + 3, K)).astype(f32)   # A may have more rows than S
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    out = _check(e, rowptr, col, val, A, B, "random K=%d" % K)
    assert not out[17].any()
    # repeatable, and the ordinary run still works on the same context
    np.testing.assert_array_equal(out, e.run_fused())
    e.plan(capi.AUTO); e.run()
    ok, worst, i = O.check_values(e.values(), O.sddmm_csr(rowptr, col, val, A, B), mag=O.sddmm_csr_f64(rowptr, col, val, A, B)[1])
    assert ok
    e.close()


def test_fused_rows_split_into_segments(engine_factory, monkeypatch):
    """Rows longer than a segment are accumulated by several wavefronts (atomic adds)."""
    monkeypatch.setenv("SDDMM_FUSED_SEG", "128")
    rng = np.random.default_rng(31)
    M, N, K = 40, 3000, 32
    rows = [np.sort(rng.choice(N, int(rng.choice([0, 5, 127, 128, 129, 700, 2500])), replace=False)) for _ in range(M)]
    lens = np.array([len(x) for x in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    _check(e, rowptr, col, val, A, B, "segments")
    e.close()


@pytest.mark.parametrize("name", ["fem_banded", "power_law", "mixed_density"])
def test_fused_benchmark_shapes_scaled_down(engine_factory, name):
    w = W.make(name, "small")
    e = engine_factory()
    e.set_dense(w.A, w.B)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    _check(e, w.rowptr, w.col, w.sval, w.A, w.B, name)
    # COO with sorted rows takes the same path
    e.set_coo(w.M, w.N, w.rows(), w.col, w.sval)
    _check(e, w.rowptr, w.col, w.sval, w.A, w.B, name + " coo")
    e.close()


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("K", [8, 32, 64, 136, 256])
def test_fused_16bit_operands(engine_factory, dtype, K):
    """bf16 / fp16 A and B (fp32 accumulation, fp32 P and O) against the fp32 oracle on the
    rounded inputs, short rows (one lane group per row) and rows split into segments."""
    rng = np.random.default_rng(1300 + K + dtype)
    M, N = 210, 3000
    lens = rng.choice([0, 1, 7, 30, 64, 65, 300, 2500], M)
    rows = [np.sort(rng.choice(N, int(n), replace=False)) for n in lens]
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    if dtype == capi.BF16:
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        Ar, Br = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K)
    else:
        Ab, Bb = capi.to_f16(A).reshape(M, K), capi.to_f16(B).reshape(N, K)
        Ar, Br = capi.from_f16(Ab).reshape(M, K), capi.from_f16(Bb).reshape(N, K)
    e = engine_factory()
    e.set_dense(Ab, Bb, dtype)
    e.set_csr(M, N, rowptr, col, val)
    _check(e, rowptr, col, val, Ar, Br, "16-bit K=%d dtype=%d" % (K, dtype))
    e.close()


def test_fused_unsupported_and_state(engine_factory):
    rng = np.random.default_rng(3)
    rowptr = np.array([0, 1, 2], np.int32); col = np.array([1, 0], np.int32); val = np.ones(2, f32)
    e = engine_factory()
    for K, dt in ((33, capi.F32), (260, capi.F32), (264, capi.BF16)):
        A = rng.uniform(-1, 1, (2, K)).astype(f32)
        if dt == capi.BF16:
            e.set_dense(capi.to_bf16(A).reshape(2, K), capi.to_bf16(A).reshape(2, K), dt)
        else:
            e.set_dense(A, A)
        e.set_csr(2, 2, rowptr, col, val)
        with pytest.raises(capi.SddmmError) as ei:
            e.run_fused()
        assert ei.value.code == capi.ERR_UNSUPPORTED
    A = rng.uniform(-1, 1, (2, 8)).astype(f32)
    e.set_dense(A, A)
    e.set_coo(2, 2, np.array([1, 0], np.int32), col, val)     # rows not sorted: no row pointer
    with pytest.raises(capi.SddmmError) as ei:
        e.run_fused()
    assert ei.value.code == capi.ERR_UNSUPPORTED
    e.set_csr(2, 2, rowptr, col, val)
    out = e.run_fused()
    want = np.stack([(A[0] @ A[1]) * A[1], (A[1] @ A[0]) * A[0]]).astype(f32)
    np.testing.assert_allclose(out, want, rtol=1e-6, atol=1e-6)
    e.close()


def test_fused_non_finite_rows_of_b_stay_in_their_own_entries(engine_factory):
    """Global entry 0 and the last entry of a long row point at B rows that hold an
    infinity and a NaN.  Steps past the end of a row work on clamped positions (entry 0
    for an empty row, the row's last entry otherwise): nothing of those B rows may reach
    the output row of another row, or turn into inf * 0 inside its own."""
    rng = np.random.default_rng(77)
    M, N, K = 70, 400, 32
    rows = [np.sort(rng.choice(N - 2, int(n), replace=False)) for n in rng.integers(1, 40, M)]
    rows[0] = np.array([N - 2])                              # entry 0 of the matrix -> B row N-2
    rows[5] = np.zeros(0, np.int64)                          # empty rows share wavefronts with the others
    rows[6] = np.zeros(0, np.int64)
    rows[9] = np.sort(np.concatenate([rng.choice(N - 2, 129, replace=False), [N - 1]]))   # long row ends in B row N-1
    lens = np.array([len(x) for x in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    B[N - 2, 3] = np.inf
    B[N - 1, 11] = np.nan
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    got_o = e.run_fused()
    got_p = e.values()
    with np.errstate(all="ignore"):
        ref_p, ref_o = O.fusedmm_csr(rowptr, col, val, A, B)
    rows_of = np.repeat(np.arange(M), lens)
    bad_entry = (col == N - 2) | (col == N - 1)
    assert np.array_equal(~np.isfinite(got_p), bad_entry)
    bad_row = np.zeros(M, bool)
    bad_row[rows_of[bad_entry]] = True
    assert np.array_equal(~np.isfinite(got_o).all(axis=1), bad_row), np.nonzero(~np.isfinite(got_o).all(axis=1))
    assert not got_o[5].any() and not got_o[6].any()
    clean = ~bad_row
    np.testing.assert_allclose(got_o[clean], ref_o[clean], rtol=1e-4, atol=1e-5)
    e.close()


def test_fused_output_rows_keep_nothing_of_an_earlier_call(engine_factory):
    """O is written, not cleared and added to, for the rows the short-row kernel owns: a second call on
    the same context with fewer rows in S, other rows long and other rows empty must not show anything
    of the first call's output, and the rows of A beyond S's rows come back as zeros."""
    rng = np.random.default_rng(611)
    MA, N, K = 96, 700, 32
    A = rng.uniform(-1, 1, (MA, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    e = engine_factory()
    e.set_dense(A, B)

    def pattern(M, lens):
        rows = [np.sort(rng.choice(N, int(n), replace=False)) for n in lens]
        rowptr = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int32)
        col = np.concatenate(rows).astype(np.int32) if rowptr[-1] else np.zeros(0, np.int32)
        return rowptr, col, rng.uniform(-1, 1, len(col)).astype(f32)

    lens1 = rng.choice([0, 3, 20, 64, 65, 300, 650], MA)
    rowptr, col, val = pattern(MA, lens1)
    e.set_csr(MA, N, rowptr, col, val)
    _check(e, rowptr, col, val, A, B, "first call")
    M2 = 60
    lens2 = np.where(lens1[:M2] > 64, 0, 500)             # long rows become empty, the others long
    lens2[::7] = 5
    rowptr, col, val = pattern(M2, lens2)
    e.set_csr(M2, N, rowptr, col, val)
    got = _check(e, rowptr, col, val, A[:M2], B, "second call, fewer rows")
    assert got.shape[0] == MA and not got[M2:].any()
    e.close()


@pytest.mark.parametrize("K", [8, 32, 64, 128])
@pytest.mark.parametrize("forced", [False, True])
def test_fused_rows_of_very_different_lengths(engine_factory, monkeypatch, K, forced):
    """A power-law-like pattern (most rows one to three entries, many empty, a few dozens, some beyond
    64): the short rows average 3.2 entries, fewer than half the 8 lanes of an entry at K >= 32, so the
    wavefronts deal whole rows out to their lane groups by entry count (forced: that kernel whatever K
    and on rows of 20 to 40 entries too).  A row count
    that is no multiple of 64, rows of A beyond S's rows, an infinity in a B row that one short row has."""
    if forced:
        monkeypatch.setenv("SDDMM_FUSED_BALANCED", "1")
    rng = np.random.default_rng(7300 + K + forced)
    M, MA, N = 64 * 37 + 29, 64 * 37 + 40, 5000
    lens = rng.choice([0, 0, 1, 1, 1, 1, 1, 1, 2, 2, 2, 3, 3, 20, 65, 200] if not forced else [0, 20, 25, 33, 40, 64, 65], M)
    lens[:64] = 0                                         # a wavefront without entries
    lens[64:128] = 1
    lens[200] = 64
    rows = [np.sort(rng.choice(N - 1, int(n), replace=False)) for n in lens]
    rows[130] = np.array([5, N - 1])
    lens[130] = 2
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (MA, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    e.plan(capi.AUTO)
    got = _check(e, rowptr, col, val, A[:M], B, "rows of very different lengths K=%d" % K)
    assert got.shape[0] == MA and not got[M:].any()
    B2 = B.copy()
    B2[N - 1, K // 2] = np.inf
    e.set_dense(A, B2)
    e.set_csr(M, N, rowptr, col, val)
    e.plan(capi.AUTO)
    got = e.run_fused()
    bad = ~np.isfinite(got).all(axis=1)
    assert bad[130] and bad.sum() == 1
    with np.errstate(all="ignore"):
        _, ref_o = O.fusedmm_csr(rowptr, col, val, A[:M], B2)
        _, mag_o = O.fusedmm_csr_f64(rowptr, col, val, A[:M], B2)
    keep = ~bad[:M]
    ok, worst, i = O.check_values(got[:M][keep].ravel(), ref_o[keep].ravel(), mag=mag_o[keep].ravel())
    assert ok, (K, forced, i, worst)
    e.close()


def _panel_pattern(rng, N, panel_lens, loose_lens):
    """8-row panels (one column list per panel) with loose rows in between, in groups of 8 so
    that the panels stay 8-aligned."""
    rows = []
    for i, n in enumerate(panel_lens):
        cols = np.sort(rng.choice(N, int(n), replace=False))
        rows += [cols] * 8
        if i < len(loose_lens):
            rows += [np.sort(rng.choice(N, int(m), replace=False)) for m in loose_lens[i]]
    lens = np.array([len(x) for x in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    return len(rows), rowptr, col


@pytest.mark.parametrize("K", [32, 64, 128])
@pytest.mark.parametrize("strategy", [capi.AUTO, capi.LDS_TILED])
def test_fused_row_panels_on_the_matrix_cores(engine_factory, monkeypatch, K, strategy):
    """fp32 rows of 128 / 256 / 512 bytes: the 8-row panels of the plan take the panel kernel (P and O
    from one pass over the gathered B rows), the other rows the gather kernels.  Panel lengths
    around the group sizes (16, 32, 64 columns) and items that cut a panel's list."""
    monkeypatch.setenv("SDDMM_PANEL_SEG", "128")
    rng = np.random.default_rng(4100 + K + strategy)
    N = 1500
    panel_lens = [4, 5, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 300, 700]
    loose = [[0, 3, 70, 1, 0, 200, 9, 64]] * 5 + [[12] * 8] * 3
    M, rowptr, col = _panel_pattern(rng, N, panel_lens, loose)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    e.plan(strategy)
    out = _check(e, rowptr, col, val, A, B, "panels K=%d strategy=%d" % (K, strategy))
    assert e.stats().kernels_launched == 3               # short rows, long rows, panels
    monkeypatch.setenv("SDDMM_FUSED_PANELS", "0")
    plain = _check(e, rowptr, col, val, A, B, "panels off")
    assert e.stats().kernels_launched == 2
    assert out.shape == plain.shape                      # (both were held to the oracle's bar above)
    monkeypatch.delenv("SDDMM_FUSED_PANELS")
    # the SDDMM alone still works on the same plan, and a new plan without panels drops them
    e.run()
    ok, _, _ = O.check_values(e.values(), O.sddmm_csr(rowptr, col, val, A, B), mag=O.sddmm_csr_f64(rowptr, col, val, A, B)[1])
    assert ok
    e.plan(capi.FLAT)
    _check(e, rowptr, col, val, A, B, "after a plan without panels")
    assert e.stats().kernels_launched == 2
    e.close()


def _rounded(A, dtype):
    """(stored 16-bit array, the fp32 values it holds)"""
    if dtype == capi.BF16:
        h = capi.to_bf16(A).reshape(A.shape)
        return h, capi.from_bf16(h).reshape(A.shape)
    h = capi.to_f16(A).reshape(A.shape)
    return h, capi.from_f16(h).reshape(A.shape)


@pytest.mark.parametrize("dtype", [capi.BF16, capi.F16])
@pytest.mark.parametrize("K", [32, 64, 128])
def test_fused_row_panels_of_16bit_operands(engine_factory, monkeypatch, K, dtype):
    """bf16 / fp16 rows of 64 / 128 / 256 bytes: the panels take the panel kernel here too (the B
    units widened to fp32 for the second product), against the fp32 oracle on the rounded operands.
    One panel's list ends on an infinite B row right after an item boundary."""
    monkeypatch.setenv("SDDMM_PANEL_SEG", "128")
    rng = np.random.default_rng(5200 + K + dtype)
    N = 1500
    panel_lens = [4, 5, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 300, 700]
    loose = [[0, 3, 70, 1, 0, 200, 9, 64]] * 5 + [[12] * 8] * 3
    M, rowptr, col = _panel_pattern(rng, N, panel_lens, loose)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    Ah, Ar = _rounded(rng.uniform(-1, 1, (M, K)).astype(f32), dtype)
    Bh, Br = _rounded(rng.uniform(-1, 1, (N, K)).astype(f32), dtype)
    e = engine_factory()
    e.set_dense(Ah, Bh, dtype)
    e.set_csr(M, N, rowptr, col, val)
    e.plan(capi.AUTO)
    _check(e, rowptr, col, val, Ar, Br, "16-bit panels K=%d dtype=%d" % (K, dtype))
    assert e.stats().kernels_launched == 3               # short rows, long rows, panels
    monkeypatch.setenv("SDDMM_FUSED_PANELS", "0")
    _check(e, rowptr, col, val, Ar, Br, "16-bit panels off")
    assert e.stats().kernels_launched == 2
    monkeypatch.delenv("SDDMM_FUSED_PANELS")
    # panels only, a list of 129 columns whose last B row holds an infinity: the other panels stay finite
    M2, rowptr2, col2 = _panel_pattern(rng, N - 1, [129, 40, 129], [])
    col2 = col2.copy()
    for r in range(8):
        col2[rowptr2[r] + 128] = N - 1
    val2 = rng.uniform(-1, 1, len(col2)).astype(f32)
    Br2 = Br.copy(); Br2[N - 1, K - 3] = np.inf
    Bh2, Br2 = _rounded(Br2, dtype)
    e.set_dense(Ah[:M2].copy(), Bh2, dtype)
    e.set_csr(M2, N, rowptr2, col2, val2)
    e.plan(capi.AUTO)
    got_o = e.run_fused()
    assert e.stats().kernels_launched == 1
    with np.errstate(all="ignore"):
        _, ref_o = O.fusedmm_csr(rowptr2, col2, val2, Ar[:M2], Br2)
    assert np.array_equal(np.isfinite(got_o[:M2]), np.isfinite(ref_o))
    assert np.isfinite(got_o[8:M2]).all() and not np.isfinite(got_o[:8]).all()
    np.testing.assert_allclose(got_o[8:M2], ref_o[8:], rtol=1e-4, atol=1e-5)
    e.close()


def test_fused_row_panels_keep_non_finite_b_rows_in_their_own_entries(engine_factory, monkeypatch):
    """A panel's list is cut into items of 128 columns and ends in the middle of a group of 16:
    the groups past an item's end load the B row of a clamped position, and the first column of
    the next item holds an infinity.  Neither may reach the output rows through 0 * inf."""
    monkeypatch.setenv("SDDMM_PANEL_SEG", "128")
    rng = np.random.default_rng(88)
    N, K = 900, 32
    M, rowptr, col = _panel_pattern(rng, N - 2, [150, 37, 200], [])
    rowptr = rowptr.copy(); col = col.copy()
    lens = np.diff(rowptr)
    # panel 1 (rows 8..15, 37 columns): its last column is B row N-1 (NaN); panel 2: column 128 of the list is B row N-2 (inf)
    for r in range(8, 16):
        col[rowptr[r] + 36] = N - 1
    for r in range(16, 24):
        seg = col[rowptr[r]:rowptr[r + 1]]
        seg[128:] = np.sort(np.concatenate([[N - 2], seg[129:]]))
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    B[N - 2, 5] = np.inf
    B[N - 1, 20] = np.nan
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    e.plan(capi.AUTO)
    got_o = e.run_fused()
    assert e.stats().kernels_launched == 1               # every row belongs to a panel
    got_p = e.values()
    with np.errstate(all="ignore"):
        ref_p, ref_o = O.fusedmm_csr(rowptr, col, val, A, B)
    bad_entry = (col == N - 2) | (col == N - 1)
    assert np.array_equal(~np.isfinite(got_p), bad_entry)
    bad_row = np.zeros(M, bool)
    bad_row[np.repeat(np.arange(M), lens)[bad_entry]] = True
    assert bad_row[8:24].all() and not bad_row[:8].any()
    assert np.array_equal(~np.isfinite(got_o).all(axis=1), bad_row)
    np.testing.assert_allclose(got_o[:8], ref_o[:8], rtol=1e-4, atol=1e-5)
    assert np.array_equal(np.isfinite(got_o), np.isfinite(ref_o))
    e.close()
