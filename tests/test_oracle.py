"""Pins the CPU oracle (oracle/sddmm_oracle.c) -- no GPU involved.

Sources of truth, in order: the closed forms of the reference's own test cases
(tests/matrix_test.cc:124-182 sddmm_coo1..4, :354-425 + :460-477 dispatcher
vectors, benchmark/dataset.hpp:183-204 DummyDataset), the reference's own headers
compiled in place (oracle/_ref, when built), and what the mathematics fixes
(all-ones S == GEMM, K=1 outer product, brute-force dense evaluation, linearity
in S, row independence).
"""
import numpy as np
import pytest

from oracle import oracle as O

f32 = np.float32


# ---- the reference's hand-checkable cases, expected values derived by hand ----
KATS = {
    # name: (A, B, triplets(row, col, val), M, N, expected P in sorted (row,col) order)
    "sddmm_coo1": ([[1, 2], [3, 4]], [[-1, 2], [-3, 4]],
                   [(0, 0, 1), (0, 1, 1), (1, 0, 1), (1, 1, 1)], 2, 2, [3, 5, 5, 7]),
    "sddmm_coo2": ([[1, 2, 3], [4, 5, 6]], [[-1, -3, 5], [2, 4, -6]],
                   [(0, 0, 1), (1, 0, 1), (1, 1, 1)], 2, 2, [8, 11, -8]),
    "sddmm_coo3": ([[1, 2, 3], [4, 5, 6]], [[-1, -3, 5]],
                   [(0, 0, 1), (1, 0, -1)], 2, 2, [8, -11]),
    "sddmm_coo4": ([[1, 2], [3, 4], [5, 6]], [[-1, -3], [2, 2], [3, 1]],
                   [(0, 0, 1), (1, 0, -1), (2, 0, 1), (2, 2, 1)], 3, 3, [-7, 15, -23, 21]),
    "dummy": ([[1, 1], [1, 1]], [[1, 1], [1, 1]],
              [(0, 0, 1), (0, 1, 1), (1, 0, 1), (1, 1, 1)], 2, 2, [2, 2, 2, 2]),
}


def _kat_arrays(name):
    A, B, trip, M, N, exp = KATS[name]
    r = np.array([t[0] for t in trip], np.int32)
    c = np.array([t[1] for t in trip], np.int32)
    v = np.array([t[2] for t in trip], f32)
    return np.array(A, f32), np.array(B, f32), r, c, v, M, N, np.array(exp, f32)


@pytest.mark.parametrize("name", list(KATS))
def test_kat_closed_forms(name):
    A, B, r, c, v, M, N, exp = _kat_arrays(name)
    # hand values double-checked by exact integer arithmetic
    dense = (np.array(A, np.int64) @ np.array(B, np.int64).T)
    assert [int(dense[i, j] * int(s)) for i, j, s in zip(r, c, v)] == [int(x) for x in exp]
    row, col, val = O.coo_from_triplets(r, c, v)
    np.testing.assert_array_equal(O.sddmm_coo(row, col, val, A, B), exp)
    rowptr, col2, val2 = O.csr_from_triplets(M, r, c, v)
    np.testing.assert_array_equal(O.sddmm_csr(rowptr, col2, val2, A, B), exp)
    np.testing.assert_array_equal(O.sddmm_csr(rowptr, col2, val2, A, B, threads=2), exp)
    np.testing.assert_array_equal(O.sddmm_csr_numpy(rowptr, col2, val2, A, B), exp)


def _random_case(rng, M, N, K, density, lo=-1.0, hi=1.0):
    mask = rng.random((M, N)) < density
    r, c = np.nonzero(mask)
    v = rng.uniform(lo, hi, len(r)).astype(f32)
    A = rng.uniform(lo, hi, (M, K)).astype(f32)
    B = rng.uniform(lo, hi, (N, K)).astype(f32)
    return r.astype(np.int32), c.astype(np.int32), v, A, B


def test_all_ones_sampling_equals_gemm():
    rng = np.random.default_rng(1)
    M, N, K = 37, 53, 19
    A = rng.integers(-4, 5, (M, K)).astype(f32)      # small integers: fp32 arithmetic is exact
    B = rng.integers(-4, 5, (N, K)).astype(f32)
    r, c = np.divmod(np.arange(M * N), N)
    rowptr, col, val = O.csr_from_triplets(M, r, c, np.ones(M * N, f32))
    P = O.sddmm_csr(rowptr, col, val, A, B)
    np.testing.assert_array_equal(P.reshape(M, N), A @ B.T)


def test_k1_is_outer_product_and_identity_b_gathers_a():
    rng = np.random.default_rng(2)
    M, N = 23, 31
    r, c, v, A, B = _random_case(rng, M, N, 1, 0.4)
    rowptr, col, val = O.csr_from_triplets(M, r, c, v)
    rows = O.coo_rows_from_csr(rowptr)
    np.testing.assert_array_equal(O.sddmm_csr(rowptr, col, val, A, B), (A[rows, 0] * B[col, 0]) * val)
    # B = identity (N x K with K = N): dot(A_i, e_j) = A[i, j]
    K = N
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    P = O.sddmm_csr(rowptr, col, np.ones_like(val), A, np.eye(N, dtype=f32))
    np.testing.assert_array_equal(P, A[rows, col])


def test_brute_force_dense_and_fp64():
    rng = np.random.default_rng(3)
    M, N, K = 41, 29, 32
    r, c, v, A, B = _random_case(rng, M, N, K, 0.3)
    rowptr, col, val = O.csr_from_triplets(M, r, c, v)
    P = O.sddmm_csr(rowptr, col, val, A, B)
    rows = O.coo_rows_from_csr(rowptr)
    dense64 = A.astype(np.float64) @ B.astype(np.float64).T
    ref64 = dense64[rows, col] * val.astype(np.float64)
    d64, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    np.testing.assert_allclose(d64, ref64, rtol=1e-13, atol=0)
    assert np.all(mag >= np.abs(d64) * (1 - 1e-12))
    # fp32 sequential result is within K ulps of the cancellation-free magnitude
    assert np.all(np.abs(P - ref64) <= K * 2.0 ** -24 * mag + 1e-30)
    # exact emulation of the k-ascending fp32 loop, one entry at a time
    for e in rng.choice(len(col), 50, replace=False):
        acc = f32(0)
        for k in range(K):
            acc = f32(acc + f32(A[rows[e], k] * B[col[e], k]))
        assert P[e] == f32(acc * val[e])


def test_order_of_operations_is_mul_then_add_then_scale():
    # values chosen so that an FMA, a pairwise sum or scaling before summing would differ
    A = np.array([[1 + 2 ** -12, 1.0, 3.0]], f32)
    B = np.array([[1 + 2 ** -12, -1.0, 2 ** -24]], f32)
    rowptr, col, val = np.array([0, 1], np.int32), np.array([0], np.int32), np.array([3.0], f32)
    p0 = f32(A[0, 0] * B[0, 0])                      # rounded product (drops 2^-24)
    acc = f32(f32(p0 + f32(A[0, 1] * B[0, 1])) + f32(A[0, 2] * B[0, 2]))
    exp = f32(acc * val[0])
    assert O.sddmm_csr(rowptr, col, val, A, B)[0] == exp
    fma_like = np.float64(A[0, 0]) * np.float64(B[0, 0]) - 1.0
    assert f32(fma_like) != f32(p0 - 1.0)            # the case really separates FMA from mul+add


def test_linearity_in_s_and_row_independence():
    rng = np.random.default_rng(4)
    M, N, K = 64, 64, 8
    r, c, v, A, B = _random_case(rng, M, N, K, 0.2)
    rowptr, col, val = O.csr_from_triplets(M, r, c, v)
    P1 = O.sddmm_csr(rowptr, col, val, A, B)
    P2 = O.sddmm_csr(rowptr, col, (val * f32(2)).astype(f32), A, B)
    np.testing.assert_array_equal(P2, P1 * f32(2))   # scaling by 2 is exact
    A2 = A.copy()
    A2[10] = 0
    P3 = O.sddmm_csr(rowptr, col, val, A2, B)
    s, e = rowptr[10], rowptr[11]
    assert np.all(P3[s:e] == 0)
    np.testing.assert_array_equal(np.delete(P3, np.s_[s:e]), np.delete(P1, np.s_[s:e]))


def test_csr_coo_agree_and_numpy_restatement_bit_exact():
    rng = np.random.default_rng(5)
    for (M, N, K, d) in [(500, 500, 32, 0.3), (250, 250, 32, 0.7), (2000, 2000, 32, 0.001), (50, 70, 3, 0.5)]:
        r, c, v, A, B = _random_case(rng, M, N, K, d)
        rowptr, col, val = O.csr_from_triplets(M, r, c, v)
        row2, col2, val2 = O.coo_from_triplets(r, c, v)
        np.testing.assert_array_equal(col, col2)
        np.testing.assert_array_equal(O.coo_rows_from_csr(rowptr), row2)
        Pc = O.sddmm_csr(rowptr, col, val, A, B)
        np.testing.assert_array_equal(Pc, O.sddmm_coo(row2, col2, val2, A, B))
        np.testing.assert_array_equal(Pc, O.sddmm_csr_numpy(rowptr, col, val, A, B))
        np.testing.assert_array_equal(Pc, O.sddmm_csr(rowptr, col, val, A, B, threads=4))


# ---- containers ----------------------------------------------------------------
def test_triplet_sort_dedup_rules():
    # unsorted input, a duplicate with non-zero values (merged, first kept) and a
    # duplicate where one value is zero (both kept): triplet.h:12-14
    r = np.array([1, 0, 1, 0, 1, 0], np.int32)
    c = np.array([0, 1, 0, 0, 1, 1], np.int32)
    v = np.array([5, 2, 6, 1, 0, 3], f32)
    row, col, val = O.coo_from_triplets(r, c, v)
    assert row.tolist() == [0, 0, 1, 1]
    assert col.tolist() == [0, 1, 0, 1]
    assert val.tolist() == [1, 2, 5, 0]
    r = np.array([0, 0], np.int32); c = np.array([3, 3], np.int32); v = np.array([0, 7], f32)
    row, col, val = O.coo_from_triplets(r, c, v)
    assert len(row) == 2                              # an explicit zero never merges
    rowptr, col, val = O.csr_from_triplets(4, np.array([1], np.int32), np.array([0], np.int32), np.array([1], f32))
    assert rowptr.tolist() == [0, 0, 1, 1, 1]        # empty rows keep their slots


def test_representation_conversion_round_trip():
    # tests/matrix_test.cc:93-122: CSR(COO(x)) == CSR(x), random 2i x i with i samples
    rng = np.random.default_rng(6)
    for i in range(100, 1501, 175):
        rows, cols = 2 * i, i
        r = rng.integers(0, rows, i).astype(np.int32)
        c = rng.integers(0, cols, i).astype(np.int32)
        v = rng.random(i).astype(f32) + f32(0.5)
        rowptr, col, val = O.csr_from_triplets(rows, r, c, v)
        row2, col2, val2 = O.coo_from_triplets(r, c, v)
        rowptr3, col3, val3 = O.csr_from_triplets(rows, row2, col2, val2)   # CSR(COO)
        np.testing.assert_array_equal(rowptr, rowptr3)
        np.testing.assert_array_equal(col, col3)
        np.testing.assert_array_equal(val, val3)
        np.testing.assert_array_equal(O.coo_rows_from_csr(rowptr), row2)     # COO(CSR)
        assert np.all(np.diff(rowptr) >= 0) and rowptr[-1] == len(col)


# ---- nnz-balanced partition: exact vectors of tests/matrix_test.cc:354-425,460-477 ----
def _diag_rowptr(n):
    return np.arange(n + 1, dtype=np.int32)


DISPATCH_KATS = [
    # (rowptr, parts, stride, expected)
    (np.array([0, 2, 4], np.int32), 4, 1, [0, 1, 2, 2, 2]),
    (np.array([0, 2, 4], np.int32), 2, 1, [0, 1, 2]),
    (np.array([0, 1, 2, 3, 4], np.int32), 2, 1, [0, 2, 4]),
    (np.array([0, 0, 1, 1, 1], np.int32), 2, 1, [0, 4, 4]),
    (_diag_rowptr(64), 4, 16, [0, 16, 32, 48, 64]),
]


@pytest.mark.parametrize("case", range(len(DISPATCH_KATS)))
def test_dispatch_kats(case):
    rowptr, parts, stride, exp = DISPATCH_KATS[case]
    assert O.dispatch(rowptr, parts, stride).tolist() == exp


def test_dispatch_large_regular():
    n = 150000
    got = O.dispatch(_diag_rowptr(n), n // 2)
    np.testing.assert_array_equal(got, 2 * np.arange(n // 2 + 1))


def test_density_is_64bit():
    assert O.density(2_600_000, 2_600_000, 36_000_000) == pytest.approx(36e6 / 2.6e6 ** 2)


# ---- against the reference's own headers compiled in place ----------------------
needs_ref = pytest.mark.skipif(not O.Ref.available(), reason="oracle/_ref not built (reference tree absent)")


@needs_ref
def test_against_reference_cpu_basic():
    ref = O.Ref()
    rng = np.random.default_rng(7)
    for (M, N, K, d, lo) in [(500, 500, 32, 0.3, -1.0), (250, 250, 32, 0.7, 0.0), (300, 200, 3, 0.2, -1.0),
                             (120, 90, 128, 0.5, -1.0), (64, 64, 1, 0.5, -1.0)]:
        r, c, v, A, B = _random_case(rng, M, N, K, d, lo=lo, hi=100.0 if lo == 0.0 else 1.0)
        p = rng.permutation(len(r))                   # the constructors must sort
        rp_ref, col_ref, P_ref = ref.cpu_basic_csr(M, N, r[p], c[p], v[p], A, B)
        rowptr, col, val = O.csr_from_triplets(M, r[p], c[p], v[p])
        np.testing.assert_array_equal(rowptr, rp_ref)
        np.testing.assert_array_equal(col, col_ref)
        np.testing.assert_array_equal(O.sddmm_csr(rowptr, col, val, A, B), P_ref)   # bit-exact
        row_ref, col_ref2, val_ref, Pcoo_ref = ref.cpu_basic_coo(M, N, r[p], c[p], v[p], A, B)
        row2, col2, val2 = O.coo_from_triplets(r[p], c[p], v[p])
        np.testing.assert_array_equal(row2, row_ref)
        np.testing.assert_array_equal(col2, col_ref2)
        np.testing.assert_array_equal(val2, val_ref)
        np.testing.assert_array_equal(O.sddmm_coo(row2, col2, val2, A, B), Pcoo_ref)


@needs_ref
def test_kats_against_reference():
    ref = O.Ref()
    for name in KATS:
        A, B, r, c, v, M, N, exp = _kat_arrays(name)
        _, _, _, P = ref.cpu_basic_coo(M, N, r, c, v, A, B)
        np.testing.assert_array_equal(P, exp)


@needs_ref
def test_dispatch_against_reference():
    ref = O.Ref()
    rng = np.random.default_rng(8)
    for trial in range(12):
        M = int(rng.integers(16, 400)) // 16 * 16 + 16
        N = int(rng.integers(4, 200))
        n = int(rng.integers(1, 4000))
        r = rng.integers(0, M, n).astype(np.int32)
        if trial % 3 == 0:
            r = (r // 7 * 7).astype(np.int32)        # clustered rows, many empty
        c = rng.integers(0, N, n).astype(np.int32)
        v = np.ones(n, f32)
        rowptr, _, _ = O.csr_from_triplets(M, r, c, v)
        for parts, stride in [(1, 1), (3, 1), (7, 1), (64, 1), (M, 1), (2 * M, 1), (4, 16)]:
            np.testing.assert_array_equal(O.dispatch(rowptr, parts, stride),
                                          ref.dispatch(M, N, r, c, v, parts, stride),
                                          err_msg="M=%d parts=%d stride=%d" % (M, parts, stride))


@needs_ref
def test_container_round_trip_against_reference():
    ref = O.Ref()
    rng = np.random.default_rng(9)
    for i in (100, 525, 1500):
        rows, cols = 2 * i, i
        r = rng.integers(0, rows, i).astype(np.int32)
        c = rng.integers(0, cols, i).astype(np.int32)
        v = (rng.random(i) + 0.5).astype(f32)
        a = ref.csr_build(rows, cols, r, c, v, via_coo=False)
        b = ref.csr_build(rows, cols, r, c, v, via_coo=True)
        mine = O.csr_from_triplets(rows, r, c, v)
        for x, y, z in zip(a, b, mine):
            np.testing.assert_array_equal(x, y)
            np.testing.assert_array_equal(x, z)


def test_comparator():
    ref = np.array([1.0, -2.0, 0.0, 1e-3], f32)
    ok, worst, _ = O.check_values(ref, ref)
    assert ok and worst == 0
    ok, _, i = O.check_values(ref * f32(1 + 3e-5), ref)
    assert not ok
    ok, _, _ = O.check_values(np.array([1.0, -2.0, 1e-7, 1e-3], f32), ref)
    assert not ok                                     # zero reference, no floor: any error fails
    mag = np.array([1.0, 2.0, 1.0, 1.0])
    ok, _, _ = O.check_values(np.array([1.0, -2.0, 1e-7, 1e-3], f32), ref, mag=mag)
    assert ok                                         # 1e-7 <= 1e-5 * 0.25 * 1.0
    ok, _, _ = O.check_values(np.array([1.0, 2.0, 0.0, 1e-3], f32), ref, mag=mag)
    assert not ok                                     # sign error is caught (the reference's == would pass it)


def test_fast_comparator_gives_the_answers_of_the_numpy_one():
    """oracle_compare (C, all cores; what bench.py uses on tens of millions of entries)
    against check_values on exact matches, small and large errors, zero references with
    and without a magnitude floor, NaN and infinities on either side."""
    rng = np.random.default_rng(5)
    n = 200_003
    ref = rng.uniform(-1, 1, n).astype(f32)
    ref[::97] = 0
    mag = np.abs(ref).astype(np.float64) + rng.random(n)
    cases = []
    cases.append(ref.copy())
    g = ref.copy(); g[1234] *= f32(1 + 2e-5); cases.append(g)
    g = ref.copy(); g[97 * 5] = f32(1e-7); cases.append(g)
    g = (ref * (1 + rng.uniform(-4e-6, 4e-6, n))).astype(f32); cases.append(g)
    g = ref.copy(); g[77] = np.nan; cases.append(g)
    g = ref.copy(); g[n - 1] = np.inf; g[5] = -np.inf; cases.append(g)
    for i, got in enumerate(cases):
        for m in (None, mag):
            for rtol in (1e-5, 1e-2):
                a = O.check_values(got, ref, mag=m, rtol=rtol)
                b = O.check_values_fast(got, ref, mag=m, rtol=rtol)
                assert a[0] == b[0] and a[2] == b[2], (i, m is None, rtol, a, b)
                assert a[1] == b[1] or abs(a[1] - b[1]) <= 1e-12 * abs(a[1]), (i, a, b)
    bad_ref = ref.copy(); bad_ref[10] = np.inf
    got = bad_ref.copy()
    a, b = O.check_values(got, bad_ref, mag=mag), O.check_values_fast(got, bad_ref, mag=mag)
    assert a[0] == b[0] and a[2] == b[2] and not a[0]          # inf - inf is NaN: never passes
    assert O.check_values_fast(np.zeros(0, f32), np.zeros(0, f32)) == (True, 0.0, -1)
    assert O.check_values_fast(np.zeros(3, f32), np.zeros(4, f32))[0] is False


# ---- SDDMM followed by SpMM (no counterpart in the reference: pinned by identities) ----
def test_fusedmm_oracle_against_dense_algebra():
    """O = (S o (A B^T)) B.  Brute force in float64 on small inputs, the all-ones S
    special case (O = A B^T B), a diagonal S (each output row is a multiple of one B
    row), linearity in S, and the P half against the SDDMM oracle bit for bit."""
    rng = np.random.default_rng(77)
    M, N, K = 23, 17, 12
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (N, K)).astype(np.float32)
    dense = rng.random((M, N)) < 0.4
    dense[5, :] = False                                        # an empty row gives a zero output row
    r, c = np.nonzero(dense)
    v = rng.uniform(-1, 1, len(r)).astype(np.float32)
    rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
    P, Out = O.fusedmm_csr(rowptr, col, val, A, B)
    np.testing.assert_array_equal(P.view(np.uint32), O.sddmm_csr(rowptr, col, val, A, B).view(np.uint32))
    S = np.zeros((M, N)); S[r, c] = v
    want = (S * (A.astype(np.float64) @ B.astype(np.float64).T)) @ B.astype(np.float64)
    np.testing.assert_allclose(Out, want, rtol=0, atol=2e-5)
    assert not Out[5].any()
    o64, mag = O.fusedmm_csr_f64(rowptr, col, val, A, B)
    np.testing.assert_allclose(o64, want, rtol=1e-12, atol=1e-12)
    assert (mag >= np.abs(o64) - 1e-12).all()
    # all-ones S: plain matrix products
    rr, cc = np.nonzero(np.ones((M, N), bool))
    rp1, c1, v1 = O.csr_from_triplets(M, rr.astype(np.int32), cc.astype(np.int32), np.ones(len(rr), np.float32))
    _, O1 = O.fusedmm_csr(rp1, c1, v1, A, B)
    np.testing.assert_allclose(O1, A.astype(np.float64) @ B.astype(np.float64).T @ B.astype(np.float64), rtol=0, atol=5e-5)
    # diagonal S: O[i] = s_i <a_i, b_i> b_i, three roundings
    n = min(M, N)
    d = np.arange(n, dtype=np.int32)
    sv = rng.uniform(0.5, 2, n).astype(np.float32)
    rpd, cd, vd = O.csr_from_triplets(M, d, d, sv)
    Pd, Od = O.fusedmm_csr(rpd, cd, vd, A, B)
    for i in range(n):
        np.testing.assert_array_equal(Od[i], (Pd[i] * B[i]).astype(np.float32))
    assert not Od[n:].any()
    # linear in S, exactly for a factor 2
    _, O2 = O.fusedmm_csr(rowptr, col, (val * np.float32(2)).astype(np.float32), A, B)
    np.testing.assert_array_equal(O2, Out * np.float32(2))
