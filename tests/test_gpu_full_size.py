"""Parity at the benchmark's full sizes.  Besides the comparison with the
(OpenMP) oracle these use properties that do not depend on the size: the result is
linear in S (a factor 2 is exact in fp32), strategies built from the same per-entry
arithmetic agree bitwise, empty rows stay empty, and a sum over all entries matches
the float64 reference within the accumulated tolerance."""
import sys

import numpy as np
import pytest

from dphpc_amd import capi, workloads as W
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32

CASES = [("fem_banded", 32, capi.ROW_WAVE), ("fem_banded", 128, capi.ROW_WAVE), ("mixed_density", 32, capi.FLAT),
         ("mixed_density", 256, capi.FLAT), ("power_law", 32, capi.FLAT), ("dense_tiles", 128, capi.ROW_WAVE),
         ("dense_tiles", 512, capi.FLAT)]


@pytest.mark.parametrize("name,K,other", CASES)
def test_full_size(engine_factory, name, K, other):
    w = W.make(name, "full", K=K)
    print("full size", name, K, "nnz", w.nnz, flush=True)
    sys.stdout.flush()
    bf16 = w.dtype == "bf16"
    e = engine_factory()
    if bf16:
        e.set_dense(w.A_bits, w.B_bits, capi.BF16)
    else:
        e.set_dense(w.A, w.B)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    e.plan(capi.AUTO)
    e.run()
    auto = e.values()
    st = e.stats()
    ref = O.sddmm_csr(w.rowptr, w.col, w.sval, w.A, w.B, threads=0)
    d64, mag = O.sddmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
    ok, worst, i = O.check_values(auto, ref, mag=mag)
    assert ok, (name, K, i, auto[i], ref[i], worst)
    assert abs(auto.astype(np.float64).sum() - d64.sum()) <= 1e-5 * mag.sum()
    assert st.nnz == w.nnz and st.bytes_gathered == w.bytes_gathered()
    # linear in S: doubling S doubles P exactly
    e.update_values((w.sval * f32(2)).astype(f32))
    e.run()
    np.testing.assert_array_equal(e.values(), auto * f32(2))
    e.update_values(w.sval)
    # a fixed strategy on the same context (the pattern is set again: that clears P, so a
    # kernel that wrote nothing could not pass on the previous strategy's values)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    e.plan(other)
    e.run()
    fixed = e.values()
    assert O.check_values(fixed, ref, mag=mag)[0]
    if st.mfma_tiles == 0 and st.panels == 0:        # only gather kernels: same per-entry arithmetic
        np.testing.assert_array_equal(fixed.view(np.uint32), auto.view(np.uint32))
    # the exact-order kernel is the CPU loop bit for bit, also at this size
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    e.plan(capi.EXACT)
    e.run()
    np.testing.assert_array_equal(e.values().view(np.uint32), ref.view(np.uint32))
    e.close()


@pytest.mark.parametrize("name,K,dtype", [("fem_banded", 32, capi.F32), ("fem_banded", 128, capi.F32),
                                          ("mixed_density", 64, capi.F32), ("fem_banded", 64, capi.BF16),
                                          ("power_law", 32, capi.F32)])
def test_fused_full_size(engine_factory, name, K, dtype):
    """SDDMM followed by SpMM at the benchmark's sizes: the panel kernel (fem_banded, fp32 and bf16
    operands) and the gather kernels (mixed_density, power_law) against the oracle on the operands as
    stored, and the row sums of O against float64."""
    w = W.make(name, "full", K=K)
    print("fused full size", name, K, "nnz", w.nnz, flush=True)
    e = engine_factory()
    if dtype == capi.BF16:
        Ab, Bb = capi.to_bf16(w.A).reshape(w.A.shape), capi.to_bf16(w.B).reshape(w.B.shape)
        w.A, w.B = capi.from_bf16(Ab).reshape(w.A.shape), capi.from_bf16(Bb).reshape(w.B.shape)
        e.set_dense(Ab, Bb, capi.BF16)
    else:
        e.set_dense(w.A, w.B)
    e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
    e.plan(capi.AUTO)
    got_o = e.run_fused()
    got_p = e.values()
    ref_p, ref_o = O.fusedmm_csr(w.rowptr, w.col, w.sval, w.A, w.B)
    _, mag_p = O.sddmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
    o64, mag_o = O.fusedmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
    ok, worst, i = O.check_values(got_p, ref_p, mag=mag_p)
    assert ok, (name, K, "P", i, worst)
    ok, worst, i = O.check_values(got_o[:w.M].ravel(), ref_o.ravel(), mag=mag_o.ravel())
    assert ok, (name, K, "O", i, worst)
    assert abs(got_o[:w.M].astype(np.float64).sum() - o64.sum()) <= 1e-5 * mag_o.sum()
    if name == "fem_banded":
        assert e.stats().kernels_launched == 1        # every row belongs to a panel
    e.close()


def test_positions_beyond_2_to_the_30(engine_factory):
    """1.2e9 stored entries: positions above 2^30, byte offsets above 4 GiB in the entry
    arrays.  Groups of 8 identical rows, so AUTO takes the panel kernel; the exact kernel
    must match the oracle bit for bit, the others to the usual tolerance (all values are
    of order one here, checked in slices to keep host memory flat)."""
    M, L, N, K = 300000, 4000, 50000, 32
    rng = np.random.default_rng(7)
    starts = np.repeat(rng.integers(0, 2000, M // 8), 8).astype(np.int32)
    col = (starts[:, None] + (12 * np.arange(L, dtype=np.int32))[None, :]).reshape(-1)
    rowptr = (np.arange(M + 1, dtype=np.int64) * L).astype(np.int32)
    nnz = len(col)
    assert nnz > 2 ** 30
    val = rng.random(nnz, dtype=f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    print("entries", nnz, flush=True)
    ref = O.sddmm_csr(rowptr, col, val, A, B, threads=0)
    sample = np.unique(np.concatenate([rng.integers(0, nnz, 2_000_000), np.arange(1000), np.arange(nnz - 1000, nnz)]))
    mag_sample = np.abs(val[sample].astype(np.float64)) * np.abs(
        A[sample // L].astype(np.float64) * B[col[sample]].astype(np.float64)).sum(axis=1)
    e = engine_factory()
    e.set_dense(A, B)
    step = 1 << 26
    for strategy in (capi.EXACT, capi.AUTO, capi.FLAT):
        print("strategy", capi.STRATEGY_NAMES[strategy], flush=True)
        e.set_csr(M, N, rowptr, col, val)                  # clears P
        e.plan(strategy)
        e.run()
        got = e.values()
        st = e.stats()
        if strategy == capi.AUTO:
            assert st.panels == M // 8 and st.nnz_panel == nnz
        for i in range(0, nnz, step):
            g, r = got[i:i + step], ref[i:i + step]
            if strategy == capi.EXACT:
                assert np.array_equal(g.view(np.uint32), r.view(np.uint32)), i
            else:
                # a coarse net over every entry (values are of order one) ...
                assert float(np.abs(g - r).max()) <= 1.5e-5, (capi.STRATEGY_NAMES[strategy], i)
        # ... and the parity bar proper on a sample that includes the ends of the arrays
        ok, worst, j = O.check_values(got[sample], ref[sample], mag=mag_sample)
        assert ok, (capi.STRATEGY_NAMES[strategy], int(sample[j]), worst)
        del got
    e.close()


def test_a_grid_beyond_one_dispatch_is_refused_not_truncated(engine_factory):
    """2^26 + 1000 rows: one wavefront per row would be a launch of more than 2^32 threads,
    of which the hardware would run a part without any error.  The library must refuse that
    strategy and compute the same matrix with the strategies that fit."""
    M, N, K = (1 << 26) + 1000, 64, 4
    rng = np.random.default_rng(8)
    rowptr = np.arange(M + 1, dtype=np.int32)              # one entry per row
    col = rng.integers(0, N, M).astype(np.int32)
    val = rng.random(M, dtype=f32)
    A = rng.random((M, K), dtype=f32)
    B = rng.random((N, K), dtype=f32)
    ref = O.sddmm_csr(rowptr, col, val, A, B, threads=0)
    for strategy in (capi.ROW_WAVE, capi.AUTO, capi.FLAT, capi.EXACT):
        print("strategy", capi.STRATEGY_NAMES[strategy], flush=True)
        e = engine_factory()                               # a fresh context: P starts at zero
        e.set_dense(A, B)
        e.set_csr(M, N, rowptr, col, val)
        if strategy == capi.ROW_WAVE:
            e.plan(strategy)
            with pytest.raises(capi.SddmmError) as ei:
                e.run()
            assert ei.value.code == capi.ERR_UNSUPPORTED and "2^32" in str(ei.value)
        else:
            e.plan(strategy)
            e.run()
            got = e.values()
            if strategy == capi.EXACT:
                assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
            else:
                assert float(np.abs(got - ref).max()) <= 1e-5 * K      # |ref| < K
        e.close()
