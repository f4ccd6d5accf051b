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
    # a fixed strategy on the same context
    e.plan(other)
    e.run()
    fixed = e.values()
    assert O.check_values(fixed, ref, mag=mag)[0]
    if st.mfma_tiles == 0 and st.panels == 0:        # only gather kernels: same per-entry arithmetic
        np.testing.assert_array_equal(fixed.view(np.uint32), auto.view(np.uint32))
    # the exact-order kernel is the CPU loop bit for bit, also at this size
    e.plan(capi.EXACT)
    e.run()
    np.testing.assert_array_equal(e.values().view(np.uint32), ref.view(np.uint32))
    e.close()
