"""Golden vectors written by the reference's own CPUBasic (tests/golden/make_golden.py).

CPU part: the oracle reproduces them bit for bit.  GPU part: the EXACT strategy
reproduces them bit for bit, every other strategy within the fp32 bar."""
import os

import numpy as np
import pytest

from dphpc_amd import capi, workloads as W
from oracle import oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SAMPLED = [("fem_banded", 32), ("fem_banded", 128), ("power_law", 32), ("mixed_density", 32),
           ("mixed_density", 64), ("mixed_density", 256), ("dense_tiles", 128), ("dense_tiles", 512)]


def _full():
    g = np.load(os.path.join(GOLD, "small_uniform_K32.npz"))
    return {k: g[k] for k in g.files}


def _sampled(name, K):
    g = np.load(os.path.join(GOLD, "sampled_%s_K%d.npz" % (name, K)))
    w = W.make(name, "small", K=K)
    assert int(g["nnz"]) == w.nnz and int(g["col_sum"]) == int(w.col.astype(np.int64).sum()), \
        "the seeded workload no longer matches the fixture"
    return g, w


def test_oracle_reproduces_config1_golden():
    g = _full()
    w = W.make("small_uniform")
    for k in ("rowptr", "col", "sval", "A", "B"):
        np.testing.assert_array_equal(getattr(w, k), g[k])      # the generator is the one that made the fixture
    P = O.sddmm_csr(g["rowptr"], g["col"], g["sval"], g["A"], g["B"])
    np.testing.assert_array_equal(P.view(np.uint32), g["P"].view(np.uint32))
    np.testing.assert_array_equal(O.sddmm_coo(w.rows(), g["col"], g["sval"], g["A"], g["B"]).view(np.uint32),
                                  g["P"].view(np.uint32))


@pytest.mark.parametrize("name,K", SAMPLED)
def test_oracle_reproduces_sampled_golden(name, K):
    g, w = _sampled(name, K)
    P = O.sddmm_csr(w.rowptr, w.col, w.sval, w.A, w.B, threads=0)
    np.testing.assert_array_equal(P[g["pos"]].view(np.uint32), g["val"].view(np.uint32))
    assert P.astype(np.float64).sum() == float(g["total"])


@pytest.mark.gpu
def test_gpu_config1_against_golden(engine_factory):
    g = _full()
    _, mag = O.sddmm_csr_f64(g["rowptr"], g["col"], g["sval"], g["A"], g["B"])
    for strategy in (capi.EXACT, capi.AUTO, capi.FLAT, capi.ROW_WAVE, capi.SHORT_ROWS, capi.LDS_TILED, capi.MFMA_TILE):
        e = engine_factory()
        e.set_dense(g["A"], g["B"])
        e.set_csr(656, 656, g["rowptr"], g["col"], g["sval"])
        e.plan(strategy)
        e.run()
        got = e.values()
        e.close()
        if strategy == capi.EXACT:
            np.testing.assert_array_equal(got.view(np.uint32), g["P"].view(np.uint32))
        ok, worst, i = O.check_values(got, g["P"], mag=mag)
        assert ok, (capi.STRATEGY_NAMES[strategy], i, got[i], g["P"][i], worst)


@pytest.mark.gpu
@pytest.mark.parametrize("name,K", SAMPLED)
def test_gpu_sampled_golden(engine_factory, name, K):
    g, w = _sampled(name, K)
    _, mag = O.sddmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
    bf16 = w.dtype == "bf16"
    for strategy in (capi.EXACT, capi.AUTO):
        e = engine_factory()
        if bf16:
            e.set_dense(w.A_bits, w.B_bits, capi.BF16)
        else:
            e.set_dense(w.A, w.B)
        e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
        e.plan(strategy)
        e.run()
        got = e.values()
        e.close()
        if strategy == capi.EXACT:
            np.testing.assert_array_equal(got[g["pos"]].view(np.uint32), g["val"].view(np.uint32))
            assert got.astype(np.float64).sum() == float(g["total"])
        else:
            ok, worst, i = O.check_values(got[g["pos"]], g["val"], mag=mag[g["pos"]])
            assert ok, (name, K, i, worst)
            assert abs(got.astype(np.float64).sum() - float(g["total"])) <= 1e-5 * mag.sum()
