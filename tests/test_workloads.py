"""The synthetic workloads have the structure the benchmark shapes call for."""
import numpy as np
import pytest

from dphpc_amd import workloads as W


@pytest.mark.parametrize("name", list(W.CONFIGS))
def test_small_presets_are_valid_csr(name):
    w = W.make(name, "small")
    assert w.rowptr[0] == 0 and w.rowptr[-1] == w.nnz and len(w.rowptr) == w.M + 1
    assert np.all(np.diff(w.rowptr) >= 0)
    assert w.col.min() >= 0 and w.col.max() < w.N
    r = w.rows()
    assert np.all((np.diff(r) > 0) | (np.diff(w.col) > 0)), "columns sorted and unique inside rows"
    assert w.A.shape == (w.M, w.K) and w.B.shape == (w.N, w.K)
    assert w.A.dtype == np.float32 and w.sval.dtype == np.float32
    w2 = W.make(name, "small")
    np.testing.assert_array_equal(w.col, w2.col)       # seeded
    np.testing.assert_array_equal(w.A, w2.A)


def test_shapes_at_benchmark_size():
    w = W.make("small_uniform")
    assert w.M == 656 and abs(w.nnz - 18964) < 400
    w = W.make("fem_banded")
    assert w.M == 36000 and abs(w.nnz - 14.2e6) < 0.2e6
    lens = np.diff(w.rowptr)
    assert lens.min() >= 8 * 49 and lens.max() <= 8 * 50
    r = w.rows()
    assert np.abs(w.col.astype(np.int64) - r).max() <= 3000 + 8
    # dense 8x8 blocks: the 8 rows of a block row share their column list
    np.testing.assert_array_equal(w.col[w.rowptr[8]:w.rowptr[9]], w.col[w.rowptr[15]:w.rowptr[16]])
    w = W.make("mixed_density")
    lens = np.diff(w.rowptr)
    assert w.M == 30000 and abs(w.nnz - 2.0e6) < 0.1e6
    assert np.count_nonzero(lens > 300) == 3000 and np.all(lens[lens <= 300] <= 20)
    w = W.make("dense_tiles")
    assert (w.M, w.N) == (4562, 5761) and w.nnz == 9621 * 256 and w.dtype == "bf16"
    assert w.A_bits.dtype == np.uint16
    assert np.all(np.diff(w.rowptr) % 16 == 0)


def test_power_law_small_is_skewed():
    w = W.make("power_law", "small")
    lens = np.diff(w.rowptr)
    assert np.median(lens) <= 10 and lens.max() > 500
    assert np.all(w.sval == 1.0)
    counts = np.bincount(w.col, minlength=w.N)
    top = np.sort(counts)[::-1]
    assert top[: w.N // 100].sum() > 0.1 * w.nnz       # hot columns
