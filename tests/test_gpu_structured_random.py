"""Seeded random matrices with mixed structure (dense tiles, repeated row groups,
block rows, long rows, empty stretches), every strategy against the oracle.  The
point is the ownership logic: each stored entry must be computed by exactly one of
the tile, panel and row kernels, whatever the mixture."""
import numpy as np
import pytest

from dphpc_amd import capi
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32
STRATEGIES = [capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED, capi.ROW_WAVE, capi.SHORT_ROWS, capi.FLAT]


def build_case(seed):
    rng = np.random.default_rng(seed)
    K = int(rng.choice([16, 32, 32, 64, 128, 48, 20]))
    N = int(rng.integers(40, 900))
    rows = []
    target = int(rng.integers(20, 400))
    while len(rows) < target:
        kind = rng.integers(0, 7)
        if kind == 0:                                   # identical group of 8/16/3 rows
            n = int(rng.choice([8, 8, 16, 3, 24]))
            cols = np.sort(rng.choice(N, int(rng.integers(1, min(N, 200))), replace=False))
            rows += [cols.copy() for _ in range(n)]
        elif kind == 1:                                 # dense tile strip: 16 rows over aligned 16-col tiles
            tiles = np.sort(rng.choice(max(1, N // 16), int(rng.integers(1, max(2, N // 32))), replace=False))
            cols = (tiles[:, None] * 16 + np.arange(16)[None, :]).ravel()
            cols = cols[cols < N]
            fill = rng.choice([1.0, 0.7, 0.4])
            for _ in range(16):
                keep = rng.random(len(cols)) < fill
                rows.append(cols[keep])
        elif kind == 2:                                 # short random rows
            for _ in range(int(rng.integers(1, 40))):
                rows.append(np.sort(rng.choice(N, int(rng.integers(0, min(N, 12))), replace=False)))
        elif kind == 3:                                 # a long row
            rows.append(np.sort(rng.choice(N, int(rng.integers(N // 2, N)), replace=False)))
        elif kind == 4:                                 # empty rows
            rows += [np.zeros(0, np.int64)] * int(rng.integers(1, 20))
        elif kind == 5:                                 # 8-row block rows with 8-wide blocks (FEM like)
            nb = int(rng.integers(1, max(2, N // 16)))
            bc = np.sort(rng.choice(max(1, N // 8), nb, replace=False))
            cols = (bc[:, None] * 8 + np.arange(8)[None, :]).ravel()
            cols = cols[cols < N]
            rows += [cols.copy() for _ in range(8)]
        else:                                           # medium random rows
            for _ in range(int(rng.integers(1, 10))):
                rows.append(np.sort(rng.choice(N, int(rng.integers(20, min(N, 150))), replace=False)))
    # misalign everything now and then
    if rng.random() < 0.5:
        rows = [np.zeros(0, np.int64)] * int(rng.integers(1, 7)) + rows
    M = len(rows)
    lens = np.array([len(r) for r in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = (np.concatenate(rows) if lens.sum() else np.zeros(0)).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    return M, N, K, rowptr, col, val, A, B


@pytest.mark.parametrize("seed", range(40))
def test_structured_random(engine_factory, seed):
    M, N, K, rowptr, col, val, A, B = build_case(1000 + seed)
    ref = O.sddmm_csr(rowptr, col, val, A, B)
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    e = engine_factory()
    e.set_dense(A, B)
    e.set_csr(M, N, rowptr, col, val)
    for strategy in STRATEGIES:
        e.plan(strategy)
        e.run()
        got = e.values()
        st = e.stats()
        ok, worst, i = O.check_values(got, ref, mag=mag)
        assert ok, (seed, capi.STRATEGY_NAMES[strategy], M, N, K, i, got[i], ref[i], worst)
        if st.strategy_used in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
            owned = st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long
            assert owned == len(col), (seed, capi.STRATEGY_NAMES[strategy], st.as_dict())
    # bf16 on the same structure
    Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
    if K % 8 == 0:
        Af, Bf = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K)
        refb = O.sddmm_csr(rowptr, col, val, Af, Bf)
        _, magb = O.sddmm_csr_f64(rowptr, col, val, Af, Bf)
        e.set_dense(Ab, Bb, capi.BF16)
        for strategy in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
            e.plan(strategy)
            e.run()
            ok, worst, i = O.check_values(e.values(), refb, mag=magb)
            assert ok, (seed, "bf16", capi.STRATEGY_NAMES[strategy], i, worst)
    e.close()
