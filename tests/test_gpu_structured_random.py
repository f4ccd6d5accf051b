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
    for strategy in STRATEGIES:
        e.set_csr(M, N, rowptr, col, val)    # again for every strategy: clears P, nothing passes on stale values
        e.plan(strategy)
        e.run()
        got = e.values()
        st = e.stats()
        ok, worst, i = O.check_values(got, ref, mag=mag)
        assert ok, (seed, capi.STRATEGY_NAMES[strategy], M, N, K, i, got[i], ref[i], worst)
        if st.strategy_used in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
            owned = st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long
            assert owned == len(col), (seed, capi.STRATEGY_NAMES[strategy], st.as_dict())
    # SDDMM followed by SpMM on the same mixture: the panels of the plan take their own kernel,
    # rows that tiles own in the SDDMM take the gather kernels
    if K % 4 == 0:
        ref_p, ref_o = O.fusedmm_csr(rowptr, col, val, A, B)
        _, mag_o = O.fusedmm_csr_f64(rowptr, col, val, A, B)
        for strategy in (capi.AUTO, capi.LDS_TILED):
            e.set_csr(M, N, rowptr, col, val)
            e.plan(strategy)
            got_o = e.run_fused()
            ok, worst, i = O.check_values(e.values(), ref, mag=mag)
            assert ok, (seed, "fused P", capi.STRATEGY_NAMES[strategy], i, worst)
            ok, worst, i = O.check_values(got_o[:M].ravel(), ref_o.ravel(), mag=mag_o.ravel())
            assert ok, (seed, "fused O", capi.STRATEGY_NAMES[strategy], i, worst)
    # bf16 on the same structure
    Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
    if K % 8 == 0:
        Af, Bf = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K)
        refb = O.sddmm_csr(rowptr, col, val, Af, Bf)
        _, magb = O.sddmm_csr_f64(rowptr, col, val, Af, Bf)
        e.set_dense(Ab, Bb, capi.BF16)
        for strategy in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
            e.set_csr(M, N, rowptr, col, val)
            e.plan(strategy)
            e.run()
            ok, worst, i = O.check_values(e.values(), refb, mag=magb)
            assert ok, (seed, "bf16", capi.STRATEGY_NAMES[strategy], i, worst)
    e.close()


def _host_tile_model(M, rowptr, col, min_fill):
    """What the strip classifier must decide: a 16-row strip goes to the tile path iff
    every row is strictly increasing and it holds at least min_fill entries per
    non-empty 16x16 tile on average."""
    tiles = entries = 0
    for s in range((M + 15) // 16):
        lo, hi = rowptr[s * 16], rowptr[min(M, s * 16 + 16)]
        if hi == lo:
            continue
        ok = True
        tset = set()
        for r in range(s * 16, min(M, s * 16 + 16)):
            c = col[rowptr[r]:rowptr[r + 1]].astype(np.int64)
            if len(c) > 1 and (np.diff(c) <= 0).any():
                ok = False
                break
            tset.update((c >> 4).tolist())
        if ok and (hi - lo) >= min_fill * len(tset):
            tiles += len(tset)
            entries += hi - lo
    return tiles, entries


@pytest.mark.parametrize("seed", range(12))
def test_strip_classifier_matches_host_model(engine_factory, monkeypatch, seed):
    """Tile counts and covered entries reported by the device classifier against the
    host model, on matrices whose strips mix clustered, scattered, unsorted and
    duplicated rows (K=16: 64-byte rows, so the tile path applies).  Strips of
    gathered rows are switched off for the comparison and checked on top of it."""
    monkeypatch.setenv("SDDMM_GATHERED", "0")
    rng = np.random.default_rng(7000 + seed)
    N = int(rng.choice([100, 1000, 40000, 600_000]))
    M = int(rng.integers(17, 400))
    rows = []
    for r in range(M):
        kind = rng.integers(0, 6)
        if kind == 0:
            c = np.zeros(0, np.int64)
        elif kind == 1:                                   # clustered around a few tile columns
            base = rng.choice(max(1, N // 16), int(rng.integers(1, 6))) * 16
            c = np.unique(np.clip((base[:, None] + np.arange(16)[None, :]).ravel(), 0, N - 1))
            c = c[rng.random(len(c)) < rng.choice([1.0, 0.6])]
        elif kind == 2:                                   # scattered
            c = np.sort(rng.choice(N, int(rng.integers(1, min(N, 60))), replace=False))
        elif kind == 3:                                   # long clustered run
            s0 = int(rng.integers(0, max(1, N - 700)))
            c = np.arange(s0, min(N, s0 + int(rng.integers(100, 700))))
        elif kind == 4 and rng.random() < 0.3:            # not sorted
            c = rng.permutation(np.sort(rng.choice(N, int(rng.integers(2, min(N, 30))), replace=False)))
        elif kind == 5 and rng.random() < 0.3:            # a duplicate
            c = np.sort(rng.choice(N, int(rng.integers(2, min(N, 30))), replace=False))
            c[1] = c[0]
        else:
            c = np.sort(rng.choice(N, int(rng.integers(1, min(N, 20))), replace=False))
        rows.append(c.astype(np.int64))
    # make some strips homogeneous so that whole strips qualify
    for s in range(0, M - 16, 48):
        base = rng.choice(max(1, N // 16), 3) * 16
        c = np.unique(np.clip((base[:, None] + np.arange(16)[None, :]).ravel(), 0, N - 1))
        for r in range(s, s + 16):
            rows[r] = c[rng.random(len(c)) < 0.8]
    lens = np.array([len(r) for r in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    K = 16
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    ref = O.sddmm_csr(rowptr, col, val, A, B)
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    e = engine_factory()
    e.set_dense(A, B)
    for strategy, min_fill in ((capi.MFMA_TILE, 1), (capi.AUTO, 96)):
        e.set_csr(M, N, rowptr, col, val)    # clears P
        e.plan(strategy)
        e.run()
        st = e.stats()
        want_tiles, want_entries = _host_tile_model(M, rowptr, col, min_fill)
        if st.strategy_used != capi.FLAT:                 # AUTO may resolve to FLAT when nothing qualifies
            assert (st.mfma_tiles, st.nnz_mfma) == (want_tiles, want_entries), (seed, capi.STRATEGY_NAMES[strategy], N, M)
        else:
            assert want_tiles == 0
        ok, worst, i = O.check_values(e.values(), ref, mag=mag)
        assert ok, (seed, capi.STRATEGY_NAMES[strategy], i, worst)
    # gathered strips can only add to what the 16-row strips took, and every entry
    # still has exactly one owner
    natural = (st.mfma_tiles, st.nnz_mfma) if st.strategy_used != capi.FLAT else (0, 0)
    monkeypatch.setenv("SDDMM_GATHERED", "1")
    e.set_csr(M, N, rowptr, col, val)
    e.plan(capi.AUTO)
    e.run()
    st = e.stats()
    if st.strategy_used != capi.FLAT:
        assert st.mfma_tiles >= natural[0] and st.nnz_mfma >= natural[1]
        assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == len(col)
    ok, worst, i = O.check_values(e.values(), ref, mag=mag)
    assert ok, (seed, "AUTO with gathered strips", i, worst)
    e.close()


def build_similarity_case(seed):
    """Mixtures aimed at the ownership logic of the tile paths: groups of similar rows
    (union strips), near-dense rows in windows (gathered strips), identical groups
    (panels), aligned dense tiles, with short, long, empty, unsorted and duplicated rows
    in between; K, N and the operand type vary with the seed."""
    rng = np.random.default_rng(90000 + seed)
    N = int(rng.choice([300, 5000, 100000, 400000]))
    K = int(rng.choice([16, 32, 64, 128, 256, 24]))
    dt = str(rng.choice(["f32", "f32", "bf16", "f16"])) if K % 8 == 0 else "f32"
    rows = []
    target = int(rng.integers(30, 700))
    while len(rows) < target:
        kind = int(rng.integers(0, 8))
        if kind == 0:
            g = int(rng.choice([3, 8, 16, 16, 20, 32]))
            bl = int(rng.integers(20, min(N, 300)))
            win = int(min(N, bl * rng.integers(1, 30)))
            base = np.sort(rng.choice(win, bl, replace=False)) + int(rng.integers(0, N - win + 1))
            flip = float(rng.choice([0.0, 0.05, 0.3]))
            rows += [base[rng.random(bl) >= flip] for _ in range(g)]
        elif kind == 1:
            win = int(min(N, rng.integers(100, 1500)))
            c0 = int(rng.integers(0, N - win + 1))
            rows.append(c0 + np.nonzero(rng.random(win) < rng.choice([0.3, 0.6, 0.95]))[0])
        elif kind == 2:
            rows += [np.sort(rng.choice(N, int(rng.integers(0, 15)), replace=False)) for _ in range(int(rng.integers(1, 30)))]
        elif kind == 3:
            rows.append(np.sort(rng.choice(N, int(rng.integers(min(N, 100), min(N, 3000))), replace=False)))
        elif kind == 4:
            rows += [np.zeros(0, np.int64)] * int(rng.integers(1, 20))
        elif kind == 5:
            base = np.sort(rng.choice(N, int(rng.integers(4, min(N, 200))), replace=False))
            rows += [base.copy() for _ in range(int(rng.choice([8, 16, 24])))]
        elif kind == 6:
            tcs = np.sort(rng.choice(max(1, N // 16), int(rng.integers(1, 6)), replace=False))
            cols = (tcs[:, None] * 16 + np.arange(16)[None, :]).ravel()
            cols = cols[cols < N]
            rows += [cols[rng.random(len(cols)) < rng.choice([1.0, 0.5])] for _ in range(16)]
        else:
            c = np.sort(rng.choice(N, int(rng.integers(2, 40)), replace=False))
            if rng.random() < 0.5:
                c = c[::-1].copy()
            else:
                c[1] = c[0]
            rows.append(c)
    M = len(rows)
    lens = np.array([len(r) for r in rows])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    return M, N, K, dt, rowptr, col, val, A, B


@pytest.mark.parametrize("seed", range(30))
def test_similarity_mixtures(engine_factory, seed):
    M, N, K, dt, rowptr, col, val, A, B = build_similarity_case(seed)
    e = engine_factory()
    if dt == "bf16":
        Ab, Bb = capi.to_bf16(A).reshape(M, K), capi.to_bf16(B).reshape(N, K)
        A, B = capi.from_bf16(Ab).reshape(M, K), capi.from_bf16(Bb).reshape(N, K)
        e.set_dense(Ab, Bb, capi.BF16)
    elif dt == "f16":
        Ab, Bb = capi.to_f16(A).reshape(M, K), capi.to_f16(B).reshape(N, K)
        A, B = capi.from_f16(Ab).reshape(M, K), capi.from_f16(Bb).reshape(N, K)
        e.set_dense(Ab, Bb, capi.F16)
    else:
        e.set_dense(A, B)
    ref = O.sddmm_csr(rowptr, col, val, A, B)
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    for strategy in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED, capi.FLAT):
        e.set_csr(M, N, rowptr, col, val)    # clears P
        e.plan(strategy)
        e.run()
        st = e.stats()
        ok, worst, i = O.check_values(e.values(), ref, mag=mag)
        assert ok, (seed, capi.STRATEGY_NAMES[strategy], dt, M, N, K, i, worst)
        if st.strategy_used in (capi.AUTO, capi.MFMA_TILE, capi.LDS_TILED):
            assert st.nnz_mfma + st.nnz_panel + st.nnz_short + st.nnz_medium + st.nnz_long == len(col), (seed, strategy)
    e.close()
