"""Seeded synthetic SDDMM workloads: the five benchmark shapes.

Every generator returns a `Workload` with a CSR sampling matrix whose columns are
sorted and unique inside each row (what the reference's CSR constructor produces,
src/matrices/CSR.hpp:169-194) and dense fp32 A (M x K), B (N x K).  `size` scales
a shape down for tests ("full" is the benchmark size).  The reference draws its
own synthetic inputs from an unseeded std::random_device
(src/utils/random_generator.hpp:13-14), so nothing here can or needs to match it
draw for draw; seeds are fixed so that runs are reproducible.
"""
from dataclasses import dataclass, field

import numpy as np

SEED_BASE = 0x5DD3300


@dataclass
class Workload:
    name: str
    M: int
    N: int
    K: int
    rowptr: np.ndarray
    col: np.ndarray
    sval: np.ndarray
    A: np.ndarray                 # fp32 (for bf16 workloads: the bf16-rounded values)
    B: np.ndarray
    dtype: str = "f32"            # "f32" | "bf16" | "f16"
    A_bits: np.ndarray = None     # uint16 bit patterns when dtype is "bf16" or "f16"
    B_bits: np.ndarray = None
    meta: dict = field(default_factory=dict)

    @property
    def nnz(self):
        return int(len(self.col))

    def rows(self):
        """Row index per stored entry (COO view, same entry order)."""
        return np.repeat(np.arange(self.M, dtype=np.int32), np.diff(self.rowptr)).astype(np.int32)

    def flops(self):
        return 2.0 * self.nnz * self.K

    def bytes_gathered(self):
        e = 4 if self.dtype == "f32" else 2
        nonempty = int(np.count_nonzero(np.diff(self.rowptr)))
        return 4.0 * (self.M + 1) + 12.0 * self.nnz + e * self.K * nonempty + e * self.K * self.nnz

    def bytes_compulsory(self):
        e = 4 if self.dtype == "f32" else 2
        nonempty = int(np.count_nonzero(np.diff(self.rowptr)))
        touched = int(len(np.unique(self.col)))
        return 4.0 * (self.M + 1) + 12.0 * self.nnz + e * self.K * (nonempty + touched)


def _csr_from_keys(M, N, keys):
    """keys = row*N + col (int64, any order, duplicates allowed) -> sorted unique CSR."""
    keys = np.unique(keys)
    rows = keys // N
    col = (keys - rows * N).astype(np.int32)
    counts = np.bincount(rows, minlength=M)
    rowptr = np.zeros(M + 1, np.int32)
    np.cumsum(counts, out=rowptr[1:])
    return rowptr, col


def _dense(rng, rows, K, dist):
    if dist == "uniform":
        return rng.uniform(-1.0, 1.0, size=(rows, K)).astype(np.float32)
    if dist == "normal":
        return rng.standard_normal(size=(rows, K), dtype=np.float32)
    raise ValueError(dist)


# --------------------------------------------------------------------------- 1
def small_uniform(K=32, M=656, nnz_target=18964, seed=SEED_BASE + 1):
    """Square S, ~4.4% density, column positions uniform per row, S ~ U[0,1)."""
    rng = np.random.default_rng(seed)
    N = M
    per = nnz_target / M
    lens = np.clip(np.rint(per + rng.integers(-2, 3, size=M)), 0, N).astype(np.int64)
    cols = [np.sort(rng.choice(N, size=int(l), replace=False)) for l in lens]
    rowptr = np.zeros(M + 1, np.int32)
    np.cumsum(lens, out=rowptr[1:])
    col = np.concatenate(cols).astype(np.int32) if M else np.zeros(0, np.int32)
    sval = rng.random(len(col), dtype=np.float32)
    return Workload("small_uniform", M, N, K, rowptr, col, sval,
                    _dense(rng, M, K, "uniform"), _dense(rng, N, K, "uniform"))


# --------------------------------------------------------------------------- 2
def fem_banded(K=32, M=36000, half_width=3000, blocks_per_row=49.4, seed=SEED_BASE + 2):
    """Dense 8x8 blocks scattered inside a band around the diagonal."""
    assert M % 8 == 0
    rng = np.random.default_rng(seed)
    N = M
    nbr = M // 8
    hw = max(1, half_width // 8)
    base = int(np.floor(blocks_per_row))
    extra = blocks_per_row - base
    col_parts, len_parts = [], []
    off8 = np.arange(8, dtype=np.int32)
    for b in range(nbr):
        lo, hi = max(0, b - hw), min(nbr - 1, b + hw)
        nb = min(hi - lo + 1, base + (1 if rng.random() < extra else 0))
        bc = np.sort(rng.choice(hi - lo + 1, size=nb, replace=False) + lo).astype(np.int32)
        rowcols = (bc[:, None] * 8 + off8[None, :]).ravel()
        col_parts.append(np.tile(rowcols, 8))
        len_parts.append(np.full(8, len(rowcols), np.int64))
    col = np.concatenate(col_parts).astype(np.int32)
    lens = np.concatenate(len_parts)
    rowptr = np.zeros(M + 1, np.int32)
    np.cumsum(lens, out=rowptr[1:])
    sval = rng.random(len(col), dtype=np.float32)
    return Workload("fem_banded", M, N, K, rowptr, col, sval,
                    _dense(rng, M, K, "uniform"), _dense(rng, N, K, "uniform"),
                    meta={"half_width": half_width, "block": 8})


# --------------------------------------------------------------------------- 3
def _zipf_alpha_for_mean(mean, trunc):
    k = np.arange(1, trunc + 1, dtype=np.float64)
    lo, hi = 1.01, 4.0
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        w = k ** (-mid)
        m = float((k * w).sum() / w.sum())
        if m > mean:
            lo = mid
        else:
            hi = mid
    return 0.5 * (lo + hi)


def power_law(K=32, M=2_600_000, nnz_target=36_000_000, trunc=50_000, col_beta=0.8, seed=SEED_BASE + 3):
    """Zipf row lengths (alpha fitted so that the truncated mean gives ~nnz_target;
    ~1.8-1.9 at full size), Zipf-skewed column popularity over a random permutation
    of the columns, S values all 1.0, A,B ~ N(0,1)."""
    rng = np.random.default_rng(seed)
    N = M
    trunc = int(min(trunc, N))
    # duplicates drawn inside a row are dropped, so aim a little high
    alpha = _zipf_alpha_for_mean(1.095 * nnz_target / M, trunc)
    k = np.arange(1, trunc + 1, dtype=np.float64)
    cdf = np.cumsum(k ** (-alpha))
    cdf /= cdf[-1]
    lens = (np.searchsorted(cdf, rng.random(M), side="left") + 1).astype(np.int64)
    total = int(lens.sum())
    rows = np.repeat(np.arange(M, dtype=np.int64), lens)
    # continuous inverse CDF of p(x) ~ x^-beta on [1, N+1)
    u = rng.random(total)
    one_m = 1.0 - col_beta
    rank = np.floor((u * ((N + 1.0) ** one_m - 1.0) + 1.0) ** (1.0 / one_m)).astype(np.int64) - 1
    np.clip(rank, 0, N - 1, out=rank)
    perm = rng.permutation(N).astype(np.int64)
    keys = rows * N + perm[rank]
    del rows, rank, u
    rowptr, col = _csr_from_keys(M, N, keys)
    sval = np.ones(len(col), np.float32)
    return Workload("power_law", M, N, K, rowptr, col, sval,
                    _dense(rng, M, K, "normal"), _dense(rng, N, K, "normal"),
                    meta={"alpha": alpha, "col_beta": col_beta, "trunc": trunc})


# --------------------------------------------------------------------------- 4
def mixed_density(K=32, M=30000, dense_frac=0.10, window=1385, fill=0.40, seed=SEED_BASE + 4):
    """10% of the rows near-dense inside a contiguous column window, 90% with 5..20
    uniform-random entries."""
    rng = np.random.default_rng(seed)
    N = M
    window = min(window, N)
    n_dense = int(round(M * dense_frac))
    dense_rows = np.sort(rng.choice(M, size=n_dense, replace=False))
    is_dense = np.zeros(M, bool)
    is_dense[dense_rows] = True
    keys = []
    starts = rng.integers(0, N - window + 1, size=n_dense)
    for r, s in zip(dense_rows, starts):
        cols = np.nonzero(rng.random(window) < fill)[0] + s
        keys.append(r * np.int64(N) + cols.astype(np.int64))
    sparse_rows = np.nonzero(~is_dense)[0]
    lens = rng.integers(5, 21, size=len(sparse_rows))
    lens = np.minimum(lens, N)
    rr = np.repeat(sparse_rows.astype(np.int64), lens)
    keys.append(rr * N + rng.integers(0, N, size=len(rr)))
    rowptr, col = _csr_from_keys(M, N, np.concatenate(keys))
    sval = rng.random(len(col), dtype=np.float32)
    return Workload("mixed_density", M, N, K, rowptr, col, sval,
                    _dense(rng, M, K, "uniform"), _dense(rng, N, K, "uniform"),
                    meta={"dense_rows": n_dense, "window": window, "fill": fill})


# --------------------------------------------------------------------------- 5
def dense_tiles(K=128, M=4562, N=5761, tile_frac=0.09377, seed=SEED_BASE + 5, bf16=True, f16=False):
    """Fully dense 16x16 tiles at random tile positions; A,B in bf16 (round to
    nearest even of U[-1,1]) with the fp32 view of the rounded values kept for the
    oracle.  bf16=False: fp32 operands; f16=True: IEEE half instead of bf16."""
    from .capi import to_bf16, from_bf16, to_f16, from_f16
    rng = np.random.default_rng(seed)
    tr, tc = M // 16, N // 16
    n_tiles = int(round(tr * tc * tile_frac))
    picks = np.sort(rng.choice(tr * tc, size=n_tiles, replace=False))
    ti, tj = picks // tc, picks % tc
    off = np.arange(16, dtype=np.int64)
    rows = (ti[:, None, None] * 16 + off[None, :, None]) + np.zeros((1, 1, 16), np.int64)
    cols = (tj[:, None, None] * 16 + off[None, None, :]) + np.zeros((1, 16, 1), np.int64)
    keys = (rows * N + cols).ravel()
    rowptr, col = _csr_from_keys(M, N, keys)
    sval = rng.random(len(col), dtype=np.float32)
    A = _dense(rng, M, K, "uniform")
    B = _dense(rng, N, K, "uniform")
    if f16:
        Ab, Bb = to_f16(A), to_f16(B)
        return Workload("dense_tiles", M, N, K, rowptr, col, sval,
                        from_f16(Ab).reshape(M, K), from_f16(Bb).reshape(N, K), dtype="f16",
                        A_bits=Ab.reshape(M, K), B_bits=Bb.reshape(N, K), meta={"tiles": n_tiles})
    if not bf16:
        return Workload("dense_tiles", M, N, K, rowptr, col, sval, A, B, meta={"tiles": n_tiles})
    Ab, Bb = to_bf16(A), to_bf16(B)
    return Workload("dense_tiles", M, N, K, rowptr, col, sval,
                    from_bf16(Ab).reshape(M, K), from_bf16(Bb).reshape(N, K), dtype="bf16",
                    A_bits=Ab.reshape(M, K), B_bits=Bb.reshape(N, K), meta={"tiles": n_tiles})


# --------------------------------------------------------------------------- 6
def similar_rows(K=32, M=40000, group=16, base_len=200, drop=0.10, window=800, seed=SEED_BASE + 6):
    """Groups of `group` consecutive rows that share most of their columns without being
    identical (rows of a mesh with mostly common neighbours): every group draws base_len
    columns inside a window of `window` columns, every row of the group drops a fraction
    `drop` of them.  Not one of the benchmark configurations of the reference; the shape
    the union strips are for."""
    rng = np.random.default_rng(seed)
    N = M
    keys = []
    for g in range(M // group):
        c0 = int(rng.integers(0, N - window + 1))
        base = np.sort(rng.choice(window, size=base_len, replace=False)) + c0
        for i in range(group):
            keep = base[rng.random(base_len) >= drop]
            keys.append((g * group + i) * np.int64(N) + keep.astype(np.int64))
    rowptr, col = _csr_from_keys(M, N, np.concatenate(keys))
    sval = rng.random(len(col), dtype=np.float32)
    return Workload("similar_rows", M, N, K, rowptr, col, sval,
                    _dense(rng, M, K, "uniform"), _dense(rng, N, K, "uniform"),
                    meta={"group": group, "base_len": base_len, "drop": drop})


# ---------------------------------------------------------------------------
# name -> (generator, kwargs at benchmark size, kwargs at test size)
CONFIGS = {
    "small_uniform": (small_uniform, {}, {}),
    "fem_banded": (fem_banded, {}, dict(M=2880, half_width=480, blocks_per_row=24.4)),
    "power_law": (power_law, {}, dict(M=60000, nnz_target=600000, trunc=4000)),
    "mixed_density": (mixed_density, {}, dict(M=3000, window=700)),
    "dense_tiles": (dense_tiles, {}, dict(M=1140, N=1445)),
    "similar_rows": (similar_rows, {}, dict(M=1600)),
}


def make(name, size="full", **overrides):
    gen, full, small = CONFIGS[name]
    kw = dict(full if size == "full" else small)
    kw.update(overrides)
    return gen(**kw)

