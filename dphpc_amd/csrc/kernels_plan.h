// Structure kernels of the plan phase: validation, CSR<->COO index expansion,
// row statistics.  Everything that looks at S's pattern runs here, on the
// device; the host reads back only the small PlanCounters block.
#pragma once
#include "device_utils.h"

namespace sddmm {

// Host-side summary of what the structure kernels counted.
struct PlanCounters {
    unsigned int bad_pattern;      // != 0: malformed CSR/COO
    unsigned int coo_unsorted;     // != 0: COO rows not non-decreasing
    unsigned int max_len;          // longest row
    unsigned long long rows_nonempty;
    unsigned long long rows_short, rows_medium, rows_long;
    unsigned long long nnz_short, nnz_medium, nnz_long;
    unsigned long long n_items;    // work items of the wave-per-segment kernel
    unsigned long long n_tiles, nnz_tiles, tiles_scanned;     // dense-tile path: 16-row and gathered strips
    unsigned long long n_utiles, nnz_utiles, utiles_scanned;  // dense-tile path: union strips
    unsigned long long n_panels, nnz_panels, panel_items;     // row-panel path
};

// The same counters on the device.  Sums that thousands of workgroups contribute to
// are spread over SPREAD slots chosen by workgroup id (same-address atomics were
// measured at ~10 ns each, which made the counting kernels atomic-bound); the host
// adds the slots up after the copy.
constexpr int SPREAD = 64;
enum CounterKind {
    K_ROWS_NONEMPTY = 0,
    K_ROWS_SHORT, K_ROWS_MEDIUM, K_ROWS_LONG, K_NNZ_SHORT, K_NNZ_MEDIUM, K_NNZ_LONG,   // row classifier
    K_TILES, K_NNZ_TILES, K_UTILES, K_NNZ_UTILES, K_PANELS, K_NNZ_PANELS,              // ownership classifiers
    K_KINDS
};
struct DevCounters {
    unsigned int bad_pattern, coo_unsorted, pad0, pad1;
    unsigned long long n_items, tiles_scanned, panel_items;          // scan totals, one writer each
    unsigned long long n_candidates;                                 // rows offered to the gathered strips
    unsigned long long utiles_scanned, short_scanned;                // scan totals: union strips, entries of the short rows
    unsigned int max_len[SPREAD];
    unsigned long long k[K_KINDS][SPREAD];
};

__device__ __forceinline__ void spread_add(DevCounters *dc, int kind, unsigned long long v) {
    if (v) atomicAdd(&dc->k[kind][blockIdx.x & (SPREAD - 1)], v);
}

inline PlanCounters summarize(const DevCounters &d) {
    PlanCounters p{};
    p.bad_pattern = d.bad_pattern;
    p.coo_unsorted = d.coo_unsorted;
    unsigned long long sum[K_KINDS] = {0};
    for (int s = 0; s < SPREAD; ++s) {
        p.max_len = d.max_len[s] > p.max_len ? d.max_len[s] : p.max_len;
        for (int k = 0; k < K_KINDS; ++k) sum[k] += d.k[k][s];
    }
    p.rows_nonempty = sum[K_ROWS_NONEMPTY];
    p.rows_short = sum[K_ROWS_SHORT]; p.rows_medium = sum[K_ROWS_MEDIUM]; p.rows_long = sum[K_ROWS_LONG];
    p.nnz_short = sum[K_NNZ_SHORT]; p.nnz_medium = sum[K_NNZ_MEDIUM]; p.nnz_long = sum[K_NNZ_LONG];
    p.n_tiles = sum[K_TILES]; p.nnz_tiles = sum[K_NNZ_TILES];
    p.n_utiles = sum[K_UTILES]; p.nnz_utiles = sum[K_NNZ_UTILES]; p.utiles_scanned = d.utiles_scanned;
    p.n_panels = sum[K_PANELS]; p.nnz_panels = sum[K_NNZ_PANELS];
    p.n_items = d.n_items; p.tiles_scanned = d.tiles_scanned; p.panel_items = d.panel_items;
    return p;
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ unsigned int wave_max_u32(unsigned int v) {
    for (int o = 32; o > 0; o >>= 1) {
        unsigned int x = __shfl_xor(v, o, WAVE);
        v = x > v ? x : v;
    }
    return v;
}

// What a plan clears before its classifiers run, in one launch (a fill through the
// runtime is a launch of its own for every region): the row-ownership bytes and every
// counter except what validation measured (non-empty rows, longest row).  rows_only: just
// the row classes and the item total, for the second count after the gathered strips.
__global__ __launch_bounds__(256) void k_plan_reset(unsigned char *__restrict__ owner, int64_t owner_bytes,
                                                    DevCounters *pc, int rows_only) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (!rows_only) {
        // 16 bytes per thread (the array is 256-byte aligned and padded to 64 bytes past the rows)
        const int64_t at = i * 16;
        if (at + 16 <= owner_bytes) *reinterpret_cast<uint4 *>(owner + at) = make_uint4(0u, 0u, 0u, 0u);
        else for (int64_t q = at; q < owner_bytes; ++q) owner[q] = 0;
    }
    if (blockIdx.x == 0) {
        const int first = K_ROWS_SHORT, last = rows_only ? K_NNZ_LONG : K_NNZ_PANELS;
        for (int k = first; k <= last; ++k)
            for (int sl = threadIdx.x; sl < SPREAD; sl += blockDim.x) pc->k[k][sl] = 0ull;
        if (threadIdx.x == 0) {
            pc->n_items = 0ull;
            pc->short_scanned = 0ull;
            if (!rows_only) {
                pc->tiles_scanned = 0ull; pc->panel_items = 0ull; pc->n_candidates = 0ull; pc->utiles_scanned = 0ull;
            }
        }
    }
}

// rowptr[0]==0, rowptr[M]==nnz, non-decreasing; also counts non-empty rows and the
// longest row.  One lane per row, one set of atomics per workgroup.
__global__ __launch_bounds__(256) void k_check_rowptr(const int32_t *__restrict__ rowptr, int M,
                                                      int64_t nnz, DevCounters *pc) {
    __shared__ unsigned int sh_ne, sh_mx, sh_bad;
    if (threadIdx.x == 0) { sh_ne = 0; sh_mx = 0; sh_bad = 0; }
    __syncthreads();
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned int bad = 0, len = 0;
    if (i < M) {
        const int32_t s = rowptr[i], e = rowptr[i + 1];
        if (e < s || s < 0) bad = 1; else len = (unsigned int)(e - s);
        if (i == 0 && s != 0) bad = 1;
        if (i == M - 1 && (int64_t)e != nnz) bad = 1;
    }
    const unsigned int ne = (unsigned int)__builtin_popcountll(__ballot(len > 0));
    const unsigned int mx = wave_max_u32(len);
    const unsigned long long anybad = __ballot(bad != 0);
    if (lane_id() == 0) {
        if (ne) atomicAdd(&sh_ne, ne);
        if (mx) atomicMax(&sh_mx, mx);
        if (anybad) atomicOr(&sh_bad, 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        spread_add(pc, K_ROWS_NONEMPTY, sh_ne);
        if (sh_mx) atomicMax(&pc->max_len[blockIdx.x & (SPREAD - 1)], sh_mx);
        if (sh_bad) atomicOr(&pc->bad_pattern, 1u);
    }
}

// every column index in [0,N)
__global__ __launch_bounds__(256) void k_check_index(const int32_t *__restrict__ idx, int64_t n,
                                                     int bound, DevCounters *pc) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    unsigned int bad = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int32_t c = idx[i];
        bad |= (c < 0 || c >= bound) ? 1u : 0u;
    }
    if (__ballot(bad != 0) && lane_id() == 0) atomicOr(&pc->bad_pattern, 1u);
}

// rowptr -> row index per stored entry (what the flat kernels read).  A wavefront
// takes 64 rows: short rows are written by their own lane, long ones by the
// whole wavefront.  Positions outside [0, limit) are never written, whatever the
// row pointer holds (it may come unvalidated from the caller).
__global__ __launch_bounds__(256) void k_expand_rows(const int32_t *__restrict__ rowptr, int M,
                                                     int32_t *__restrict__ rowidx, int64_t limit) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = lane_id();
    int32_t s = 0, e = 0;
    if (i < M) {
        s = rowptr[i];
        e = rowptr[i + 1];
        s = s < 0 ? 0 : s;
        e = (int64_t)e > limit ? (int32_t)limit : e;
    }
    const int len = e - s;
    constexpr int SHORT = 8;
    if (len <= SHORT) {
        for (int q = 0; q < len; ++q) rowidx[s + q] = (int32_t)i;
    }
    unsigned long long longmask = __ballot(len > SHORT);
    while (longmask) {
        const int src = __builtin_ctzll(longmask);
        longmask &= longmask - 1;
        const int32_t ss = __shfl(s, src, WAVE), ee = __shfl(e, src, WAVE);
        const int32_t rr = (int32_t)(i - lane + src);
        for (int32_t q = ss + lane; q < ee; q += WAVE) rowidx[q] = rr;
    }
}

// COO rows non-decreasing?  (one lane per entry)
__global__ __launch_bounds__(256) void k_check_coo_sorted(const int32_t *__restrict__ row, int64_t nnz,
                                                          DevCounters *pc) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    unsigned int uns = 0;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i + 1 < nnz; i += stride)
        uns |= row[i] > row[i + 1] ? 1u : 0u;
    if (__ballot(uns != 0) && lane_id() == 0) atomicOr(&pc->coo_unsorted, 1u);
}

// sorted COO row array -> rowptr.  Entry n closes every row in (row[n-1], row[n]].
__global__ __launch_bounds__(256) void k_rowptr_from_sorted_coo(const int32_t *__restrict__ row,
                                                                int64_t nnz, int M,
                                                                int32_t *__restrict__ rowptr) {
    const int64_t n = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (n > nnz) return;
    const int lo = n == 0 ? -1 : row[n - 1];
    const int hi = n == nnz ? M : row[n];
    for (int r = lo + 1; r <= hi; ++r) rowptr[r] = (int32_t)n;
}

}  // namespace sddmm

// ===========================================================================
// Row classifier of the AUTO strategy.
//
// A row is "short" when it has fewer than `ts` stored entries; short rows are
// computed by k_short_rows straight from rowptr, 64 consecutive rows per
// wavefront, and need no list.  Every other row becomes ceil(len/seg) work items
// of the wave-per-segment kernel; the item list is built with an exclusive scan
// of the per-row item counts (three kernels: block sums, scan of the block sums,
// write).  Nothing here touches col/values: the cost is O(M).
namespace sddmm {

constexpr int SCAN_BLOCK = 256;
constexpr int SCAN_ITEMS = 4;                       // rows per thread
constexpr int SCAN_TILE = SCAN_BLOCK * SCAN_ITEMS;  // rows per block

// owner (may be null): one byte per row, non-zero when the dense-tile path (1: a
// 16-row strip, 3: a strip of rows gathered by column window) or the row-panel path
// (2) computes the row; such rows count as empty here
// (only != 0: just the rows of that owner count as empty)
__device__ __forceinline__ unsigned int row_item_count(const int32_t *__restrict__ rowptr,
                                                       const unsigned char *__restrict__ owner, int64_t i,
                                                       int M, int ts, int seg, unsigned int *len_out, int only = 0) {
    if (i >= M || (owner && (only ? owner[i] == only : owner[i] != 0))) { *len_out = 0; return 0; }
    const unsigned int len = (unsigned int)(rowptr[i + 1] - rowptr[i]);
    *len_out = len;
    return len >= (unsigned int)ts ? (len + seg - 1) / seg : 0u;
}

// block-wide exclusive scan of one value per thread (SCAN_BLOCK threads); returns
// the exclusive prefix, *total receives the block sum
__device__ __forceinline__ unsigned int block_exclusive_scan(unsigned int v, unsigned int *total) {
    __shared__ unsigned int wave_sums[SCAN_BLOCK / WAVE];
    const int lane = lane_id(), wid = threadIdx.x >> 6;
    unsigned int incl = v;
    for (int o = 1; o < WAVE; o <<= 1) {
        const unsigned int up = __shfl_up(incl, o, WAVE);
        if (lane >= o) incl += up;
    }
    if (lane == WAVE - 1) wave_sums[wid] = incl;
    __syncthreads();
    unsigned int before = 0, all = 0;
    for (int w = 0; w < SCAN_BLOCK / WAVE; ++w) {
        const unsigned int s = wave_sums[w];
        if (w < wid) before += s;
        all += s;
    }
    __syncthreads();
    *total = all;
    return before + incl - v;
}

// pass 1: items per block of SCAN_TILE rows, plus the row statistics
__global__ __launch_bounds__(SCAN_BLOCK) void k_classify_count(const int32_t *__restrict__ rowptr,
                                                               const unsigned char *__restrict__ owner, int M,
                                                               int ts, int seg, unsigned int *__restrict__ block_sums,
                                                               DevCounters *pc, int only,
                                                               unsigned int *__restrict__ short_sums) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    unsigned int items = 0;
    unsigned long long r_short = 0, r_med = 0, r_long = 0, n_short = 0, n_med = 0, n_long = 0;
    for (int q = 0; q < SCAN_ITEMS; ++q) {
        unsigned int len;
        const unsigned int cnt = row_item_count(rowptr, owner, base + q, M, ts, seg, &len, only);
        items += cnt;
        if (len == 0) continue;
        if (cnt == 0) { ++r_short; n_short += len; }
        else if (cnt == 1) { ++r_med; n_med += len; }
        else { ++r_long; n_long += len; }
    }
    unsigned int total;
    (void)block_exclusive_scan(items, &total);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
    // statistics: wave sums, then one set of atomics per workgroup
    __shared__ unsigned long long sh[6];
    if (threadIdx.x < 6) sh[threadIdx.x] = 0;
    __syncthreads();
    r_short = wave_sum_u64(r_short); r_med = wave_sum_u64(r_med); r_long = wave_sum_u64(r_long);
    n_short = wave_sum_u64(n_short); n_med = wave_sum_u64(n_med); n_long = wave_sum_u64(n_long);
    if (lane_id() == 0) {
        if (r_short) atomicAdd(&sh[0], r_short);
        if (r_med) atomicAdd(&sh[1], r_med);
        if (r_long) atomicAdd(&sh[2], r_long);
        if (n_short) atomicAdd(&sh[3], n_short);
        if (n_med) atomicAdd(&sh[4], n_med);
        if (n_long) atomicAdd(&sh[5], n_long);
    }
    __syncthreads();
    if (threadIdx.x < 6) spread_add(pc, K_ROWS_SHORT + (int)threadIdx.x, sh[threadIdx.x]);
    // entries of this block's short rows, for the entry list (k_short_list_write)
    if (short_sums && threadIdx.x == 0) short_sums[blockIdx.x] = (unsigned int)sh[3];
}

// pass 2: exclusive scan of the block sums in place (one workgroup), total -> *total_out
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_block_sums(unsigned int *__restrict__ block_sums, int n,
                                                                unsigned long long *__restrict__ total_out) {
    unsigned int carry = 0;
    for (int base = 0; base < n; base += SCAN_BLOCK) {
        const int i = base + (int)threadIdx.x;
        const unsigned int v = i < n ? block_sums[i] : 0u;
        unsigned int total;
        const unsigned int ex = block_exclusive_scan(v, &total);
        if (i < n) block_sums[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) *total_out = carry;
}

// the whole exclusive scan of a short array in one workgroup (one launch instead of three)
constexpr int SCAN_SMALL_ITEMS = 8;
constexpr int SCAN_SMALL_MAX = 16384;
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_small(const unsigned int *__restrict__ in, int n,
                                                           unsigned int *__restrict__ out,
                                                           unsigned long long *__restrict__ total_out) {
    unsigned int carry = 0;
    for (int base = 0; base < n; base += SCAN_BLOCK * SCAN_SMALL_ITEMS) {
        const int i0 = base + (int)threadIdx.x * SCAN_SMALL_ITEMS;
        unsigned int v[SCAN_SMALL_ITEMS], mine = 0;
#pragma unroll
        for (int q = 0; q < SCAN_SMALL_ITEMS; ++q) {
            v[q] = i0 + q < n ? in[i0 + q] : 0u;
            mine += v[q];
        }
        unsigned int total;
        unsigned int at = carry + block_exclusive_scan(mine, &total);
#pragma unroll
        for (int q = 0; q < SCAN_SMALL_ITEMS; ++q) {
            if (i0 + q < n) out[i0 + q] = at;
            at += v[q];
        }
        carry += total;
    }
    if (threadIdx.x == 0) *total_out = carry;
}

// Several short scans in one launch: workgroup j takes job j (in == out is allowed: a thread
// writes only the positions it has read).
constexpr int SCAN_JOBS_MAX = 8;
struct ScanJob {
    const unsigned int *in;
    unsigned int *out;
    unsigned long long *total;
    int n;
    int pad;
};
struct ScanJobs { ScanJob job[SCAN_JOBS_MAX]; };
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_jobs(ScanJobs jobs) {
    const ScanJob jb = jobs.job[blockIdx.x];
    unsigned int carry = 0;
    for (int base = 0; base < jb.n; base += SCAN_BLOCK * SCAN_SMALL_ITEMS) {
        const int i0 = base + (int)threadIdx.x * SCAN_SMALL_ITEMS;
        unsigned int v[SCAN_SMALL_ITEMS], mine = 0;
#pragma unroll
        for (int q = 0; q < SCAN_SMALL_ITEMS; ++q) {
            v[q] = i0 + q < jb.n ? jb.in[i0 + q] : 0u;
            mine += v[q];
        }
        unsigned int total;
        unsigned int at = carry + block_exclusive_scan(mine, &total);
#pragma unroll
        for (int q = 0; q < SCAN_SMALL_ITEMS; ++q) {
            if (i0 + q < jb.n) jb.out[i0 + q] = at;
            at += v[q];
        }
        carry += total;
    }
    if (threadIdx.x == 0) *jb.total = carry;
}

// The entry list of the short rows: {position, row} of every stored entry of the rows that
// have fewer than ts entries and no owner, in storage order.  The kernels take it 64 entries
// per wavefront, whatever the lengths of the rows (block_offsets: exclusive scan of the
// short_sums of k_classify_count).
__global__ __launch_bounds__(SCAN_BLOCK) void k_short_list_write(const int32_t *__restrict__ rowptr,
                                                                 const unsigned char *__restrict__ owner, int M,
                                                                 int ts, const unsigned int *__restrict__ block_offsets,
                                                                 int2 *__restrict__ list) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    unsigned int len[SCAN_ITEMS], mine = 0;
    for (int q = 0; q < SCAN_ITEMS; ++q) {
        const int64_t i = base + q;
        unsigned int l = 0;
        if (i < M && !(owner && owner[i] != 0)) {
            l = (unsigned int)(rowptr[i + 1] - rowptr[i]);
            if (l >= (unsigned int)ts) l = 0;
        }
        len[q] = l;
        mine += l;
    }
    unsigned int total;
    unsigned int at = block_offsets[blockIdx.x] + block_exclusive_scan(mine, &total);
    for (int q = 0; q < SCAN_ITEMS; ++q) {
        if (len[q] == 0) continue;
        const int32_t row = (int32_t)(base + q);
        const int32_t rs = rowptr[row];
        for (unsigned int e = 0; e < len[q]; ++e) list[at++] = make_int2(rs + (int32_t)e, row);
    }
}

// pass 3: write the items
__global__ __launch_bounds__(SCAN_BLOCK) void k_classify_write(const int32_t *__restrict__ rowptr,
                                                               const unsigned char *__restrict__ owner, int M,
                                                               int ts, int seg,
                                                               const unsigned int *__restrict__ block_offsets,
                                                               RowItem *__restrict__ items, int only) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    unsigned int cnt[SCAN_ITEMS], mine = 0;
    for (int q = 0; q < SCAN_ITEMS; ++q) {
        unsigned int len;
        cnt[q] = row_item_count(rowptr, owner, base + q, M, ts, seg, &len, only);
        mine += cnt[q];
    }
    unsigned int total;
    unsigned int at = block_offsets[blockIdx.x] + block_exclusive_scan(mine, &total);
    for (int q = 0; q < SCAN_ITEMS; ++q) {
        if (cnt[q] == 0) continue;
        const int32_t row = (int32_t)(base + q);
        const int32_t s = rowptr[row], e = rowptr[row + 1];
        for (unsigned int k = 0; k < cnt[q]; ++k) {
            const int32_t a = s + (int32_t)k * seg;
            const int32_t b = a + seg < e ? a + seg : e;
            items[at++] = RowItem{row, a, b, 0};
        }
    }
}

// ---------------------------------------------------------------------------
// Row-panel detector: panel p = rows [8p, 8p+8).  It qualifies when all 8 rows
// exist, are not owned by the dense-tile path, have the same length >= min_len and
// the same column list.  One wavefront per panel; lanes stride over the list.
// counts[p] = work items of the panel (ceil(len/pseg)) or 0; owner = 2 on its rows when taken.
__global__ __launch_bounds__(256) void k_panel_flags(const int32_t *__restrict__ rowptr,
                                                     const int32_t *__restrict__ col, int M, int64_t n_panels,
                                                     int min_len, int pseg, unsigned char *__restrict__ owner,
                                                     unsigned int *__restrict__ counts, DevCounters *pc) {
    const int64_t p = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (p >= n_panels) return;
    const int lane = lane_id();
    const int64_t row0 = p * 8;
    bool ok = row0 + 8 <= M && owner[row0] == 0;   // strips own aligned groups of 16 rows
    int s0 = 0, len = 0;
    if (ok) {
        s0 = rowptr[row0];
        len = rowptr[row0 + 1] - s0;
        ok = len >= min_len;
        for (int r = 1; ok && r < 8; ++r) ok = rowptr[row0 + r + 1] - rowptr[row0 + r] == len;
    }
    // ok is the same in every lane here.  Equal lengths make the 8 rows equally spaced
    // in the CSR arrays (row r starts at s0 + r*len), so the 7 comparisons of one
    // position are independent loads.
    if (ok) {
        bool differ = false;
        for (int e = lane; e < len; e += WAVE) {
            const int32_t *pc0 = col + s0 + e;
            const int c0 = pc0[0];
            int d = 0;
#pragma unroll
            for (int r = 1; r < 8; ++r) d |= pc0[(int64_t)r * len] ^ c0;
            differ |= d != 0;
        }
        ok = __ballot(differ) == 0;
    }
    if (ok && lane < 8) owner[row0 + lane] = 2;
    if (lane == 0) {
        counts[p] = ok ? (unsigned int)((len + pseg - 1) / pseg) : 0u;
        if (ok) {
            spread_add(pc, K_PANELS, 1ull);
            spread_add(pc, K_NNZ_PANELS, (unsigned long long)len * 8ull);
        }
    }
}

// items of the taken panels: {first row, [start,end) inside the shared list}
__global__ __launch_bounds__(256) void k_panel_items(const int32_t *__restrict__ rowptr, int64_t n_panels, int pseg,
                                                     const unsigned int *__restrict__ counts,
                                                     const unsigned int *__restrict__ offsets,
                                                     RowItem *__restrict__ items) {
    const int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= n_panels) return;
    const unsigned int n = counts[p];
    if (n == 0) return;
    const int32_t row0 = (int32_t)(p * 8);
    const int32_t rs0 = rowptr[row0];
    const int32_t len = rowptr[row0 + 1] - rs0;
    unsigned int at = offsets[p];
    for (unsigned int k = 0; k < n; ++k) {
        const int32_t a = (int32_t)k * pseg;
        const int32_t b = a + pseg < len ? a + pseg : len;
        // pad carries the CSR position of the panel's first row: the 8 rows have the same
        // length and follow each other, so row r starts at pad + r*len and a kernel can
        // start reading the column list without first waiting for a row pointer
        items[at++] = RowItem{row0, a, b, rs0};
    }
}

}  // namespace sddmm
