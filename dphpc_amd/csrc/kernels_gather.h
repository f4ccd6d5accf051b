// Gather kernels: every stored entry (i,j) of S reads row i of A and row j of B.
//
// Lane layout (all kernels below).  A wavefront works on a "chunk" of up to 64
// consecutive stored entries.  Lane l loads the column index / S value of entry
// l of the chunk and finally stores its P value: plain coalesced 64-wide
// accesses.  For the dot products the 64 lanes are cut into G = 64/LPN groups of
// LPN lanes.  A row of K elements is KU units of 16 bytes; lane j of a group owns
// units j, j+LPN, j+2*LPN, ... (UPL of them), so every load instruction has LPN
// neighbouring lanes reading LPN*16 contiguous bytes of one row: at K=32 fp32,
// LPN=8 and UPL=1, 8 lanes read one whole 128-byte B row (one cache line) per
// instruction; at K=128, LPN=8 and UPL=4, four instructions read four lines.
// In step t group g computes entry t*G+g, i.e. a step covers G
// consecutive entries and a chunk of n entries needs ceil(n/G) steps (a short
// chunk costs proportionally less).  Steps are issued in batches: all gathers of
// a batch are in flight before the first FMA.  Lane (g*LPN+t) keeps the group
// total of step t; one permute at the end brings entry l back to lane l.
//
// Per-entry arithmetic depends on K only (FMA chain over the lane's units in k
// order, then the fixed tree of group_sum), so all strategies built from these
// kernels return bit-identical values.
#pragma once
#include "device_utils.h"

namespace sddmm {

constexpr int BLOCK = 256;                 // 4 wavefronts
constexpr int WAVES_PER_BLOCK = BLOCK / WAVE;

// Byte offset of a row: 32-bit when the whole operand is below 4 GiB (one VALU
// multiply, scalar base + 32-bit vector offset addressing), 64-bit otherwise.
template <bool WIDE> struct Off;
template <> struct Off<false> { using T = uint32_t; };
template <> struct Off<true> { using T = uint64_t; };

template <class T, class O>
__device__ __forceinline__ T load_at(const void *__restrict__ base, O byte_off) {
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(base) + byte_off);
}

template <class O>
__device__ __forceinline__ O shfl_off(O v, int src) {
    if constexpr (sizeof(O) == 4) return (O)__shfl((int)v, src, WAVE);
    else {
        const uint32_t lo = (uint32_t)__shfl((int)(uint32_t)v, src, WAVE);
        const uint32_t hi = (uint32_t)__shfl((int)(uint32_t)(v >> 32), src, WAVE);
        return ((uint64_t)hi << 32) | lo;
    }
}

// Dot products of up to 64 entries, one unit-set per lane.
//   U, LPN, UPL  unit type, lanes per entry, units per lane (KU <= LPN*UPL)
//   FULLK        KU == LPN*UPL: no lane is idle, no unit is masked
//   WITH_ROWS    true: the A row differs per entry; false: `a` already holds the
//                lane's units of the one A row
//   WIDE         64-bit byte offsets
template <class U, int LPN, int UPL, bool FULLK, bool WITH_ROWS, bool WIDE>
struct Chunk {
    using T = typename U::T;
    using O = typename Off<WIDE>::T;
    static constexpr int G = WAVE / LPN;
    // gathers in flight per batch: about 8 x 16 bytes per lane (twice that with A)
    static constexpr int NB_ = 8 / UPL < 1 ? 1 : 8 / UPL;
    static constexpr int BIG = NB_ < LPN ? NB_ : LPN;
    static constexpr int SMALL = 1;

    struct Areg { T u[UPL]; };

    static __device__ __forceinline__ bool unit_on(int j, int i, int KU) { return FULLK || (j + i * LPN) < KU; }

    static __device__ __forceinline__ Areg load_a(const void *__restrict__ A, O row_off, int j, int KU) {
        Areg a;
#pragma unroll
        for (int i = 0; i < UPL; ++i) {
            const int u = unit_on(j, i, KU) ? j + i * LPN : 0;
            a.u[i] = load_at<T, O>(A, row_off + (O)(u * (int)sizeof(T)));
        }
        return a;
    }

    template <int NB, class Hook>
    static __device__ __forceinline__ void batch(int t0, const void *__restrict__ A, const void *__restrict__ B,
                                                 int KU, const Areg &a, O boff, O aoff, int lane, float &out,
                                                 Hook &&after_issue) {
        const int g = lane / LPN, j = lane & (LPN - 1);
        T bf[NB][UPL];
        T af[WITH_ROWS ? NB : 1][UPL];
#pragma unroll
        for (int s = 0; s < NB; ++s) {
            const int src = ((t0 + s) * G + g) & (WAVE - 1);
            const O bo = shfl_off<O>(boff, src);
            O ao = 0;
            if constexpr (WITH_ROWS) ao = shfl_off<O>(aoff, src);
#pragma unroll
            for (int i = 0; i < UPL; ++i) {
                const int u = unit_on(j, i, KU) ? j + i * LPN : 0;
                bf[s][i] = load_at<T, O>(B, bo + (O)(u * (int)sizeof(T)));
                if constexpr (WITH_ROWS) af[s][i] = load_at<T, O>(A, ao + (O)(u * (int)sizeof(T)));
            }
        }
        after_issue();
#pragma unroll
        for (int s = 0; s < NB; ++s) {
            float p = 0.f;
#pragma unroll
            for (int i = 0; i < UPL; ++i) {
                float q;
                if constexpr (WITH_ROWS) q = U::dot(af[s][i], bf[s][i], p);
                else q = U::dot(a.u[i], bf[s][i], p);
                p = unit_on(j, i, KU) ? q : p;
            }
            p = group_sum<LPN>(p);
            if (j == t0 + s) out = p;
        }
    }

    // boff / aoff: byte offset of this lane's entry's B row / A row (a valid row in
    // every lane, row 0 past the end of the chunk); count = entries in the chunk.
    // `prefetch` is called once, right after the first gathers have been issued:
    // the place to start the index loads of the next chunk, so that they travel
    // while this chunk computes (loads return in issue order, so anything issued
    // before the gathers would have to land before them).
    template <class Hook>
    static __device__ __forceinline__ float run(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                const Areg &a, O boff, O aoff, int count, int lane,
                                                Hook &&prefetch) {
        int steps = (count + G - 1) / G;
        steps = steps < LPN ? steps : LPN;
        float out = 0.f;
        int t0 = 0;
        bool fired = false;
        auto once = [&]() { if (!fired) { prefetch(); fired = true; } };
        for (; t0 + BIG <= steps; t0 += BIG) batch<BIG>(t0, A, B, KU, a, boff, aoff, lane, out, once);
        if constexpr (BIG > 1)
            for (; t0 < steps; t0 += SMALL) batch<SMALL>(t0, A, B, KU, a, boff, aoff, lane, out, once);
        once();
        // entry l = t*G+g was kept by lane g*LPN+t
        return __shfl(out, (lane % G) * LPN + lane / G, WAVE);
    }
};

// K too long for the register layout (more than 64 units per row): one entry per
// step, all 64 lanes stride over the row.
template <class U>
__device__ __forceinline__ float chunk_long(const typename U::T *__restrict__ A,
                                            const typename U::T *__restrict__ B, int KU, int c, int r,
                                            int count, int lane) {
    float out = 0.f;
    for (int t = 0; t < count; ++t) {
        const int cc = __shfl(c, t, WAVE);
        const int rr = __shfl(r, t, WAVE);
        const typename U::T *__restrict__ Ar = A + (int64_t)rr * KU;
        const typename U::T *__restrict__ Br = B + (int64_t)cc * KU;
        float p = 0.f;
        for (int u = lane; u < KU; u += WAVE) p = U::dot(Ar[u], Br[u], p);
        p = group_sum<WAVE>(p);
        if (lane == t) out = p;
    }
    return out;
}

// Compile-time description of one (K, dtype) family.  LPN == 0 selects chunk_long.
template <class U_, int LPN_, int UPL_, bool FULLK_, bool WIDE_>
struct Layout {
    using U = U_;
    static constexpr int LPN = LPN_, UPL = UPL_;
    static constexpr bool FULLK = FULLK_, WIDE = WIDE_, LONG = (LPN_ == 0);
};

// ---------------------------------------------------------------------------
// FLAT: entries [0,nnz) in order, row index per entry read from rowidx (the COO
// row array, or the expansion of rowptr built by the plan).  Perfectly balanced
// whatever the row lengths are; A units are gathered per entry like B units
// (L1/L2 hits while the row does not change).
template <class L>
__global__ __launch_bounds__(BLOCK) void k_flat(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                const int32_t *__restrict__ rowidx,
                                                const int32_t *__restrict__ col,
                                                const float *__restrict__ sval,
                                                float *__restrict__ P, int64_t nnz,
                                                int chunks_per_wave, int64_t nblocks) {
    using U = typename L::U;
    using T = typename U::T;
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int lane = lane_id();
    const int64_t wave = blk * WAVES_PER_BLOCK + wave_in_block();
    int64_t base = wave * (int64_t)chunks_per_wave * WAVE;
    if (base >= nnz) return;
    int64_t stop = base + (int64_t)chunks_per_wave * WAVE;
    stop = stop < nnz ? stop : nnz;
    // Index loads are unconditional (clamped to the last entry of the range): lanes
    // past the end then hold a valid row/column whose result is never stored, and
    // the loads need no branch, which keeps the wait counts of the gathers exact.
    const int64_t last = stop - 1;
    const int64_t n0 = base + lane < last ? base + lane : last;
    int c = ld_stream(col + n0), r = ld_stream(rowidx + n0);
    float s = ld_stream(sval + n0);
    for (; base < stop; base += WAVE) {
        const int64_t n = base + lane;
        const bool valid = n < stop;
        const int64_t left = stop - base;
        const int count = left < WAVE ? (int)left : WAVE;
        int cn = 0, rn = 0;
        float sn = 0.f;
        auto prefetch = [&]() {
            const int64_t pn = n + WAVE < last ? n + WAVE : last;
            cn = ld_stream(col + pn); rn = ld_stream(rowidx + pn); sn = ld_stream(sval + pn);
        };
        float res;
        if constexpr (L::LONG) {
            prefetch();
            res = chunk_long<U>((const T *)A, (const T *)B, KU, c, r, count, lane);
        } else {
            using C = Chunk<U, L::LPN, L::UPL, L::FULLK, true, L::WIDE>;
            using O = typename C::O;
            const O rb = (O)KU * (O)sizeof(T);
            typename C::Areg none;
            res = C::run(A, B, KU, none, (O)c * rb, (O)r * rb, count, lane, prefetch);
        }
        if (valid) st_stream(P + n, res * s);
        c = cn; r = rn; s = sn;
    }
}

// ---------------------------------------------------------------------------
// Bodies shared by the stand-alone kernels and the fused AUTO kernel.

// One wavefront, one work item = entries [start,end) of `row`.  The lane's units
// of the A row stay in registers for the whole segment; no row index is read.
template <class L>
__device__ __forceinline__ void row_segment_body(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                 const int32_t *__restrict__ col, const float *__restrict__ sval,
                                                 float *__restrict__ P, int row, int start, int end, int lane) {
    using U = typename L::U;
    using T = typename U::T;
    if (start >= end) return;
    if constexpr (L::LONG) {
        for (int base = start; base < end; base += WAVE) {
            const int n = base + lane;
            const bool valid = n < end;
            const int c = valid ? ld_stream(col + n) : 0;
            const float s = valid ? ld_stream(sval + n) : 0.f;
            const int left = end - base;
            const float res = chunk_long<U>((const T *)A, (const T *)B, KU, c, row, left < WAVE ? left : WAVE, lane);
            if (valid) st_stream(P + n, res * s);
        }
    } else {
        using C = Chunk<U, L::LPN, L::UPL, L::FULLK, false, L::WIDE>;
        using O = typename C::O;
        const O rb = (O)KU * (O)sizeof(T);
        const typename C::Areg a = C::load_a(A, (O)row * rb, lane & (L::LPN - 1), KU);
        // Index loads are unconditional (clamped to the last entry of the range): lanes
        // past the end then hold a valid column whose result is never stored, and the
        // loads need no branch, which keeps the wait counts of the gathers exact.
        const int last = end - 1;
        const int n0 = start + lane < last ? start + lane : last;
        int c = ld_stream(col + n0);
        float s = ld_stream(sval + n0);
        for (int base = start; base < end; base += WAVE) {
            const int n = base + lane;
            const bool valid = n < end;
            const int left = end - base;
            int cn = 0;
            float sn = 0.f;
            auto prefetch = [&]() {
                const int pn = n + WAVE < last ? n + WAVE : last;
                cn = ld_stream(col + pn); sn = ld_stream(sval + pn);
            };
            const float res = C::run(A, B, KU, a, (O)c * rb, (O)0, left < WAVE ? left : WAVE, lane, prefetch);
            if (valid) st_stream(P + n, res * s);
            c = cn; s = sn;
        }
    }
}

// One wavefront, `rpw` consecutive rows starting at r0 (rpw <= 64); only rows with
// fewer than `ts` entries are computed (the others belong to the segment items).
// The entries of the short rows are numbered consecutively across the rows, so
// the lanes stay full whatever the individual lengths are; the row of an entry is
// found by bisection over the wave's inclusive prefix sums (registers only), one
// chunk ahead, so that the index loads of chunk i+1 travel while chunk i computes.
template <class L>
__device__ __forceinline__ void short_rows_body(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                const int32_t *__restrict__ rowptr,
                                                const unsigned char *__restrict__ owner,
                                                const int32_t *__restrict__ col, const float *__restrict__ sval,
                                                float *__restrict__ P, int M, int ts, int64_t r0, int rpw, int lane) {
    using U = typename L::U;
    using T = typename U::T;
    int rs = 0, len = 0;
    if (lane < rpw && r0 + lane < M) {
        rs = rowptr[r0 + lane];
        len = rowptr[r0 + lane + 1] - rs;
        if (len >= ts) len = 0;
        // rows computed by the dense-tile or the row-panel path
        if (owner && owner[r0 + lane] != 0) len = 0;
    }
    int incl = len;
    for (int o = 1; o < WAVE; o <<= 1) {
        const int up = __shfl_up(incl, o, WAVE);
        if (lane >= o) incl += up;
    }
    const int total = __builtin_amdgcn_readfirstlane(__shfl(incl, WAVE - 1, WAVE));
    if (total == 0) return;
    const int excl = incl - len;
    // entry index and row of virtual entry v (clamped to the last one)
    auto locate = [&](int v, int &n, int &row) {
        v = v < total ? v : total - 1;
        int lo = 0;
#pragma unroll
        for (int step = WAVE / 2; step > 0; step >>= 1) {
            const int probe = __shfl(incl, lo + step - 1, WAVE);
            if (probe <= v) lo += step;
        }
        n = __shfl(rs, lo, WAVE) + (v - __shfl(excl, lo, WAVE));
        row = (int)r0 + lo;
    };
    int n, row;
    locate(lane, n, row);
    int c = ld_stream(col + n);
    float s = ld_stream(sval + n);
    for (int base = 0; base < total; base += WAVE) {
        const bool valid = base + lane < total;
        const int left = total - base;
        const int count = left < WAVE ? left : WAVE;
        int nn = n, rown = row, cn = 0;
        float sn = 0.f;
        auto prefetch = [&]() {
            locate(base + WAVE + lane, nn, rown);
            cn = ld_stream(col + nn); sn = ld_stream(sval + nn);
        };
        float res;
        if constexpr (L::LONG) {
            prefetch();
            res = chunk_long<U>((const T *)A, (const T *)B, KU, c, row, count, lane);
        } else {
            using C = Chunk<U, L::LPN, L::UPL, L::FULLK, true, L::WIDE>;
            using O = typename C::O;
            const O rb = (O)KU * (O)sizeof(T);
            typename C::Areg none;
            res = C::run(A, B, KU, none, (O)c * rb, (O)row * rb, count, lane, prefetch);
        }
        if (valid) st_stream(P + n, res * s);
        n = nn; row = rown; c = cn; s = sn;
    }
}

// One wavefront, entries [64 chunk, 64 chunk + 64) of the plan's entry list of the short rows
// ({position, row} per entry, k_short_list_write): the flat kernel's body on a subset of the
// entries.  Three dependent round trips (list, index and S value, gathers) and full lanes
// whatever the row lengths; short_rows_body pays two round trips and a dozen lane exchanges
// before its first index load and one more round trip per chunk.
template <class L>
__device__ __forceinline__ void entry_list_body(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                const int2 *__restrict__ list, int64_t n_list,
                                                const int32_t *__restrict__ col, const float *__restrict__ sval,
                                                float *__restrict__ P, int64_t chunk, int lane) {
    using U = typename L::U;
    using T = typename U::T;
    const int64_t base = chunk * WAVE;
    if (base >= n_list) return;
    const int64_t left = n_list - base;
    const int count = left < WAVE ? (int)left : WAVE;
    const bool valid = lane < count;
    const int2 pr = list[base + (valid ? lane : count - 1)];   // lanes past the end repeat the last entry
    const int c = ld_stream(col + pr.x);
    const float s = ld_stream(sval + pr.x);
    float res;
    if constexpr (L::LONG) {
        res = chunk_long<U>((const T *)A, (const T *)B, KU, c, pr.y, count, lane);
    } else {
        using C = Chunk<U, L::LPN, L::UPL, L::FULLK, true, L::WIDE>;
        using O = typename C::O;
        const O rb = (O)KU * (O)sizeof(T);
        typename C::Areg none;
        res = C::run(A, B, KU, none, (O)c * rb, (O)pr.y * rb, count, lane, []() {});
    }
    if (valid) st_stream(P + pr.x, res * s);
}

// ---------------------------------------------------------------------------
// ROW_WAVE: one wavefront per work item.  With items == nullptr item w is the
// whole row w.
template <class L>
__global__ __launch_bounds__(BLOCK) void k_row_wave(const void *__restrict__ A, const void *__restrict__ B,
                                                    int KU, const int32_t *__restrict__ rowptr,
                                                    const int32_t *__restrict__ col,
                                                    const float *__restrict__ sval,
                                                    float *__restrict__ P,
                                                    const RowItem *__restrict__ items,
                                                    int64_t n_items, int64_t nblocks) {
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t w = blk * WAVES_PER_BLOCK + wave_in_block();
    if (w >= n_items) return;
    int row, start, end;
    if (items) {
        const RowItem it = items[w];
        row = it.row; start = it.start; end = it.end;
    } else {
        row = (int)w; start = rowptr[w]; end = rowptr[w + 1];
    }
    // the same in every lane: keep them in scalar registers
    row = __builtin_amdgcn_readfirstlane(row);
    start = __builtin_amdgcn_readfirstlane(start);
    end = __builtin_amdgcn_readfirstlane(end);
    row_segment_body<L>(A, B, KU, col, sval, P, row, start, end, lane_id());
}

// ---------------------------------------------------------------------------
// SHORT_ROWS as a strategy of its own: every row counts as short (ts = INT_MAX).
template <class L>
__global__ __launch_bounds__(BLOCK) void k_short_rows(const void *__restrict__ A, const void *__restrict__ B,
                                                      int KU, const int32_t *__restrict__ rowptr,
                                                      const int32_t *__restrict__ col,
                                                      const float *__restrict__ sval,
                                                      float *__restrict__ P, int M, int ts, int rpw,
                                                      int64_t nblocks) {
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t r0 = (blk * WAVES_PER_BLOCK + wave_in_block()) * rpw;
    if (r0 >= M) return;
    short_rows_body<L>(A, B, KU, rowptr, nullptr, col, sval, P, M, ts, r0, rpw, lane_id());
}

// ---------------------------------------------------------------------------
// AUTO: one launch for both row classes.  Logical blocks [0, short_blocks) run the
// many-rows-per-wave body over all rows (skipping the rows that have items), the
// blocks after them run one segment item per wavefront.  The item blocks come
// last in the XCD-contiguous order, after the short-row work of the same XCD.
template <class L>
__global__ __launch_bounds__(BLOCK) void k_auto(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                const int32_t *__restrict__ rowptr,
                                                const unsigned char *__restrict__ owner,
                                                const int32_t *__restrict__ col,
                                                const float *__restrict__ sval, float *__restrict__ P, int M,
                                                int ts, int rpw, int64_t short_blocks,
                                                const RowItem *__restrict__ items, int64_t n_items,
                                                int64_t nblocks, const int2 *__restrict__ short_list,
                                                int64_t n_short_list) {
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    // interleave: the item blocks of a long-row-heavy matrix start early instead
    // of forming a tail; block b is an item block when b*item_blocks/nblocks steps
    const int64_t item_blocks = nblocks - short_blocks;
    const int64_t items_before = blk * item_blocks / nblocks;
    const bool is_item = ((blk + 1) * item_blocks / nblocks) != items_before;
    if (is_item) {
        const int64_t w = items_before * WAVES_PER_BLOCK + wave_in_block();
        if (w >= n_items) return;
        const RowItem it = items[w];
        const int row = __builtin_amdgcn_readfirstlane(it.row);
        const int start = __builtin_amdgcn_readfirstlane(it.start);
        const int end = __builtin_amdgcn_readfirstlane(it.end);
        row_segment_body<L>(A, B, KU, col, sval, P, row, start, end, lane_id());
    } else {
        const int64_t sb = blk - items_before;
        if (short_list) {
            entry_list_body<L>(A, B, KU, short_list, n_short_list, col, sval, P, sb * WAVES_PER_BLOCK + wave_in_block(),
                               lane_id());
            return;
        }
        const int64_t r0 = (sb * WAVES_PER_BLOCK + wave_in_block()) * rpw;
        if (r0 >= M) return;
        short_rows_body<L>(A, B, KU, rowptr, owner, col, sval, P, M, ts, r0, rpw, lane_id());
    }
}

// ---------------------------------------------------------------------------
// ROW PANEL: 8 consecutive rows with the same column list (the 8 rows of a dense
// 8x8-block row of a finite-element matrix, the halves of a 16-row dense tile
// strip).  One wavefront per work item = entries [start,end) of the shared list.
// The column indices are read once for the 8 rows and every gathered B unit is
// multiplied with the units of all 8 A rows, which stay in registers: one eighth
// of the gather traffic of the per-row kernels.  Lane (g, j) computes, in step t,
// column t*8+g of the chunk for all 8 rows and keeps row j's total, so S values
// and P are accessed as 8 runs of 8 consecutive floats per instruction.
// Needs the 8-lanes-per-entry layout with no masked unit (K*elem a multiple of 128).
constexpr int PANEL_ROWS = 8;
// Register budget: forcing more than 2 workgroups per CU makes the compiler spill
// the A rows (measured 3x slower on MI355X), so the kernel runs at 2 waves per
// SIMD and hides latency with its own software pipeline instead.
#ifndef SDDMM_PANEL_OCC
#define SDDMM_PANEL_OCC 2
#endif

template <class L>
__global__ __launch_bounds__(BLOCK, SDDMM_PANEL_OCC) void k_panel(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                 const int32_t *__restrict__ rowptr,
                                                 const int32_t *__restrict__ col,
                                                 const float *__restrict__ sval, float *__restrict__ P,
                                                 const RowItem *__restrict__ items, int64_t n_items,
                                                 int64_t nblocks) {
    using U = typename L::U;
    using T = typename U::T;
    static_assert(L::LPN == 8 && L::FULLK && !L::LONG, "row panels use the 8-lane full-K layout");
    constexpr int UPL = L::UPL;
    using O = typename Off<L::WIDE>::T;
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t w = blk * WAVES_PER_BLOCK + wave_in_block();
    if (w >= n_items) return;
    const RowItem it = items[w];
    const int row0 = __builtin_amdgcn_readfirstlane(it.row);
    const int start = __builtin_amdgcn_readfirstlane(it.start);
    const int end = __builtin_amdgcn_readfirstlane(it.end);
    if (start >= end) return;
    const int lane = lane_id();
    const int g = lane >> 3, j = lane & 7;
    const O rb = (O)KU * (O)sizeof(T);
    // units of the 8 A rows
    T a[PANEL_ROWS][UPL];
#pragma unroll
    for (int r = 0; r < PANEL_ROWS; ++r)
#pragma unroll
        for (int i = 0; i < UPL; ++i)
            a[r][i] = load_at<T, O>(A, (O)(row0 + r) * rb + (O)((j + i * 8) * (int)sizeof(T)));
    const int rs0 = __builtin_amdgcn_readfirstlane(rowptr[row0]);   // the shared column list
    const int rsj = rowptr[row0 + j];                               // this lane's output row
    const int last = end - 1;
    auto col_off = [&](int base) {      // byte offset of the B row of this lane's column
        const int e = base + lane < last ? base + lane : last;
        return (O)col[rs0 + e] * rb;
    };
    auto reduce_step = [&](const T (&bfs)[UPL]) {
        float keep = 0.f;
#pragma unroll
        for (int r = 0; r < PANEL_ROWS; ++r) {
            float p = 0.f;
#pragma unroll
            for (int i = 0; i < UPL; ++i) p = U::dot(a[r][i], bfs[i], p);
            p = group_sum<8>(p);
            keep = j == r ? p : keep;
        }
        return keep;
    };
    if constexpr (UPL == 1) {
        // Three chunks in flight, every load unconditional (clamped) so that the wait
        // counts stay exact: iteration i loads the column indices of chunk i+2, the B
        // units and S values of chunk i+1, and computes chunk i.
        auto gather = [&](O boff, T (&bf)[8][1]) {
#pragma unroll
            for (int t = 0; t < 8; ++t) bf[t][0] = load_at<T, O>(B, shfl_off<O>(boff, t * 8 + g) + (O)(j * (int)sizeof(T)));
        };
        auto load_s = [&](int base, float (&sv)[8]) {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int et = base + t * 8 + g < last ? base + t * 8 + g : last;
                sv[t] = sval[rsj + et];
            }
        };
        T bf_cur[8][1], bf_nxt[8][1];
        float sv_cur[8], sv_nxt[8];
        O boff_nxt = col_off(start + WAVE);
        {
            const O boff0 = col_off(start);
            gather(boff0, bf_cur);
            load_s(start, sv_cur);
        }
        for (int base = start; base < end; base += WAVE) {
            const O boff_nn = col_off(base + 2 * WAVE);
            gather(boff_nxt, bf_nxt);
            load_s(base + WAVE, sv_nxt);
            float out[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) out[t] = reduce_step(bf_cur[t]);
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int et = base + t * 8 + g;
                if (et < end) P[rsj + et] = out[t] * sv_cur[t];
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) { bf_cur[t][0] = bf_nxt[t][0]; sv_cur[t] = sv_nxt[t]; }
            boff_nxt = boff_nn;
        }
    } else {
        constexpr int NB = 8 / UPL < 1 ? 1 : 8 / UPL;               // steps per batch of gathers
        O boff = col_off(start);
        for (int base = start; base < end; base += WAVE) {
            const O boff_nxt = col_off(base + WAVE);                // travels while this chunk computes
            float sv[8], out[8];
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int et = base + t * 8 + g < last ? base + t * 8 + g : last;
                sv[t] = sval[rsj + et];
            }
#pragma unroll
            for (int t0 = 0; t0 < 8; t0 += NB) {
                T bf[NB][UPL];
#pragma unroll
                for (int s = 0; s < NB; ++s) {
                    const O bo = shfl_off<O>(boff, (t0 + s) * 8 + g);
#pragma unroll
                    for (int i = 0; i < UPL; ++i) bf[s][i] = load_at<T, O>(B, bo + (O)((j + i * 8) * (int)sizeof(T)));
                }
#pragma unroll
                for (int s = 0; s < NB; ++s) out[t0 + s] = reduce_step(bf[s]);
            }
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const int et = base + t * 8 + g;
                if (et < end) P[rsj + et] = out[t] * sv[t];
            }
            boff = boff_nxt;
        }
    }
}

// ---------------------------------------------------------------------------
// EXACT: one lane per entry, k ascending, separate fp32 multiply and add (the
// translation unit is compiled with -ffp-contract=off), then the multiply by S:
// the operation sequence of the CPU loop, hence bit-identical to it.
template <int DT>
__global__ __launch_bounds__(BLOCK) void k_exact(const void *__restrict__ Av, const void *__restrict__ Bv,
                                                 int K, const int32_t *__restrict__ rowidx,
                                                 const int32_t *__restrict__ col,
                                                 const float *__restrict__ sval,
                                                 float *__restrict__ P, int64_t nnz) {
    const int64_t n = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (n >= nnz) return;
    const int64_t r = rowidx[n], c = col[n];
    float acc = 0.f;
    if constexpr (DT == DT_BF16) {
        const uint16_t *a = (const uint16_t *)Av + r * K;
        const uint16_t *b = (const uint16_t *)Bv + c * K;
        for (int k = 0; k < K; ++k) {
            const float x = __builtin_bit_cast(float, (uint32_t)a[k] << 16);
            const float y = __builtin_bit_cast(float, (uint32_t)b[k] << 16);
            const float prod = x * y;
            acc = acc + prod;
        }
    } else if constexpr (DT == DT_F16) {
        const _Float16 *a = (const _Float16 *)Av + r * K;
        const _Float16 *b = (const _Float16 *)Bv + c * K;
        for (int k = 0; k < K; ++k) {
            const float x = (float)a[k], y = (float)b[k];
            const float prod = x * y;
            acc = acc + prod;
        }
    } else {
        const float *a = (const float *)Av + r * K;
        const float *b = (const float *)Bv + c * K;
        for (int k = 0; k < K; ++k) {
            const float prod = a[k] * b[k];
            acc = acc + prod;
        }
    }
    P[n] = acc * sval[n];
}

}  // namespace sddmm
