// Dense-tile path: 16-row strips of S whose 16x16 tiles are well filled are
// computed on the matrix cores, one MFMA accumulator per tile, instead of one
// gathered B row per stored entry.
//
//   * a strip is rows [16*ti, 16*ti+16); a tile is the strip's entries whose
//     column lies in [16*tj, 16*tj+16);
//   * the classifier (k_strip_count / k_strip_tiles / k_tile_rows, plan phase,
//     device only) finds the non-empty tiles of every strip and emits one TileDesc
//     per tile: for every row the CSR position of its first entry inside the tile
//     and a 16-bit mask of the columns present;
//   * a strip goes to this path as a whole (then every one of its entries is
//     computed here, sparse tiles included) or not at all, so the gather kernels
//     and this one never share a row;
//   * k_tile computes the full 16x16 product A[strip rows] * B[tile cols]^T with
//     fp32 accumulation (bf16 / fp16: v_mfma_f32_16x16x32_bf16 / _f16, fp32: v_mfma_f32_16x16x4_f32,
//     both exact products of the stored inputs), multiplies by the S values and
//     writes only the positions the masks name -- P keeps S's order.
//
// The B tile costs 16 rows per tile whatever its fill, a gathered entry costs one
// row each: the tile path moves fewer bytes once a tile holds more than 16
// entries, and far fewer at the 25-100 % fill it is used for.
#pragma once
#include "device_utils.h"
#include "kernels_gather.h"
#include "kernels_plan.h"

namespace sddmm {

struct alignas(16) TileDesc {
    int32_t strip;      // 16-row strip index
    int32_t tj;         // tile column: columns [16*tj, 16*tj+16)
    int32_t pad[2];
    int32_t off[16];    // per row: CSR position of the row's first entry in the tile
    uint16_t mask[16];  // per row: bit c set <=> column 16*tj+c is stored
};
static_assert(sizeof(TileDesc) == 112, "TileDesc layout");

// ---- 16-lane helpers (a strip is walked by 16 neighbouring lanes) -------------
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
    return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, false);
}
__device__ __forceinline__ int min16(int v) {
    int o;
    o = dpp_i32<DPP_QUAD_XOR1>(v); v = o < v ? o : v;
    o = dpp_i32<DPP_QUAD_XOR2>(v); v = o < v ? o : v;
    o = dpp_i32<DPP_ROW_HALF_MIRROR>(v); v = o < v ? o : v;
    o = dpp_i32<DPP_ROW_MIRROR>(v); v = o < v ? o : v;
    return v;
}
__device__ __forceinline__ int sum16(int v) {
    v += dpp_i32<DPP_QUAD_XOR1>(v);
    v += dpp_i32<DPP_QUAD_XOR2>(v);
    v += dpp_i32<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_i32<DPP_ROW_MIRROR>(v);
    return v;
}

// Walks the tiles of one strip in increasing tile column.  All 16 lanes of the
// strip call on_tile(tj, first, mask) together; `first` / `mask` are this lane's
// row's first position and column mask in the tile (mask 0: row absent).  The walk
// stops early when on_tile returns false (it must return the same in all 16 lanes).
// Returns false in a lane whose row is not strictly increasing in column.
struct __attribute__((packed, aligned(4))) I4u { int x, y, z, w; };
struct __attribute__((packed, aligned(4))) F4u { float x, y, z, w; };

template <class F>
__device__ __forceinline__ bool walk_strip(const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col, int M,
                                           int64_t strip, int sub, F &&on_tile) {
    const int64_t row = strip * 16 + sub;
    int p = 0, end = 0;
    if (row < M) { p = rowptr[row]; end = rowptr[row + 1]; }
    bool sorted = true;
    int prev = -1;
    // The row is read 8 column indices at a time (two 16-byte loads, clamped to the
    // row's last entry), so the walk is not one dependent load per entry.
    int buf[8];
    int buf_at = p;                       // buf[i] = col[min(buf_at + i, end - 1)]
    auto refill = [&](int at) {
        buf_at = at;
        if (at < end) {
            const int last = end - 1;
            if (at + 7 <= last) {
                const I4u lo = *reinterpret_cast<const I4u *>(col + at);
                const I4u hi = *reinterpret_cast<const I4u *>(col + at + 4);
                buf[0] = lo.x; buf[1] = lo.y; buf[2] = lo.z; buf[3] = lo.w;
                buf[4] = hi.x; buf[5] = hi.y; buf[6] = hi.z; buf[7] = hi.w;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) buf[i] = col[at + i < last ? at + i : last];
            }
        }
    };
    auto peek = [&](int at) {             // col[at] for buf_at <= at < buf_at + 8
        const int i = at - buf_at;
        int v = buf[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) v = i == k ? buf[k] : v;
        return v;
    };
    refill(p);
    int c = p < end ? peek(p) : -1;
    while (true) {
        const int mine = p < end ? (c >> 4) : INT32_MAX;
        const int t = min16(mine);
        if (t == INT32_MAX) break;
        const int first = p;
        unsigned int mask = 0;
        while (p < end && (c >> 4) == t) {
            if (c <= prev) sorted = false;
            prev = c;
            mask |= 1u << (c & 15);
            ++p;
            if (p - buf_at >= 8) refill(p);
            c = p < end ? peek(p) : -1;
        }
        if (!on_tile(t, first, mask)) break;
    }
    return sorted;
}

// Every tile lists its 16 B rows (tile_cols, 16 per descriptor, ascending; INT32_MAX
// where a union tile has fewer): consecutive columns for the aligned tiles.
__device__ __forceinline__ void write_aligned_cols(int32_t *__restrict__ tile_cols, int64_t at, int tj) {
    int4 *dst = reinterpret_cast<int4 *>(tile_cols + at * 16);
    const int c0 = tj * 16;
    dst[0] = make_int4(c0, c0 + 1, c0 + 2, c0 + 3);
    dst[1] = make_int4(c0 + 4, c0 + 5, c0 + 6, c0 + 7);
    dst[2] = make_int4(c0 + 8, c0 + 9, c0 + 10, c0 + 11);
    dst[3] = make_int4(c0 + 12, c0 + 13, c0 + 14, c0 + 15);
}

// ---- parallel strip classifier ---------------------------------------------------
// One wavefront per strip, four strips per workgroup.  The strip's entries are
// contiguous in the CSR arrays, so the wave streams them 64 per load, several
// loads in flight, instead of merging 16 sorted lists entry by entry:
//
//   * walking the entries in storage order, the tile column changes at least once
//     per (row, tile) pair minus the 15 row boundaries, and a strip has at least
//     (pairs / 16) tiles: the number of changes bounds the tile count from below
//     without any merging, and the scan stops as soon as that bound exceeds what
//     the fill threshold allows (a strip of scattered entries is given up after
//     its first few hundred);
//   * the same scan marks the tile column after every change in a bitmap in LDS
//     that covers the strip's column span -- every tile present is marked at least
//     once; the number of set bits is the number of tiles, the rank of a bit the
//     position of its tile in the strip's (column-ordered) descriptor range;
//   * rows are strictly increasing iff the only places where a column does not
//     exceed its predecessor are row boundaries: the scan counts all such places,
//     the 16 row starts are checked apart;
//   * a strip whose span does not fit the bitmap is scanned without it and, if it
//     passes, merged by the walk above in its first 16 lanes.
//
// The bitmap is private to its wave: LDS operations of one wave execute in program
// order, so clearing, marking and counting need no workgroup barrier, only that
// the compiler keeps their order (wave_lds_order).
constexpr int STRIP_BM_WORDS = 1024;          // 32768 tile columns: a span of 524288 columns
constexpr int STRIP_UNROLL = 4;               // loads of 256 entries per batch, two batches in flight
constexpr int STRIPS_PER_BLOCK = 4;

__device__ __forceinline__ int wave_sum_i32(int v) {
    for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}

// Streams entries [e0, e1).  Returns the number of tile-column changes, or -1 as
// soon as it exceeds `budget`; *descents receives the number of entries whose
// column does not exceed the column stored before them.  BITS == 1: also sets bit
// (col>>4) - lo in bm after every change (tile columns); BITS == 2: sets bit col - lo
// for every entry (columns).
// A lane takes four consecutive entries per load (16 bytes; the column array is only
// 4-byte aligned at a strip's start, which global loads allow), a load instruction 256
// entries, a batch STRIP_UNROLL of them with the next batch in flight: a strip of 8 000
// entries is eight dependent round trips.
template <int BITS>
__device__ __forceinline__ int64_t strip_scan(const int32_t *__restrict__ col, int e0, int e1, int64_t budget,
                                              int lo, int span, unsigned int *bm, int64_t *descents) {
    const int lane = lane_id();
    constexpr int PER_LOAD = WAVE * 4;
    constexpr int BATCH = PER_LOAD * STRIP_UNROLL;
    int64_t changes = 0, desc = 0;
    int carry = -1;                           // column before the batch; -1: entry e0 counts as a change
    auto load = [&](int base, I4u (&c)[STRIP_UNROLL]) {
#pragma unroll
        for (int u = 0; u < STRIP_UNROLL; ++u) {
            const int b = base + u * PER_LOAD;
            if (b + PER_LOAD <= e1) {                             // wave-uniform: every lane's four entries exist
                c[u] = *reinterpret_cast<const I4u *>(col + b + 4 * lane);
            } else if (b < e1 || u == 0) {                        // the last load of the strip: clamped, entry by entry
                const int last = e1 - 1, i0 = b + 4 * lane;
                c[u].x = col[i0 < last ? i0 : last];
                c[u].y = col[i0 + 1 < last ? i0 + 1 : last];
                c[u].z = col[i0 + 2 < last ? i0 + 2 : last];
                c[u].w = col[i0 + 3 < last ? i0 + 3 : last];
            } else {
                c[u] = I4u{0, 0, 0, 0};
            }
        }
    };
    auto mark = [&](bool on, int column) {
        if constexpr (BITS == 1) {
            const int t = (column >> 4) - lo;
            if (on && (unsigned int)t < (unsigned int)span) atomicOr(&bm[t >> 5], 1u << (t & 31));
        } else if constexpr (BITS == 2) {
            const int t = column - lo;
            if (on && (unsigned int)t < (unsigned int)span) atomicOr(&bm[t >> 5], 1u << (t & 31));
        }
    };
    I4u cur[STRIP_UNROLL], nxt[STRIP_UNROLL];
    load(e0, cur);
    for (int base = e0; base < e1; base += BATCH) {
        load(base + BATCH, nxt);
        int my_changes = 0, my_desc = 0;
#pragma unroll
        for (int u = 0; u < STRIP_UNROLL; ++u) {
            const int cbase = base + u * PER_LOAD;
            if (cbase >= e1) break;                               // wave-uniform
            const int i0 = cbase + 4 * lane;
            const I4u c = cur[u];
            // column of the entry before this lane's first: the last of lane - 1 (wave_shr:1), lane 0 takes the carry
            const int prev = __builtin_amdgcn_update_dpp(carry, c.w, 0x138, 0xF, 0xF, false);
            carry = __builtin_amdgcn_readlane(c.w, WAVE - 1);
            const bool v0 = i0 < e1, v1 = i0 + 1 < e1, v2 = i0 + 2 < e1, v3 = i0 + 3 < e1;
            const bool c0 = v0 && (c.x >> 4) != (prev >> 4), c1 = v1 && (c.y >> 4) != (c.x >> 4);
            const bool c2 = v2 && (c.z >> 4) != (c.y >> 4), c3 = v3 && (c.w >> 4) != (c.z >> 4);
            if constexpr (BITS == 1) { mark(c0, c.x); mark(c1, c.y); mark(c2, c.z); mark(c3, c.w); }
            if constexpr (BITS == 2) { mark(v0, c.x); mark(v1, c.y); mark(v2, c.z); mark(v3, c.w); }
            my_changes += (int)c0 + (int)c1 + (int)c2 + (int)c3;
            my_desc += (int)(v0 && c.x <= prev) + (int)(v1 && c.y <= c.x) + (int)(v2 && c.z <= c.y) + (int)(v3 && c.w <= c.z);
        }
        changes += wave_sum_i32(my_changes);
        desc += wave_sum_i32(my_desc);
        if (changes > budget) return -1;
#pragma unroll
        for (int u = 0; u < STRIP_UNROLL; ++u) cur[u] = nxt[u];
    }
    *descents = desc;
    return changes;
}

// From the first and last entry of each of the 16 rows (lane i < 16: row i, whose
// rowptr is lane_rp): the strip's column span in tile columns (SHIFT 4) or columns
// (SHIFT 0), [lo, lo + span)
// (exact when the rows are sorted; span <= 0 when they are not or no row has an
// entry), and the number of row starts whose column does not exceed the column
// stored before them -- the descents a sorted strip is allowed.
template <int SHIFT = 4>
__device__ __forceinline__ void strip_bounds(const int32_t *__restrict__ col, int lane_rp, int e0, int *lo, int *span,
                                             int *boundary_descents) {
    const int lane = lane_id();
    const int nxt = __shfl_down(lane_rp, 1, WAVE);
    const bool has = lane < 16 && nxt > lane_rp;
    const int first_col = has ? col[lane_rp] : INT32_MAX;
    const int last_col = has ? col[nxt - 1] : -1;
    const int before = has && lane_rp > e0 ? col[lane_rp - 1] : -1;
    const int l = __builtin_amdgcn_readfirstlane(min16(has ? first_col >> SHIFT : INT32_MAX));
    const int hneg = __builtin_amdgcn_readfirstlane(min16(has ? -(last_col >> SHIFT) : 1));
    *lo = l;
    *span = l == INT32_MAX ? 0 : -hneg - l + 1;
    *boundary_descents = __popcll(__ballot(has && first_col <= before));
}

// pass 1: strip_ntiles[s] = number of tiles of a strip that goes to the tile path
// (sorted rows, at least min_fill entries per tile on average), else 0.
__global__ __launch_bounds__(WAVE * STRIPS_PER_BLOCK) void k_strip_count(
    const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col, int M, int64_t n_strips, int min_fill,
    unsigned int *__restrict__ strip_ntiles, unsigned char *__restrict__ owner, DevCounters *pc) {
    __shared__ unsigned int bm_all[STRIPS_PER_BLOCK][STRIP_BM_WORDS];
    const int64_t strip = (int64_t)blockIdx.x * STRIPS_PER_BLOCK + wave_in_block();
    if (strip >= n_strips) return;            // whole waves leave
    unsigned int *bm = bm_all[wave_in_block()];
    const int lane = lane_id();
    const int64_t r = strip * 16 + lane;
    const int lane_rp = rowptr[r < M ? r : M];
    const int e0 = __builtin_amdgcn_readlane(lane_rp, 0), e1 = __builtin_amdgcn_readlane(lane_rp, 16);
    const int64_t entries = (int64_t)e1 - (int64_t)e0;
    const int64_t max_tiles = entries / min_fill;
    // changes >= (row, tile) pairs - 15 and tiles >= pairs / 16
    const int64_t budget = 16 * max_tiles;
    int64_t tiles = 0, descents = 0;
    bool take = false;
    // most strips of a scattered matrix are given up on their first 512 entries,
    // before anything else is read
    constexpr int FIRST = 512;
    if (max_tiles > 0 &&
        strip_scan<0>(col, e0, e1 - e0 > FIRST ? e0 + FIRST : e1, budget, 0, 0, nullptr, &descents) >= 0) {
        int lo, span, allowed;
        strip_bounds(col, lane_rp, e0, &lo, &span, &allowed);
        if (span > STRIP_BM_WORDS * 32) {
            // too wide for the bitmap: scan without it, then merge the 16 rows in the first
            // 16 lanes if the strip is still a candidate
            const int64_t ch = strip_scan<0>(col, e0, e1, budget, 0, 0, nullptr, &descents);
            if (ch >= 0 && descents == allowed) {
                int t = 0;
                if (lane < 16) {
                    (void)walk_strip(rowptr, col, M, strip, lane, [&](int, int, unsigned int) {
                        ++t;
                        return (int64_t)t <= max_tiles;
                    });
                }
                tiles = __builtin_amdgcn_readfirstlane(t);
            }
        } else if (span > 0) {
            const int words = (span + 31) >> 5;
            for (int w = lane; w < words; w += WAVE) bm[w] = 0u;
            wave_lds_order();
            // Rows 0 and 8 first: their tile columns alone often exceed what the strip may have
            // (two 8-row blocks with different column lists), and the other 14 rows are then
            // never read.  The bits stay: the scan of the whole strip sets them again.
            int64_t ch = 0;
            if (entries > 4 * FIRST) {
                int64_t unused;
                const int a0 = e0, a1 = __builtin_amdgcn_readlane(lane_rp, 1);
                const int b0 = __builtin_amdgcn_readlane(lane_rp, 8), b1 = __builtin_amdgcn_readlane(lane_rp, 9);
                if (a1 > a0) (void)strip_scan<1>(col, a0, a1, INT64_MAX, lo, span, bm, &unused);
                if (b1 > b0) (void)strip_scan<1>(col, b0, b1, INT64_MAX, lo, span, bm, &unused);
                wave_lds_order();
                int t = 0;
                for (int w = lane; w < words; w += WAVE) t += __builtin_popcount(bm[w]);
                if (wave_sum_i32(t) > max_tiles) ch = -1;
            }
            if (ch >= 0) ch = strip_scan<1>(col, e0, e1, budget, lo, span, bm, &descents);
            wave_lds_order();
            if (ch >= 0 && descents == allowed) {
                int t = 0;
                for (int w = lane; w < words; w += WAVE) t += __builtin_popcount(bm[w]);
                tiles = wave_sum_i32(t);
            }
        }
        take = tiles > 0 && tiles <= max_tiles && entries >= (int64_t)min_fill * tiles;
    }
    if (take && lane < 16 && strip * 16 + lane < M) owner[strip * 16 + lane] = 1;
    if (lane == 0) {
        strip_ntiles[strip] = take ? (unsigned int)tiles : 0u;
        if (take) {
            spread_add(pc, K_TILES, (unsigned long long)tiles);
            spread_add(pc, K_NNZ_TILES, (unsigned long long)entries);
        }
    }
}

// pass 2 (after the exclusive scan of strip_ntiles into strip_off): strip and tile
// column of every descriptor, in increasing tile column.  Descriptors of a strip
// that needs the merging walk are written completely here (pad[0] = 1); the others
// get their per-row fields from k_tile_rows.
__global__ __launch_bounds__(WAVE * STRIPS_PER_BLOCK) void k_strip_tiles(
    const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col, int M, int64_t n_strips,
    const unsigned int *__restrict__ strip_ntiles, const unsigned int *__restrict__ strip_off,
    TileDesc *__restrict__ tiles, int32_t *__restrict__ tile_cols) {
    __shared__ unsigned int bm_all[STRIPS_PER_BLOCK][STRIP_BM_WORDS];
    const int64_t strip = (int64_t)blockIdx.x * STRIPS_PER_BLOCK + wave_in_block();
    if (strip >= n_strips) return;
    if (strip_ntiles[strip] == 0) return;
    unsigned int *bm = bm_all[wave_in_block()];
    const int lane = lane_id();
    const int64_t r = strip * 16 + lane;
    const int lane_rp = rowptr[r < M ? r : M];
    const int e0 = __builtin_amdgcn_readlane(lane_rp, 0), e1 = __builtin_amdgcn_readlane(lane_rp, 16);
    int lo, span, allowed;
    strip_bounds(col, lane_rp, e0, &lo, &span, &allowed);
    const int64_t first_desc = strip_off[strip];
    if (span > STRIP_BM_WORDS * 32) {
        if (lane < 16) {
            int64_t at = first_desc;
            (void)walk_strip(rowptr, col, M, strip, lane, [&](int tj, int first, unsigned int mask) {
                TileDesc *d = tiles + at;
                d->off[lane] = first;
                d->mask[lane] = (uint16_t)mask;
                if (lane == 0) { d->strip = (int32_t)strip; d->tj = tj; d->pad[0] = 1; d->pad[1] = 0; }
                tile_cols[at * 16 + lane] = tj * 16 + lane;
                ++at;
                return true;
            });
        }
        return;
    }
    const int words = (span + 31) >> 5;
    for (int w = lane; w < words; w += WAVE) bm[w] = 0u;
    wave_lds_order();
    int64_t descents;
    (void)strip_scan<1>(col, e0, e1, INT64_MAX, lo, span, bm, &descents);
    wave_lds_order();
    int64_t run = first_desc;
    for (int wb = 0; wb < words; wb += WAVE) {
        const int w = wb + lane;
        unsigned int x = w < words ? bm[w] : 0u;
        const int n = __builtin_popcount(x);
        int incl = n;
        for (int o = 1; o < WAVE; o <<= 1) {
            const int up = __shfl_up(incl, o, WAVE);
            if (lane >= o) incl += up;
        }
        int64_t at = run + (incl - n);
        while (x) {
            const int b = __builtin_ctz(x);
            x &= x - 1;
            *reinterpret_cast<int4 *>(tiles + at) = make_int4((int)strip, lo + w * 32 + b, 0, 0);
            write_aligned_cols(tile_cols, at, lo + w * 32 + b);
            ++at;
        }
        run += __builtin_amdgcn_readlane(incl, WAVE - 1);
    }
}

// ---- union strips --------------------------------------------------------------------
// A 16-row strip whose rows are similar but not aligned to 16-column blocks (mesh
// rows that share most of their neighbours) wastes the aligned tiles: its columns are
// spread over many of them.  Here the strip's tiles are cut from the sorted UNION of
// its column lists instead, 16 union columns per tile, so a B row is gathered once
// for the rows of the strip that have it -- the role of the active-column lists of
// src/competitors/gpu/gpu_preprocessing.hpp:57-141.  Same machinery as above with a
// bitmap of columns instead of tile columns: popcount = size of the union, the rank
// of a column gives its tile and its position in the tile.
constexpr int UNION_BM_WORDS = 4096;          // a column span of 131072 per strip

__device__ __forceinline__ int max16(int v) { return -min16(-v); }

__global__ __launch_bounds__(WAVE * STRIPS_PER_BLOCK) void k_union_count(
    const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col, int M, int64_t n_strips, int min_fill,
    unsigned char *__restrict__ owner, unsigned int *__restrict__ ustrip_ntiles, DevCounters *pc) {
    __shared__ unsigned int bm_all[STRIPS_PER_BLOCK][UNION_BM_WORDS];
    const int64_t strip = (int64_t)blockIdx.x * STRIPS_PER_BLOCK + wave_in_block();
    if (strip >= n_strips) return;
    unsigned int *bm = bm_all[wave_in_block()];
    const int lane = lane_id();
    const int64_t r = strip * 16 + lane;
    const int lane_rp = rowptr[r < M ? r : M];
    const int e0 = __builtin_amdgcn_readlane(lane_rp, 0), e1 = __builtin_amdgcn_readlane(lane_rp, 16);
    const int64_t entries = (int64_t)e1 - (int64_t)e0;
    // the strip must be free as a whole, and even its longest row alone must not need
    // more tiles than the threshold allows
    const bool owned = lane < 16 && r < M && owner[r] != 0;
    const int next_rp = __shfl_down(lane_rp, 1, WAVE);          // every lane takes part in the permute
    const int len = lane < 16 ? next_rp - lane_rp : 0;
    const int longest = __builtin_amdgcn_readfirstlane(max16(lane < 16 ? len : 0));
    int64_t tiles = 0;
    bool take = false;
    if (__ballot(owned) == 0ull && entries >= (int64_t)min_fill * ((longest + 15) / 16) && entries >= min_fill) {
        int lo, span, allowed;
        strip_bounds<0>(col, lane_rp, e0, &lo, &span, &allowed);
        if (span > 0 && span <= UNION_BM_WORDS * 32) {
            const int words = (span + 31) >> 5;
            for (int w = lane; w < words; w += WAVE) bm[w] = 0u;
            wave_lds_order();
            int64_t descents = 0;
            (void)strip_scan<2>(col, e0, e1, INT64_MAX, lo, span, bm, &descents);
            wave_lds_order();
            if (descents == allowed) {
                int t = 0;
                for (int w = lane; w < words; w += WAVE) t += __builtin_popcount(bm[w]);
                tiles = (wave_sum_i32(t) + 15) / 16;
                take = tiles > 0 && entries >= (int64_t)min_fill * tiles;
            }
        }
    }
    if (take && lane < 16 && r < M) owner[r] = 4;
    if (lane == 0) {
        ustrip_ntiles[strip] = take ? (unsigned int)tiles : 0u;
        if (take) {
            spread_add(pc, K_UTILES, (unsigned long long)tiles);
            spread_add(pc, K_NNZ_UTILES, (unsigned long long)entries);
        }
    }
}

// descriptors of the union strips: header and the 16 union columns of every tile
__global__ __launch_bounds__(WAVE * STRIPS_PER_BLOCK) void k_union_tiles(
    const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col, int M, int64_t n_strips,
    const unsigned int *__restrict__ ustrip_ntiles, const unsigned int *__restrict__ ustrip_off,
    TileDesc *__restrict__ tiles, int32_t *__restrict__ tile_cols) {
    __shared__ unsigned int bm_all[STRIPS_PER_BLOCK][UNION_BM_WORDS];
    const int64_t strip = (int64_t)blockIdx.x * STRIPS_PER_BLOCK + wave_in_block();
    if (strip >= n_strips) return;
    const unsigned int ntiles = ustrip_ntiles[strip];
    if (ntiles == 0) return;
    unsigned int *bm = bm_all[wave_in_block()];
    const int lane = lane_id();
    const int64_t r = strip * 16 + lane;
    const int lane_rp = rowptr[r < M ? r : M];
    const int e0 = __builtin_amdgcn_readlane(lane_rp, 0), e1 = __builtin_amdgcn_readlane(lane_rp, 16);
    int lo, span, allowed;
    strip_bounds<0>(col, lane_rp, e0, &lo, &span, &allowed);
    const int words = (span + 31) >> 5;
    for (int w = lane; w < words; w += WAVE) bm[w] = 0u;
    wave_lds_order();
    int64_t descents = 0;
    (void)strip_scan<2>(col, e0, e1, INT64_MAX, lo, span, bm, &descents);
    wave_lds_order();
    const int64_t first = ustrip_off[strip];
    int64_t run = 0;                              // union columns before this batch of words
    for (int wb = 0; wb < words; wb += WAVE) {
        const int w = wb + lane;
        unsigned int x = w < words ? bm[w] : 0u;
        const int n = __builtin_popcount(x);
        int incl = n;
        for (int o = 1; o < WAVE; o <<= 1) {
            const int up = __shfl_up(incl, o, WAVE);
            if (lane >= o) incl += up;
        }
        int64_t rank = run + (incl - n);
        while (x) {
            const int b = __builtin_ctz(x);
            x &= x - 1;
            const int c = lo + w * 32 + b;
            const int64_t t = first + (rank >> 4);
            tile_cols[t * 16 + (rank & 15)] = c;
            if ((rank & 15) == 0) *reinterpret_cast<int4 *>(tiles + t) = make_int4((int)strip, c >> 4, 0, 0);
            ++rank;
        }
        run += __builtin_amdgcn_readlane(incl, WAVE - 1);
    }
    // the last tile of the strip may hold fewer than 16 columns
    const int tail = (int)(run & 15);
    if (tail != 0 && lane >= tail && lane < 16) tile_cols[(first + ntiles - 1) * 16 + lane] = INT32_MAX;
}

// ---- gathered strips ---------------------------------------------------------------
// Rows that are dense inside a column window need not be neighbours to share tiles:
// any 16 rows whose windows overlap form a strip for the matrix cores as well as 16
// consecutive ones do.  Candidate rows (not owned yet, at least min_len entries that
// fill a quarter of their column span or more) are sorted by (first column, row) --
// one 64-bit key per row, so the order does not depend on the order of the appends;
// every 16 consecutive rows of that order are one gathered strip, classified with
// the same bitmap and threshold as a natural strip.  TileDesc.strip of such a strip
// is GATHERED_BASE + its index, its rows are listed in a table (16 per strip, -1 for
// a missing row).
constexpr int GATHERED_BASE = 1 << 30;
constexpr int TILE_WINDOW = 4;                  // descriptors per window (what a wavefront of the tile kernels takes)

__global__ __launch_bounds__(256) void k_gather_candidates(const int32_t *__restrict__ rowptr,
                                                           const int32_t *__restrict__ col, int M,
                                                           const unsigned char *__restrict__ owner, int min_len,
                                                           unsigned long long *__restrict__ keys,
                                                           unsigned long long *__restrict__ count) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    bool cand = false;
    int first = 0;
    if (r < M && owner[r] == 0) {
        const int s = rowptr[r], e = rowptr[r + 1];
        if (e - s >= min_len) {
            first = col[s];
            const int64_t span = (int64_t)col[e - 1] - first + 1;
            cand = span > 0 && (int64_t)(e - s) * 4 >= span;
        }
    }
    // one append per wave
    const unsigned long long m = __ballot(cand);
    if (m == 0ull) return;
    const int lane = lane_id();
    unsigned long long base = 0;
    if (lane == 0) base = atomicAdd(count, (unsigned long long)__popcll(m));
    base = ((unsigned long long)(unsigned int)__builtin_amdgcn_readfirstlane((int)(base >> 32)) << 32) |
           (unsigned int)__builtin_amdgcn_readfirstlane((int)base);
    if (cand) {
        const unsigned long long at = base + (unsigned long long)__popcll(m & ((1ull << lane) - 1ull));
        keys[at] = ((unsigned long long)(unsigned int)first << 32) | (unsigned long long)(unsigned int)r;
    }
}

// The candidate keys in increasing order when there are at most RANK_SORT_MAX of them: every
// workgroup holds all keys in LDS and finds the ranks of 8 of them, 32 threads per key (keys are
// distinct, one per row, so the ranks are a permutation).  One short launch instead of the
// passes of a radix sort over 64-bit keys.
#ifndef SDDMM_RANK_SORT_SPLIT
#define SDDMM_RANK_SORT_SPLIT 32
#endif
constexpr int RANK_SORT_MAX = 8192, RANK_SORT_BLOCK = 256, RANK_SORT_SPLIT = SDDMM_RANK_SORT_SPLIT;
__global__ __launch_bounds__(RANK_SORT_BLOCK) void k_rank_sort(const unsigned long long *__restrict__ in,
                                                               unsigned long long *__restrict__ out, int n) {
    __shared__ unsigned long long v[RANK_SORT_MAX];
    for (int i = (int)threadIdx.x; i < n; i += RANK_SORT_BLOCK) v[i] = in[i];
    __syncthreads();
    const int idx = (int)blockIdx.x * (RANK_SORT_BLOCK / RANK_SORT_SPLIT) + (int)(threadIdx.x / RANK_SORT_SPLIT);
    const int part = (int)(threadIdx.x % RANK_SORT_SPLIT);
    const unsigned long long mine = v[idx < n ? idx : n - 1];
    int below = 0;
#pragma unroll 8
    for (int i = part; i < n; i += RANK_SORT_SPLIT) below += v[i] < mine ? 1 : 0;
#pragma unroll
    for (int o = 1; o < RANK_SORT_SPLIT; o <<= 1) below += __shfl_xor(below, o, WAVE);
    if (part == 0 && idx < n) out[below] = mine;
}

// Gathered strips come in PAIRS: 32 consecutive candidates of the sorted order, the first 16
// as strip 2p, the rest as strip 2p+1, with ONE list of tile columns -- every tile column that
// any of the 32 rows touches -- so that the two strips have the same descriptors in the same
// order and a wavefront can use every B tile it loads for both (tile_window_pair_wave).  The
// list is padded with absent tile columns to a multiple of TILE_WINDOW, so that no window of
// four descriptors holds two strips, and stored window by window, the four descriptors of
// strip 2p followed by the four of strip 2p+1.
//
// Rows, extent and column span of pair vp; lanes 0..31 keep one row each.
struct GatheredHead {
    int row, s, e;        // per lane (row -1: none)
    int lo, span;         // wave-uniform, in tile columns
    int halves;           // wave-uniform: 2 when the second strip has rows, else 1
    int64_t entries;      // wave-uniform
};
__device__ __forceinline__ GatheredHead gathered_head(const int32_t *__restrict__ rowptr,
                                                      const int32_t *__restrict__ col,
                                                      const unsigned long long *__restrict__ sorted_keys,
                                                      int64_t n_cand, int64_t vp) {
    GatheredHead h;
    const int lane = lane_id();
    const int64_t idx = vp * 32 + lane;
    h.row = lane < 32 && idx < n_cand ? (int)(unsigned int)sorted_keys[idx] : -1;   // low half of the key
    h.s = h.row >= 0 ? rowptr[h.row] : 0;
    h.e = h.row >= 0 ? rowptr[h.row + 1] : 0;
    const bool has = h.e > h.s;
    const int first = has ? (col[h.s] >> 4) : INT32_MAX;
    const int last = has ? (col[h.e - 1] >> 4) : -1;
    // lanes 32..63 hold the neutral values; the 16-lane reductions of rows 0 and 1 of the wave make the pair's
    const int l16 = min16(first), h16 = min16(-last), n16 = sum16(h.e - h.s);
    const int l0 = __builtin_amdgcn_readlane(l16, 0), l1 = __builtin_amdgcn_readlane(l16, 16);
    const int g0 = __builtin_amdgcn_readlane(h16, 0), g1 = __builtin_amdgcn_readlane(h16, 16);
    const int l = l0 < l1 ? l0 : l1, hneg = g0 < g1 ? g0 : g1;
    h.lo = l;
    h.span = l == INT32_MAX ? 0 : -hneg - l + 1;
    h.entries = (int64_t)__builtin_amdgcn_readlane(n16, 0) + (int64_t)__builtin_amdgcn_readlane(n16, 16);
    h.halves = vp * 32 + 16 < n_cand ? 2 : 1;
    return h;
}

// One workgroup of 16 wavefronts per pair: wave i streams rows i and 16+i of the pair into the
// pair's tile-column bitmap in LDS (the rows are not neighbours in the CSR arrays, so they are
// independent streams).  Returns false when a row is not sorted.  Every wave of the workgroup
// must call it.
constexpr int GATHERED_BLOCK = 16 * WAVE;

__device__ __forceinline__ bool gathered_mark(const int32_t *__restrict__ col, const GatheredHead &h, unsigned int *bm,
                                              int *unsorted_flag) {
    const int words = (h.span + 31) >> 5;
    for (int w = (int)threadIdx.x; w < words; w += GATHERED_BLOCK) bm[w] = 0u;
    if (threadIdx.x == 0) *unsorted_flag = 0;
    __syncthreads();
    const int wi = wave_in_block();
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const int si = half ? __builtin_amdgcn_readlane(h.s, (wi & 15) + 16) : __builtin_amdgcn_readlane(h.s, wi & 15);
        const int ei = half ? __builtin_amdgcn_readlane(h.e, (wi & 15) + 16) : __builtin_amdgcn_readlane(h.e, wi & 15);
        if (ei > si) {                               // wave-uniform
            int64_t descents = 0;
            (void)strip_scan<1>(col, si, ei, INT64_MAX, h.lo, h.span, bm, &descents);
            if (descents != 0 && lane_id() == 0) atomicOr(unsorted_flag, 1);
        }
    }
    __syncthreads();
    return *unsorted_flag == 0;
}

// pass 1 of the gathered strips: descriptors per strip of the pair (0: not taken; the same for
// both strips), the strips' row table, ownership of the rows of a taken pair.
__global__ __launch_bounds__(GATHERED_BLOCK) void k_gathered_count(
    const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col,
    const unsigned long long *__restrict__ sorted_keys,
    int64_t n_cand, int64_t n_vpairs, int min_fill, unsigned int *__restrict__ vstrip_ntiles,
    int32_t *__restrict__ vrows, unsigned char *__restrict__ owner, DevCounters *pc) {
    __shared__ unsigned int bm[STRIP_BM_WORDS];
    __shared__ int unsorted_flag, tile_total;
    const int64_t vp = blockIdx.x;
    const int lane = lane_id();
    const bool first = wave_in_block() == 0;
    const GatheredHead h = gathered_head(rowptr, col, sorted_keys, n_cand, vp);   // the same in every wave
    if (first && lane < 32) vrows[vp * 32 + lane] = h.row;
    int tiles = 0;
    bool take = false;
    if (h.span > 0 && h.span <= STRIP_BM_WORDS * 32 && h.entries >= min_fill) {   // workgroup-uniform
        const bool sorted = gathered_mark(col, h, bm, &unsorted_flag);
        if (threadIdx.x == 0) tile_total = 0;
        __syncthreads();
        const int words = (h.span + 31) >> 5;
        int t = 0;
        for (int w = (int)threadIdx.x; w < words; w += GATHERED_BLOCK) t += __builtin_popcount(bm[w]);
        t = wave_sum_i32(t);
        if (lane == 0 && t) atomicAdd(&tile_total, t);
        __syncthreads();
        tiles = tile_total;
        // the threshold is per 16x16 tile: each tile column of the pair is one tile per strip that has rows
        take = sorted && tiles > 0 && h.entries >= (int64_t)min_fill * tiles * h.halves;
    }
    const int padded = (tiles + TILE_WINDOW - 1) / TILE_WINDOW * TILE_WINDOW;
    if (first) {
        if (take && h.row >= 0) owner[h.row] = 3;
        if (lane == 0) {
            vstrip_ntiles[2 * vp] = take ? (unsigned int)padded : 0u;
            vstrip_ntiles[2 * vp + 1] = take ? (unsigned int)padded : 0u;
            if (take) {
                spread_add(pc, K_TILES, 2ull * (unsigned long long)padded);
                spread_add(pc, K_NNZ_TILES, (unsigned long long)h.entries);
            }
        }
    }
}

// A descriptor that stands for nothing (no row has an entry in it): complete, k_tile_rows skips it.
__device__ __forceinline__ void write_empty_desc(TileDesc *__restrict__ tiles, int32_t *__restrict__ tile_cols,
                                                 int64_t at, int strip, int tj) {
    int4 *d = reinterpret_cast<int4 *>(tiles + at);
    d[0] = make_int4(strip, tj, 1, 0);
#pragma unroll
    for (int k = 1; k < (int)(sizeof(TileDesc) / 16); ++k) d[k] = make_int4(0, 0, 0, 0);
    write_aligned_cols(tile_cols, at, tj);
}

// pass 2 of the gathered strips: strip and tile column of every descriptor, window by window
// (descriptor 8k + 4h + j of the pair: strip h, the (4k+j)-th tile column).  `tiles` / `tile_cols`
// point at the first gathered descriptor; the `lead` descriptors before it (fewer than
// TILE_WINDOW) fill the last window of the strips that precede the gathered ones.
__global__ __launch_bounds__(GATHERED_BLOCK) void k_gathered_tiles(
    const int32_t *__restrict__ rowptr, const int32_t *__restrict__ col,
    const unsigned long long *__restrict__ sorted_keys,
    int64_t n_cand, int64_t n_vpairs, const unsigned int *__restrict__ vstrip_ntiles,
    const unsigned int *__restrict__ vstrip_off, TileDesc *__restrict__ tiles, int32_t *__restrict__ tile_cols,
    int lead) {
    __shared__ unsigned int bm[STRIP_BM_WORDS];
    __shared__ int unsorted_flag;
    const int64_t vp = blockIdx.x;
    // (strip -1 is nobody's: the window that holds them is walked tile by tile, and they write nothing)
    if (vp == 0 && (int)threadIdx.x < lead) write_empty_desc(tiles, tile_cols, -(int64_t)lead + threadIdx.x, -1, 0);
    const unsigned int per_strip = vstrip_ntiles[2 * vp];
    if (per_strip == 0) return;                      // workgroup-uniform
    const int lane = lane_id();
    const GatheredHead h = gathered_head(rowptr, col, sorted_keys, n_cand, vp);
    (void)gathered_mark(col, h, bm, &unsorted_flag);
    if (wave_in_block() != 0) return;                // the first wave writes the descriptors in column order
    const int words = (h.span + 31) >> 5;
    const int64_t base = vstrip_off[2 * vp];
    const int strip0 = GATHERED_BASE + (int)(2 * vp);
    auto put = [&](int rank, int tj) {
        const int64_t at = base + 2 * TILE_WINDOW * (rank / TILE_WINDOW) + (rank % TILE_WINDOW);
        *reinterpret_cast<int4 *>(tiles + at) = make_int4(strip0, tj, 0, 0);
        write_aligned_cols(tile_cols, at, tj);
        *reinterpret_cast<int4 *>(tiles + at + TILE_WINDOW) = make_int4(strip0 + 1, tj, 0, 0);
        write_aligned_cols(tile_cols, at + TILE_WINDOW, tj);
    };
    int run = 0, top = -1;
    for (int wb = 0; wb < words; wb += WAVE) {
        const int w = wb + lane;
        unsigned int x = w < words ? bm[w] : 0u;
        const int n = __builtin_popcount(x);
        int incl = n;
        for (int o = 1; o < WAVE; o <<= 1) {
            const int up = __shfl_up(incl, o, WAVE);
            if (lane >= o) incl += up;
        }
        int rank = run + (incl - n);
        while (x) {
            const int b = __builtin_ctz(x);
            x &= x - 1;
            const int tj = h.lo + w * 32 + b;
            put(rank, tj);
            top = tj;                                 // ascending inside a lane and from lane to lane
            ++rank;
        }
        run += __builtin_amdgcn_readlane(incl, WAVE - 1);
    }
    // the padding: tile columns beyond the pair's last one, which no row of the pair has
    for (int o = WAVE / 2; o > 0; o >>= 1) {
        const int other = __shfl_xor(top, o, WAVE);
        top = other > top ? other : top;
    }
    // (k_tile_rows gives them their per-row positions like any other descriptor: the masks come out
    // empty, the positions say where a row's entries before that column end)
    if (run + lane < (int)per_strip) put(run + lane, top + 1 + lane);
}

// pass 3: one thread per (descriptor, row): CSR position of the row's first entry
// at or after the tile's first column, and the mask of the tile's columns present.
// Bit n of the mask stands for the n-th of the tile's 16 columns; a row's entries
// inside a tile are consecutive in CSR, in the order of the tile's columns.
__global__ __launch_bounds__(256) void k_tile_rows(const int32_t *__restrict__ rowptr,
                                                   const int32_t *__restrict__ col, int M,
                                                   const int32_t *__restrict__ vrows,
                                                   const int32_t *__restrict__ tile_cols,
                                                   TileDesc *__restrict__ tiles, int64_t n_tiles) {
    const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t t = slot >> 4;
    const int sub = (int)(slot & 15);
    if (t >= n_tiles) return;
    TileDesc *d = tiles + t;
    const int4 head = *reinterpret_cast<const int4 *>(d);     // strip, tj, pad[0], pad[1]
    if (head.z != 0) return;                                   // written by the merging walk
    const int64_t row = head.x >= GATHERED_BASE ? (int64_t)vrows[(int64_t)(head.x - GATHERED_BASE) * 16 + sub]
                                                : (int64_t)head.x * 16 + sub;
    int p = 0, end = 0;
    if (row >= 0 && row < M) { p = rowptr[row]; end = rowptr[row + 1]; }
    int tc[16];
    {
        const int4 *src = reinterpret_cast<const int4 *>(tile_cols + t * 16);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int4 v = src[k];
            tc[4 * k] = v.x; tc[4 * k + 1] = v.y; tc[4 * k + 2] = v.z; tc[4 * k + 3] = v.w;
        }
    }
    int top = tc[0];                                           // last real column of the tile
#pragma unroll
    for (int k = 1; k < 16; ++k) top = tc[k] != INT32_MAX ? tc[k] : top;
    const int target = tc[0];
    int a = p, b = end;
    while (a < b) {
        const int mid = a + ((b - a) >> 1);
        if (col[mid] < target) a = mid + 1; else b = mid;
    }
    unsigned int mask = 0;
    if (a < end) {
        const int last = end - 1;
        int cs[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) cs[j] = col[a + j < last ? a + j : last];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if (a + j <= last && cs[j] <= top) {
                int n = 0;                                     // number of tile columns below this one
#pragma unroll
                for (int k = 0; k < 16; ++k) n += tc[k] < cs[j] ? 1 : 0;
                mask |= 1u << n;
            }
        }
    }
    d->off[sub] = a;
    d->mask[sub] = (uint16_t)mask;
}

// generic exclusive scan of n unsigned ints: block sums, then apply
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_sums(const unsigned int *__restrict__ in, int64_t n,
                                                          unsigned int *__restrict__ block_sums) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    unsigned int mine = 0;
    for (int q = 0; q < SCAN_ITEMS; ++q) mine += base + q < n ? in[base + q] : 0u;
    unsigned int total;
    (void)block_exclusive_scan(mine, &total);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_apply(const unsigned int *__restrict__ in, int64_t n,
                                                           const unsigned int *__restrict__ block_offsets,
                                                           unsigned int *__restrict__ out) {
    const int64_t base = (int64_t)blockIdx.x * SCAN_TILE + (int64_t)threadIdx.x * SCAN_ITEMS;
    unsigned int v[SCAN_ITEMS], mine = 0;
    for (int q = 0; q < SCAN_ITEMS; ++q) { v[q] = base + q < n ? in[base + q] : 0u; mine += v[q]; }
    unsigned int total;
    unsigned int at = block_offsets[blockIdx.x] + block_exclusive_scan(mine, &total);
    for (int q = 0; q < SCAN_ITEMS; ++q) {
        if (base + q < n) out[base + q] = at;
        at += v[q];
    }
}

// ---- the MFMA kernel ------------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

// One wavefront computes `tiles_per_wave` consecutive tiles.  Operand layout of
// both MFMA shapes used: lane l supplies row (l & 15) of its operand and the k
// positions selected by (l >> 4); the result register i of lane l is row
// 4*(l >> 4) + i, column (l & 15).  In step s operand lane l holds the 16-byte unit
// 4*s + (l >> 4) of its row; which k positions end up in which MFMA does not matter
// as long as A and B agree.  STEPS = row bytes / 64.
// The units are READ in another layout -- four neighbouring lanes on the 64
// contiguous bytes of one row, 16 line segments per instruction instead of the 64 a
// load in operand layout touches -- and moved into the operand layout through the
// LDS crossbar (ds_bpermute): the vector memory pipeline pays per line segment that
// neighbouring lanes touch, not per byte.
//
// Software pipeline, three tiles deep, every load unconditional so that the wait
// counts stay exact (loads return in issue order):
//   iteration t issues   B rows + S values of tile t+1   (needs descriptor t+1)
//                        descriptor of tile t+2
//   and then computes    MFMAs of tile t, scale, scatter (operands landed during t-1)
// The A panel of the current strip stays in registers and is reloaded only when
// the strip changes (a wave-uniform branch placed before the iteration's loads).
// tiles [w*tiles_per_wave, (w+1)*tiles_per_wave) on the calling wavefront
template <int DT, int STEPS>
__device__ __forceinline__ void tile_wave(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                          const int32_t *__restrict__ vrows, const int32_t *__restrict__ tile_cols,
                                          const TileDesc *__restrict__ tiles, int64_t n_tiles, int tiles_per_wave,
                                          const float *__restrict__ sval, float *__restrict__ P, int64_t w) {
    int64_t t = w * tiles_per_wave;
    if (t >= n_tiles) return;
    int64_t t_end = t + tiles_per_wave;
    t_end = t_end < n_tiles ? t_end : n_tiles;
    const int64_t t_last = t_end - 1;
    const int lane = lane_id();
    const int r16 = lane & 15, q = lane >> 4;        // operand / result layout
    const int lrow = lane >> 2, lunit = lane & 3;    // memory layout: four neighbouring lanes on 64 bytes of a row
    const int to_operand_from = (4 * r16 + q) << 2;  // ds_bpermute address: operand lane (r16,q) <- memory lane 4*r16+q
    constexpr uint32_t ROW_UNITS = STEPS * 4;
    const uint4 *__restrict__ Au = (const uint4 *)A;
    const uint4 *__restrict__ Bu = (const uint4 *)B;
    const unsigned int below = (1u << r16) - 1u;
    auto to_operand = [&](const uint4 &v) {
        uint4 r;
        r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.x);
        r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.y);
        r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.z);
        r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.w);
        return r;
    };

    struct Desc {
        int strip, bcol;    // bcol: the B row this lane loads (memory layout)
        int4 off;
        uint2 mask;
    };
    struct Oper {
        uint4 b[STEPS];
        float s[4];
        int pos[4];
        unsigned int act;   // bit i: result register i is a stored entry
    };
    auto load_desc = [&](int64_t ti) {
        ti = ti < t_last ? ti : t_last;
        const TileDesc *d = tiles + ti;
        Desc r;
        r.strip = d->strip;
        r.bcol = tile_cols[ti * 16 + lrow];
        r.off = *(const int4 *)&d->off[q * 4];
        r.mask = *(const uint2 *)&d->mask[q * 4];
        return r;
    };
    auto load_oper = [&](const Desc &d) {
        Oper o;
        int64_t brow = d.bcol;
        brow = brow < N ? brow : N - 1;   // columns past N (and the filler of a short union tile) are never in a mask
        const uint4 *src = Bu + brow * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) o.b[s] = src[s * 4];
        const int offs[4] = {d.off.x, d.off.y, d.off.z, d.off.w};
        const unsigned int masks[4] = {d.mask.x & 0xFFFFu, d.mask.x >> 16, d.mask.y & 0xFFFFu, d.mask.y >> 16};
        o.act = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool on = (masks[i] >> r16) & 1u;
            o.act |= on ? (1u << i) : 0u;
            // position of (row 4q+i, column r16) in the CSR arrays; entry 0 when absent
            o.pos[i] = on ? offs[i] + __builtin_popcount(masks[i] & below) : 0;
            o.s[i] = sval[o.pos[i]];
        }
        return o;
    };

    Desc d_cur = load_desc(t);
    Oper o_cur = load_oper(d_cur);
    Desc d_nxt = load_desc(t + 1);
    int cur_strip = -1;
    uint4 a[STEPS];
    for (; t < t_end; ++t) {
        const int strip = __builtin_amdgcn_readfirstlane(d_cur.strip);
        if (strip != cur_strip) {
            cur_strip = strip;
            int64_t arow = strip >= GATHERED_BASE ? (int64_t)vrows[(int64_t)(strip - GATHERED_BASE) * 16 + lrow]
                                                  : (int64_t)strip * 16 + lrow;
            arow = arow < 0 ? 0 : (arow < M ? arow : M - 1);   // missing rows are never in a mask
            const uint4 *src = Au + arow * ROW_UNITS + lunit;
#pragma unroll
            for (int s = 0; s < STEPS; ++s) a[s] = to_operand(src[s * 4]);
        }
        const Oper o_nxt = load_oper(d_nxt);
        const Desc d_nn = load_desc(t + 2);
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const uint4 b = to_operand(o_cur.b[s]);
            if constexpr (DT == DT_BF16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                              __builtin_bit_cast(bf16x8_t, b), acc, 0, 0, 0);
            } else if constexpr (DT == DT_F16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a[s]),
                                                             __builtin_bit_cast(half8_t, b), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].x),
                                                           __builtin_bit_cast(float, b.x), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].y),
                                                           __builtin_bit_cast(float, b.y), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].z),
                                                           __builtin_bit_cast(float, b.z), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].w),
                                                           __builtin_bit_cast(float, b.w), acc, 0, 0, 0);
            }
        }
        // scale by S and scatter: result register i is row 4*q+i, column r16
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if ((o_cur.act >> i) & 1u) P[o_cur.pos[i]] = acc[i] * o_cur.s[i];
        o_cur = o_nxt;
        d_cur = d_nxt;
        d_nxt = d_nn;
    }
}

// ---- windows of four tiles ---------------------------------------------------------
// A wavefront that walks its tiles one after the other spends its life waiting: a launch
// of this path lasts a dozen microseconds, a dependent memory round trip about one, and
// the walk chains descriptor -> operands -> result for every tile.  So the unit of work is
// a WINDOW of TILE_WINDOW consecutive descriptors of one strip, handled as a batch with
// two round trips: (1) the window record, one dword per lane; (2) everything else at once
// -- the A panel, the B rows of all its tiles, and the S values and column indices.
//
// S and P are not accessed per (row, tile): the entries of row r inside the window's
// tiles are consecutive in the CSR arrays (the tiles are consecutive present tiles of the
// strip, so nothing of the row lies between them), cnt[r] entries from p0[r].  Four
// lanes per row read and write them 16 bytes at a time whatever the fill of the tiles
// (the last lane of a row moves its four entries back so that they end with the row's
// run: some entries are written twice with the same value, none is written in parts).
// The products come from the matrix cores in result layout, pass through LDS (written
// by columns of 16 rows, 16 bytes per lane) and are picked up per entry: its column says
// which tile and which column of the tile.  Per window of four tiles with 92 entries
// each: 20 memory instructions instead of 56.
//
// A window whose descriptors are not plain aligned tiles of one strip (a strip ends
// inside it, union tiles) is flagged by the plan and walked tile by tile (tile_wave).
constexpr int WIN_PITCH = 20;                 // floats per result column in LDS: 16 rows, padded, 16-byte aligned
constexpr int WIN_LDS_FLOATS = TILE_WINDOW * 16 * WIN_PITCH;

struct alignas(16) TileWindow {               // lane l < 48 loads dword l
    int32_t arow[16];    // row of A for strip row r (row 0 where the strip has no such row: then cnt is 0)
    int32_t p0[16];      // CSR position of row r's first entry inside the window
    uint16_t cnt[16];    // entries of row r inside the window (consecutive from p0)
    int32_t tj[TILE_WINDOW];   // tile columns, -1 where the window has fewer tiles
    int32_t flags;       // != 0: walk the window tile by tile
    int32_t maxcnt;      // largest cnt
    int32_t paired;      // != 0: a window of a pair of gathered strips (same tile columns as its neighbour)
    int32_t pad;
};
static_assert(sizeof(TileWindow) == 192, "TileWindow layout");

// plan: one thread per (window, strip row)
__global__ __launch_bounds__(256) void k_tile_windows(const int32_t *__restrict__ vrows, int M, int64_t nnz,
                                                      const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                      int64_t union_lo, int64_t union_hi, int64_t gathered_lo,
                                                      TileWindow *__restrict__ win, int64_t n_win) {
    const int64_t slot = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t w = slot >> 4;
    const int r = (int)(slot & 15);
    if (w >= n_win) return;                   // groups of 16 lanes leave together
    const int64_t t0 = w * TILE_WINDOW;
    const int n = (int)(n_tiles - t0 < TILE_WINDOW ? n_tiles - t0 : TILE_WINDOW);
    const int4 h0 = *reinterpret_cast<const int4 *>(tiles + t0);          // strip, tj, pad[0], pad[1]
    // the 16-byte accesses of the batch need four entries to exist
    bool mixed = (t0 < union_hi && t0 + n > union_lo) || nnz < 4;
    int tj[TILE_WINDOW];
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k) {
        tj[k] = -1;
        if (k < n) {
            const int4 h = *reinterpret_cast<const int4 *>(tiles + t0 + k);
            tj[k] = h.y;
            mixed |= h.x != h0.x;
        }
    }
    const int strip = h0.x;
    const int64_t row = strip >= GATHERED_BASE ? (int64_t)vrows[(int64_t)(strip - GATHERED_BASE) * 16 + r]
                                               : (int64_t)strip * 16 + r;
    const bool valid = row >= 0 && row < M;
    const TileDesc *last = tiles + t0 + n - 1;
    const int p0 = tiles[t0].off[r];
    int cnt = valid && !mixed ? last->off[r] + __builtin_popcount((unsigned int)last->mask[r]) - p0 : 0;
    cnt = cnt < 0 ? 0 : (cnt > 16 * TILE_WINDOW ? 16 * TILE_WINDOW : cnt);
    const int mx = max16(cnt);
    TileWindow *o = win + w;
    o->arow[r] = valid ? (int32_t)row : 0;
    o->p0[r] = p0;
    o->cnt[r] = (uint16_t)cnt;
    if (r == 0) {
#pragma unroll
        for (int k = 0; k < TILE_WINDOW; ++k) o->tj[k] = tj[k];
        o->flags = mixed ? 1 : 0;
        o->maxcnt = mx;
        o->paired = t0 >= gathered_lo ? 1 : 0;
        o->pad = 0;
    }
}

// window w on the calling wavefront; lds: WIN_LDS_FLOATS floats of its own
template <int DT, int STEPS>
__device__ __forceinline__ void tile_window_wave(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                                 const int32_t *__restrict__ vrows,
                                                 const int32_t *__restrict__ tile_cols,
                                                 const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                 const TileWindow *__restrict__ win, int64_t n_win,
                                                 const int32_t *__restrict__ col, const float *__restrict__ sval,
                                                 float *__restrict__ P, int64_t nnz, int64_t w, float *lds,
                                                 const int32_t *__restrict__ order = nullptr) {
    if (w >= n_win) return;
    if (order) w = order[w];                              // the plan's order of the windows (k_window_order)
    const int lane = lane_id();
    if (win == nullptr) {                                 // the plan chose the tile-by-tile walk for this matrix
        tile_wave<DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, TILE_WINDOW, sval, P, w);
        return;
    }
    const int32_t *rec = reinterpret_cast<const int32_t *>(win + w);
    const int dw = rec[lane < 48 ? lane : 47];
    if (__builtin_amdgcn_readlane(dw, 44) != 0) {
        tile_wave<DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, TILE_WINDOW, sval, P, w);
        return;
    }
    const int maxcnt = __builtin_amdgcn_readlane(dw, 45);
    if (maxcnt <= 0) return;
    const int r16 = lane & 15, q = lane >> 4;        // operand / result layout
    const int lrow = lane >> 2, lunit = lane & 3;    // memory layout: four neighbouring lanes on 64 bytes of a row
    const int to_operand_from = (4 * r16 + q) << 2;
    constexpr uint32_t ROW_UNITS = STEPS * 4;
    const uint4 *__restrict__ Au = (const uint4 *)A;
    const uint4 *__restrict__ Bu = (const uint4 *)B;
    auto to_operand = [&](const uint4 &v) {
        uint4 r;
        r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.x);
        r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.y);
        r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.z);
        r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.w);
        return r;
    };
    int tj[TILE_WINDOW];
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k) tj[k] = __builtin_amdgcn_readlane(dw, 40 + k);
    // the row of the S/P accesses of this lane: strip row lane>>2, its entries 4(lane&3)+16m.. of the window
    const int p0 = __shfl(dw, 16 + lrow, WAVE);
    const int cw = __shfl(dw, 32 + (lrow >> 1), WAVE);
    const int cnt = (lrow & 1) ? (int)((unsigned int)cw >> 16) : (cw & 0xFFFF);
    const int64_t arow = __shfl(dw, lrow, WAVE);
    auto entry_pos = [&](int m) {
        int ws = 4 * lunit + 16 * m;
        ws = ws < cnt - 4 ? ws : cnt - 4;
        ws = ws < 0 ? 0 : ws;
        const int64_t pos = (int64_t)p0 + ws;
        return pos < nnz - 4 ? pos : nnz - 4;            // only rows of fewer than four entries can get here
    };
    // ---- second round trip: everything at once ----------------------------------------
    uint4 a_mem[STEPS];
    {
        const uint4 *src = Au + arow * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) a_mem[s] = src[s * 4];
    }
    auto load_b = [&](int k, uint4 (&dst)[STEPS]) {
        int64_t brow = (int64_t)(tj[k] < 0 ? 0 : tj[k]) * 16 + lrow;
        brow = brow < N ? brow : N - 1;                   // columns past N are in no row's entries
        const uint4 *src = Bu + brow * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) dst[s] = src[s * 4];
    };
    // rows of up to 128 bytes: the B rows of all four tiles in flight; longer rows two tiles at a time (at 256
    // bytes four in flight cost 13 registers and a wave per SIMD of the launch that also runs rows: 22.0 -> 21.2 us)
    constexpr bool ALL_B = STEPS <= 2;
    uint4 b[ALL_B ? TILE_WINDOW : 2][STEPS];
    if constexpr (ALL_B) {
#pragma unroll
        for (int k = 0; k < TILE_WINDOW; ++k) load_b(k, b[k]);
    } else {
        load_b(0, b[0]);
    }
    const int iters = (maxcnt + 15) >> 4;                 // wave-uniform, 1..4
    I4u c_pre[2];
    F4u s_pre[2];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
        const int64_t pos = entry_pos(m < iters ? m : 0);
        c_pre[m] = *reinterpret_cast<const I4u *>(col + pos);
        s_pre[m] = *reinterpret_cast<const F4u *>(sval + pos);
    }
    // ---- products of every tile into LDS ------------------------------------------------
    uint4 a[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) a[s] = to_operand(a_mem[s]);
    auto product = [&](const uint4 (&bt)[STEPS], int k) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const uint4 bo = to_operand(bt[s]);
            if constexpr (DT == DT_BF16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                              __builtin_bit_cast(bf16x8_t, bo), acc, 0, 0, 0);
            } else if constexpr (DT == DT_F16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a[s]),
                                                             __builtin_bit_cast(half8_t, bo), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].x),
                                                           __builtin_bit_cast(float, bo.x), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].y),
                                                           __builtin_bit_cast(float, bo.y), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].z),
                                                           __builtin_bit_cast(float, bo.z), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].w),
                                                           __builtin_bit_cast(float, bo.w), acc, 0, 0, 0);
            }
        }
        // result register i of lane (r16, q) is row 4q+i, column r16 of tile k
        *reinterpret_cast<f32x4_t *>(lds + (k * 16 + r16) * WIN_PITCH + 4 * q) = acc;
    };
    if constexpr (ALL_B) {
#pragma unroll
        for (int k = 0; k < TILE_WINDOW; ++k)
            if (tj[k] >= 0) product(b[k], k);             // wave-uniform
    } else {
#pragma unroll
        for (int k = 0; k < TILE_WINDOW; ++k) {
            if (tj[k] < 0) break;                         // wave-uniform
            if (k + 1 < TILE_WINDOW && tj[k + 1 < TILE_WINDOW ? k + 1 : k] >= 0) load_b(k + 1, b[(k + 1) & 1]);
            product(b[k & 1], k);
        }
    }
    wave_lds_order();
    // ---- entries: four per lane, 16 per row and iteration -----------------------------------
    const int t1 = tj[1], t2 = tj[2], t3 = tj[3];
    auto pick = [&](int c) {
        const int tc = c >> 4;
        const int k = (tc == t1 ? 1 : 0) + (tc == t2 ? 2 : 0) + (tc == t3 ? 3 : 0);
        return lds[(k * 16 + (c & 15)) * WIN_PITCH + lrow];
    };
    for (int m = 0; m < iters; ++m) {
        I4u c4;
        F4u s4;
        if (m < 2) { c4 = c_pre[m]; s4 = s_pre[m]; }
        else {
            const int64_t pos = entry_pos(m);
            c4 = *reinterpret_cast<const I4u *>(col + pos);
            s4 = *reinterpret_cast<const F4u *>(sval + pos);
        }
        const bool active = cnt >= 4 && 4 * lunit + 16 * m < cnt;
        const F4u out{pick(c4.x) * s4.x, pick(c4.y) * s4.y, pick(c4.z) * s4.z, pick(c4.w) * s4.w};
        if (active) *reinterpret_cast<F4u *>(P + entry_pos(m)) = out;
    }
    // rows with one to three entries in the window: entry by entry
    if (cnt > 0 && cnt < 4 && lunit == 0) {
        for (int e = 0; e < cnt; ++e) P[(int64_t)p0 + e] = pick(col[(int64_t)p0 + e]) * sval[(int64_t)p0 + e];
    }
    wave_lds_order();                                     // the next window of this wave reuses the buffer
}

constexpr int PAIR_MAX_STEPS = 4;             // row bytes / 64 up to which pairs of windows share a wavefront
// Windows wa and wa+1 of a pair of gathered strips on the calling wavefront: the same four tile
// columns for 2 x 16 rows.  Every B tile is loaded and moved into operand layout once and
// multiplied with both A panels; the products of the second strip wait in registers while the
// entries of the first are picked out of the LDS buffer (one buffer, as for a single window).
template <int DT, int STEPS>
__device__ __forceinline__ void tile_window_pair_wave(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                                      const int32_t *__restrict__ vrows,
                                                      const int32_t *__restrict__ tile_cols,
                                                      const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                      const TileWindow *__restrict__ win, int64_t n_win,
                                                      const int32_t *__restrict__ col, const float *__restrict__ sval,
                                                      float *__restrict__ P, int64_t nnz, int64_t wa, float *lds) {
    if (wa >= n_win) return;
    const int lane = lane_id();
    const int li = lane < 48 ? lane : 47;
    const int dw0 = reinterpret_cast<const int32_t *>(win + wa)[li];
    const int dw1 = reinterpret_cast<const int32_t *>(win + (wa + 1 < n_win ? wa + 1 : wa))[li];
    bool plain = wa + 1 < n_win && __builtin_amdgcn_readlane(dw0, 44) == 0 && __builtin_amdgcn_readlane(dw1, 44) == 0 &&
                 __builtin_amdgcn_readlane(dw0, 46) != 0 && __builtin_amdgcn_readlane(dw1, 46) != 0;
    int tj[TILE_WINDOW];
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k) {
        tj[k] = __builtin_amdgcn_readlane(dw0, 40 + k);
        plain = plain && tj[k] == __builtin_amdgcn_readlane(dw1, 40 + k);
    }
    if (!plain) {                                         // wave-uniform: one window after the other
        for (int64_t w = wa; w < wa + 2; ++w)
            tile_window_wave<DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, win, n_win, col, sval, P, nnz, w, lds);
        return;
    }
    const int maxcnt0 = __builtin_amdgcn_readlane(dw0, 45), maxcnt1 = __builtin_amdgcn_readlane(dw1, 45);
    if (maxcnt0 <= 0 && maxcnt1 <= 0) return;
    const int r16 = lane & 15, q = lane >> 4;        // operand / result layout
    const int lrow = lane >> 2, lunit = lane & 3;    // memory layout: four neighbouring lanes on 64 bytes of a row
    const int to_operand_from = (4 * r16 + q) << 2;
    constexpr uint32_t ROW_UNITS = STEPS * 4;
    const uint4 *__restrict__ Au = (const uint4 *)A;
    const uint4 *__restrict__ Bu = (const uint4 *)B;
    auto to_operand = [&](const uint4 &v) {
        uint4 r;
        r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.x);
        r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.y);
        r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.z);
        r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.w);
        return r;
    };
    // S/P accesses of this lane in either strip: strip row lane>>2, its entries 4(lane&3)+16m.. of the window
    struct Rows { int p0, cnt; };
    auto rows_of = [&](int dw) {
        Rows r;
        r.p0 = __shfl(dw, 16 + lrow, WAVE);
        const int cw = __shfl(dw, 32 + (lrow >> 1), WAVE);
        r.cnt = (lrow & 1) ? (int)((unsigned int)cw >> 16) : (cw & 0xFFFF);
        return r;
    };
    const Rows rows0 = rows_of(dw0), rows1 = rows_of(dw1);
    auto entry_pos = [&](const Rows &r, int m) {
        int ws = 4 * lunit + 16 * m;
        ws = ws < r.cnt - 4 ? ws : r.cnt - 4;
        ws = ws < 0 ? 0 : ws;
        const int64_t pos = (int64_t)r.p0 + ws;
        return pos < nnz - 4 ? pos : nnz - 4;
    };
    // ---- second round trip: both A panels, the B tiles, the first column indices and S values ----
    uint4 a0[STEPS], a1[STEPS];
    {
        const int64_t ar0 = __shfl(dw0, lrow, WAVE), ar1 = __shfl(dw1, lrow, WAVE);
        const uint4 *s0 = Au + ar0 * ROW_UNITS + lunit, *s1 = Au + ar1 * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) { a0[s] = s0[s * 4]; a1[s] = s1[s * 4]; }
    }
    auto load_b = [&](int k, uint4 (&dst)[STEPS]) {
        int64_t brow = (int64_t)(tj[k] < 0 ? 0 : tj[k]) * 16 + lrow;
        brow = brow < N ? brow : N - 1;                   // columns past N are in no row's entries
        const uint4 *src = Bu + brow * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) dst[s] = src[s * 4];
    };
    uint4 b[2][STEPS];                                    // two B tiles in flight
    load_b(0, b[0]);
    if (tj[1] >= 0) load_b(1, b[1]);                      // wave-uniform
    struct Pre { I4u c[2]; F4u s[2]; };
    auto prefetch = [&](const Rows &r, int iters) {
        Pre p;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
            const int64_t pos = entry_pos(r, m < iters ? m : 0);
            p.c[m] = *reinterpret_cast<const I4u *>(col + pos);
            p.s[m] = *reinterpret_cast<const F4u *>(sval + pos);
        }
        return p;
    };
    const int iters0 = (maxcnt0 + 15) >> 4, iters1 = (maxcnt1 + 15) >> 4;      // wave-uniform, 0..4
    const Pre pre0 = prefetch(rows0, iters0);
    // ---- products: strip 0's into LDS, strip 1's kept ----------------------------------------------
#pragma unroll
    for (int s = 0; s < STEPS; ++s) { a0[s] = to_operand(a0[s]); a1[s] = to_operand(a1[s]); }
    f32x4_t keep[TILE_WINDOW];
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k) {
        keep[k] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (tj[k] < 0) continue;                          // wave-uniform
        f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const uint4 bo = to_operand(b[k & 1][s]);
            if constexpr (DT == DT_BF16) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a0[s]),
                                                               __builtin_bit_cast(bf16x8_t, bo), acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a1[s]),
                                                               __builtin_bit_cast(bf16x8_t, bo), acc1, 0, 0, 0);
            } else if constexpr (DT == DT_F16) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a0[s]),
                                                              __builtin_bit_cast(half8_t, bo), acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a1[s]),
                                                              __builtin_bit_cast(half8_t, bo), acc1, 0, 0, 0);
            } else {
                const float bf[4] = {__builtin_bit_cast(float, bo.x), __builtin_bit_cast(float, bo.y),
                                     __builtin_bit_cast(float, bo.z), __builtin_bit_cast(float, bo.w)};
                const float f0[4] = {__builtin_bit_cast(float, a0[s].x), __builtin_bit_cast(float, a0[s].y),
                                     __builtin_bit_cast(float, a0[s].z), __builtin_bit_cast(float, a0[s].w)};
                const float f1[4] = {__builtin_bit_cast(float, a1[s].x), __builtin_bit_cast(float, a1[s].y),
                                     __builtin_bit_cast(float, a1[s].z), __builtin_bit_cast(float, a1[s].w)};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(f0[i], bf[i], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(f1[i], bf[i], acc1, 0, 0, 0);
                }
            }
        }
        // the registers of this B tile are free: the tile after the next one
        if (k + 2 < TILE_WINDOW && tj[k + 2 < TILE_WINDOW ? k + 2 : k] >= 0) load_b(k + 2, b[k & 1]);
        // result register i of lane (r16, q) is row 4q+i, column r16 of tile k
        *reinterpret_cast<f32x4_t *>(lds + (k * 16 + r16) * WIN_PITCH + 4 * q) = acc0;
        keep[k] = acc1;
    }
    wave_lds_order();
    const Pre pre1 = prefetch(rows1, iters1);             // lands while strip 0's entries are written
    // ---- entries: four per lane, 16 per row and iteration ---------------------------------------------
    const int t1 = tj[1], t2 = tj[2], t3 = tj[3];
    auto pick = [&](int c) {
        const int tc = c >> 4;
        const int k = (tc == t1 ? 1 : 0) + (tc == t2 ? 2 : 0) + (tc == t3 ? 3 : 0);
        return lds[(k * 16 + (c & 15)) * WIN_PITCH + lrow];
    };
    auto entries = [&](const Rows &r, const Pre &pre, int iters) {
        for (int m = 0; m < iters; ++m) {
            I4u c4;
            F4u s4;
            if (m < 2) { c4 = pre.c[m]; s4 = pre.s[m]; }
            else {
                const int64_t pos = entry_pos(r, m);
                c4 = *reinterpret_cast<const I4u *>(col + pos);
                s4 = *reinterpret_cast<const F4u *>(sval + pos);
            }
            const bool active = r.cnt >= 4 && 4 * lunit + 16 * m < r.cnt;
            const F4u out{pick(c4.x) * s4.x, pick(c4.y) * s4.y, pick(c4.z) * s4.z, pick(c4.w) * s4.w};
            if (active) *reinterpret_cast<F4u *>(P + entry_pos(r, m)) = out;
        }
        // rows with one to three entries in the window: entry by entry
        if (r.cnt > 0 && r.cnt < 4 && lunit == 0) {
            for (int e = 0; e < r.cnt; ++e) P[(int64_t)r.p0 + e] = pick(col[(int64_t)r.p0 + e]) * sval[(int64_t)r.p0 + e];
        }
    };
    entries(rows0, pre0, iters0);
    wave_lds_order();
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k)
        if (tj[k] >= 0) *reinterpret_cast<f32x4_t *>(lds + (k * 16 + r16) * WIN_PITCH + 4 * q) = keep[k];
    wave_lds_order();
    entries(rows1, pre1, iters1);
    wave_lds_order();                                     // the next window of this wave reuses the buffer
}

// Wavefront `unit` of a tile launch: windows [0, n_single) one per wavefront, the windows after them (pairs of
// gathered strips) two per wavefront.
template <int DT, int STEPS>
__device__ __forceinline__ void tile_unit_wave(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                               const int32_t *__restrict__ vrows, const int32_t *__restrict__ tile_cols,
                                               const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                               const TileWindow *__restrict__ win, int64_t n_win, int64_t n_single,
                                               const int32_t *__restrict__ col, const float *__restrict__ sval,
                                               float *__restrict__ P, int64_t nnz, int64_t unit, float *lds,
                                               const int32_t *__restrict__ order) {
    // (rows beyond 256 bytes: the second A panel and the kept products do not fit the registers, the
    // plan gives such launches one wavefront per window throughout)
    if (STEPS > PAIR_MAX_STEPS || win == nullptr || unit < n_single) {     // wave-uniform
        tile_window_wave<DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, win, n_win, col, sval, P, nnz, unit, lds,
                                    order);
        return;
    }
    if constexpr (STEPS <= PAIR_MAX_STEPS)
        tile_window_pair_wave<DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, win, n_win, col, sval, P, nnz,
                                         n_single + 2 * (unit - n_single), lds);
}

template <int DT, int STEPS>
__global__ __launch_bounds__(BLOCK) void k_tile(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                                const int32_t *__restrict__ vrows,
                                                const int32_t *__restrict__ tile_cols,
                                                const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                const TileWindow *__restrict__ win, int64_t n_win,
                                                const int32_t *__restrict__ col, const float *__restrict__ sval,
                                                float *__restrict__ P, int64_t nnz, int64_t nblocks,
                                                const int32_t *__restrict__ order, int64_t n_single) {
    __shared__ __attribute__((aligned(16))) float win_lds[WAVES_PER_BLOCK][WIN_LDS_FLOATS];
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    tile_unit_wave<DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, win, n_win, n_single, col, sval, P, nnz,
                              blk * WAVES_PER_BLOCK + wave_in_block(), win_lds[wave_in_block()], order);
}

// ---- long rows, well-filled tiles: the four waves of a workgroup split K -----------------------
// A tile of long rows is 16 KB of B (1 KiB rows) for 16 MFMAs: a wavefront that walks tiles alone has
// two of them in flight, fills half the register file with them and still waits for memory most of
// the time, and a launch of a few thousand tiles is two such wavefronts per SIMD.  Here a workgroup
// takes one window of TILE_WINDOW tiles and wave j the j-th quarter of K of all of them: a quarter of
// the registers per tile, all four tiles of the window in flight, four times the wavefronts.  The
// partial 16x16 products meet in LDS (1 KiB per tile and wave); wave j then adds up tile j, scales it
// by S and scatters it from the descriptor's masks, which it loaded at the start.
constexpr int KSPLIT = WAVES_PER_BLOCK;
static_assert(KSPLIT == 4 && TILE_WINDOW == 4, "one finishing wave per tile of a window");
constexpr int KSPLIT_LDS_FLOATS = TILE_WINDOW * KSPLIT * 256;

template <int DT, int STEPS>
__global__ __launch_bounds__(BLOCK) void k_tile_ksplit(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                                       const int32_t *__restrict__ vrows,
                                                       const int32_t *__restrict__ tile_cols,
                                                       const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                       const float *__restrict__ sval, float *__restrict__ P,
                                                       int64_t nblocks, const int32_t *__restrict__ order) {
    static_assert(STEPS % KSPLIT == 0, "K in four equal parts of whole 64-byte steps");
    constexpr int SW = STEPS / KSPLIT;                    // steps of this wave
    __shared__ __attribute__((aligned(16))) float part[KSPLIT_LDS_FLOATS];
    int64_t w = xcd_remap(blockIdx.x, nblocks);
    if (w < 0) return;                                    // whole workgroups leave
    if (order) w = order[w];
    const int64_t t0 = w * TILE_WINDOW;
    if (t0 >= n_tiles) return;
    const int n = (int)(n_tiles - t0 < TILE_WINDOW ? n_tiles - t0 : TILE_WINDOW);
    const int j = wave_in_block();
    const int lane = lane_id();
    const int r16 = lane & 15, q = lane >> 4;        // operand / result layout
    const int lrow = lane >> 2, lunit = lane & 3;    // memory layout: four neighbouring lanes on 64 bytes of a row
    const int to_operand_from = (4 * r16 + q) << 2;
    constexpr uint32_t ROW_UNITS = STEPS * 4;
    const uint4 *__restrict__ Au = (const uint4 *)A + (uint32_t)(j * SW * 4);    // this wave's quarter of every row
    const uint4 *__restrict__ Bu = (const uint4 *)B + (uint32_t)(j * SW * 4);
    auto to_operand = [&](const uint4 &v) {
        uint4 r;
        r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.x);
        r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.y);
        r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.z);
        r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(to_operand_from, (int)v.w);
        return r;
    };
    // first round trip: strip and B rows of every tile, the per-row fields of this wave's own tile
    // (one load each: lane u of every quad asks for tile u, the values are dealt out inside the quad)
    int strip[TILE_WINDOW], bcol[TILE_WINDOW];
    {
        const int64_t t = t0 + (lunit < n ? lunit : n - 1);
        const int st = tiles[t].strip;
        const int bc = tile_cols[t * 16 + lrow];
        strip[0] = __builtin_amdgcn_readlane(st, 0); strip[1] = __builtin_amdgcn_readlane(st, 1);
        strip[2] = __builtin_amdgcn_readlane(st, 2); strip[3] = __builtin_amdgcn_readlane(st, 3);
        bcol[0] = dpp_i32<0x00>(bc); bcol[1] = dpp_i32<0x55>(bc);       // quad_perm: every lane takes lane k of its quad
        bcol[2] = dpp_i32<0xAA>(bc); bcol[3] = dpp_i32<0xFF>(bc);
    }
    const TileDesc *mine = tiles + t0 + (j < n ? j : n - 1);
    const int4 off4 = *(const int4 *)&mine->off[q * 4];
    const uint2 mask2 = *(const uint2 *)&mine->mask[q * 4];
    auto a_rows = [&](int st) {
        int64_t arow = st >= GATHERED_BASE ? (int64_t)vrows[(int64_t)(st - GATHERED_BASE) * 16 + lrow]
                                           : (int64_t)st * 16 + lrow;
        arow = arow < 0 ? 0 : (arow < M ? arow : M - 1);      // missing rows are never in a mask
        return Au + arow * ROW_UNITS + lunit;
    };
    // second round trip: this wave's quarter of the A panel and of all B tiles, the S values of its own tile
    uint4 a[SW], b[TILE_WINDOW][SW];
    {
        const uint4 *src = a_rows(strip[0]);
#pragma unroll
        for (int s = 0; s < SW; ++s) a[s] = src[s * 4];
    }
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k) {
        int64_t brow = bcol[k];
        brow = brow < N ? brow : N - 1;                   // columns past N (and the filler of a short union tile) are in no mask
        const uint4 *src = Bu + brow * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < SW; ++s) b[k][s] = src[s * 4];
    }
    const unsigned int below = (1u << r16) - 1u;
    const int offs[4] = {off4.x, off4.y, off4.z, off4.w};
    const unsigned int masks[4] = {mask2.x & 0xFFFFu, mask2.x >> 16, mask2.y & 0xFFFFu, mask2.y >> 16};
    unsigned int act = 0;
    int pos[4];
    float sv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const bool on = j < n && ((masks[i] >> r16) & 1u);
        act |= on ? (1u << i) : 0u;
        pos[i] = on ? offs[i] + __builtin_popcount(masks[i] & below) : 0;   // (row 4q+i, column r16); entry 0 when absent
        sv[i] = sval[pos[i]];
    }
#pragma unroll
    for (int s = 0; s < SW; ++s) a[s] = to_operand(a[s]);
#pragma unroll
    for (int k = 0; k < TILE_WINDOW; ++k) {
        if (k >= n) break;                                // workgroup-uniform
        if (k > 0 && strip[k] != strip[k - 1]) {          // workgroup-uniform: the window reaches into the next strip
            const uint4 *src = a_rows(strip[k]);
#pragma unroll
            for (int s = 0; s < SW; ++s) a[s] = to_operand(src[s * 4]);
        }
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SW; ++s) {
            const uint4 bo = to_operand(b[k][s]);
            if constexpr (DT == DT_BF16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                              __builtin_bit_cast(bf16x8_t, bo), acc, 0, 0, 0);
            } else if constexpr (DT == DT_F16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a[s]),
                                                             __builtin_bit_cast(half8_t, bo), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].x),
                                                           __builtin_bit_cast(float, bo.x), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].y),
                                                           __builtin_bit_cast(float, bo.y), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].z),
                                                           __builtin_bit_cast(float, bo.z), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].w),
                                                           __builtin_bit_cast(float, bo.w), acc, 0, 0, 0);
            }
        }
        *reinterpret_cast<f32x4_t *>(part + (k * KSPLIT + j) * 256 + lane * 4) = acc;
    }
    __syncthreads();
    if (j < n) {
        f32x4_t sum = *reinterpret_cast<const f32x4_t *>(part + (j * KSPLIT) * 256 + lane * 4);
#pragma unroll
        for (int jj = 1; jj < KSPLIT; ++jj) {
            const f32x4_t v = *reinterpret_cast<const f32x4_t *>(part + (j * KSPLIT + jj) * 256 + lane * 4);
            sum[0] += v[0]; sum[1] += v[1]; sum[2] += v[2]; sum[3] += v[3];
        }
        // result register i is row 4*q+i, column r16
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if ((act >> i) & 1u) P[pos[i]] = sum[i] * sv[i];
    }
}

// Order of the windows for operands that exceed an XCD's L2.  The launch gives every XCD a
// contiguous eighth of the logical windows (xcd_remap); sorted by the key below, that eighth is
// one block of a RB x CB grid over (strip rows, tile columns), RB * CB = 8, walked by finer
// column slices: the XCD keeps its part of A resident and streams through its part of B once,
// instead of touching all of B from every strip (the storage order of the descriptors).
// Counting sort in three launches: histogram, scan of the WINDOW_BINS counters, scatter (the
// order inside a bin is whatever the atomics give; every entry is computed on its own, so the
// result does not depend on it).
constexpr int WINDOW_SLICES = 8;                      // column slices inside a block
constexpr int WINDOW_BINS = NUM_XCD * WINDOW_SLICES;
__device__ __forceinline__ int window_bin(const TileDesc *__restrict__ tiles, int64_t w, int64_t strip_span,
                                          int64_t tile_col_span, int RB, int CB) {
    const int4 h = *reinterpret_cast<const int4 *>(tiles + w * TILE_WINDOW);        // strip, tj, ..
    int64_t strip = h.x >= GATHERED_BASE ? h.x - GATHERED_BASE : h.x;
    strip = strip < strip_span ? strip : strip_span - 1;
    int64_t tj = h.y < 0 ? 0 : h.y;
    tj = tj < tile_col_span ? tj : tile_col_span - 1;
    const int rb = (int)(strip * RB / strip_span);
    const int fine = (int)(tj * (CB * WINDOW_SLICES) / tile_col_span);               // cb * WINDOW_SLICES + slice
    return rb * (CB * WINDOW_SLICES) + fine;
}
__global__ __launch_bounds__(256) void k_window_histogram(const TileDesc *__restrict__ tiles, int64_t n_win,
                                                          int64_t strip_span, int64_t tile_col_span, int RB, int CB,
                                                          unsigned int *__restrict__ bins) {
    const int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (w < n_win) atomicAdd(&bins[window_bin(tiles, w, strip_span, tile_col_span, RB, CB)], 1u);
}
// one workgroup of WINDOW_BINS threads: counts -> start positions (also the scatter's cursors)
__global__ __launch_bounds__(WINDOW_BINS) void k_window_offsets(unsigned int *__restrict__ bins) {
    __shared__ unsigned int v[WINDOW_BINS];
    v[threadIdx.x] = bins[threadIdx.x];
    __syncthreads();
    unsigned int before = 0;
    for (int i = 0; i < (int)threadIdx.x; ++i) before += v[i];
    bins[threadIdx.x] = before;
}
__global__ __launch_bounds__(256) void k_window_scatter(const TileDesc *__restrict__ tiles, int64_t n_win,
                                                        int64_t strip_span, int64_t tile_col_span, int RB, int CB,
                                                        unsigned int *__restrict__ cursors, int32_t *__restrict__ order) {
    const int64_t w = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (w >= n_win) return;
    const unsigned int at = atomicAdd(&cursors[window_bin(tiles, w, strip_span, tile_col_span, RB, CB)], 1u);
    order[at] = (int32_t)w;
}

// AUTO in one launch when a matrix has tiles and rows: logical blocks are dealt out
// evenly between tile blocks (tile_wave), segment-item blocks and short-row blocks,
// so that every XCD gets its share of each.  Kernels of one stream run one after
// the other; two short launches leave the chip half idle twice, one launch does not.
// L must be the full-K, 32-bit-offset layout of a row of STEPS * 64 bytes.
#ifndef SDDMM_FUSED_WAVES
#define SDDMM_FUSED_WAVES 5
#endif
template <class L, int STEPS>
__global__ __launch_bounds__(BLOCK, STEPS <= 2 ? SDDMM_FUSED_WAVES : STEPS == 4 ? 4 : 1) void k_auto_tiles(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                      const int32_t *__restrict__ rowptr,
                                                      const unsigned char *__restrict__ owner,
                                                      const int32_t *__restrict__ col,
                                                      const float *__restrict__ sval, float *__restrict__ P, int M,
                                                      int N, int ts, int rpw, int64_t short_blocks,
                                                      const RowItem *__restrict__ items, int64_t n_items,
                                                      const int32_t *__restrict__ vrows,
                                                      const int32_t *__restrict__ tile_cols,
                                                      const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                      const TileWindow *__restrict__ win, int64_t n_win, int64_t nnz,
                                                      int64_t tile_blocks, int64_t nblocks,
                                                      const int2 *__restrict__ short_list, int64_t n_short_list,
                                                      int longest_first, const int32_t *__restrict__ order,
                                                      int64_t n_single) {
    __shared__ __attribute__((aligned(16))) float win_lds[WAVES_PER_BLOCK][WIN_LDS_FLOATS];
    int64_t tile_block = -1, item_block = -1, short_block = -1;
    if (longest_first) {
        // Workgroups start in the order of their ids, round-robin over the XCDs: on every XCD the
        // tile windows first (the longest wavefronts), then the segment items, then the chunks of
        // the entry list, each XCD with its contiguous eighth of each kind.
        const int x = (int)(blockIdx.x % NUM_XCD);
        int64_t j = blockIdx.x / NUM_XCD;
        const int64_t item_blocks = nblocks - tile_blocks - short_blocks;
        const int64_t t_lo = x * tile_blocks / NUM_XCD, t_n = (x + 1) * tile_blocks / NUM_XCD - t_lo;
        const int64_t i_lo = x * item_blocks / NUM_XCD, i_n = (x + 1) * item_blocks / NUM_XCD - i_lo;
        const int64_t s_lo = x * short_blocks / NUM_XCD, s_n = (x + 1) * short_blocks / NUM_XCD - s_lo;
        if (j < t_n) tile_block = t_lo + j;
        else if ((j -= t_n) < i_n) item_block = i_lo + j;
        else if ((j -= i_n) < s_n) short_block = s_lo + j;
        else return;
    } else {
        const int64_t blk = xcd_remap(blockIdx.x, nblocks);
        if (blk < 0) return;
        const int64_t tiles_before = blk * tile_blocks / nblocks;
        if (((blk + 1) * tile_blocks / nblocks) != tiles_before) {
            tile_block = tiles_before;
        } else {
            const int64_t rb = blk - tiles_before, rest = nblocks - tile_blocks;
            const int64_t item_blocks = rest - short_blocks;
            const int64_t items_before = rb * item_blocks / rest;
            if (((rb + 1) * item_blocks / rest) != items_before) item_block = items_before;
            else short_block = rb - items_before;
        }
    }
    if (tile_block >= 0) {
        tile_unit_wave<L::U::DT, STEPS>(A, B, M, N, vrows, tile_cols, tiles, n_tiles, win, n_win, n_single, col, sval, P,
                                        nnz, tile_block * WAVES_PER_BLOCK + wave_in_block(),
                                        win_lds[wave_in_block()], order);
        return;
    }
    if (item_block >= 0) {
        const int64_t w = item_block * WAVES_PER_BLOCK + wave_in_block();
        if (w >= n_items) return;
        const RowItem it = items[w];
        const int row = __builtin_amdgcn_readfirstlane(it.row);
        const int start = __builtin_amdgcn_readfirstlane(it.start);
        const int end = __builtin_amdgcn_readfirstlane(it.end);
        row_segment_body<L>(A, B, KU, col, sval, P, row, start, end, lane_id());
    } else {
        const int64_t sb = short_block;
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
// ROW PANEL on the matrix cores: 8 consecutive rows with one column list (see
// k_panel_flags).  One wavefront per work item = entries [start,end) of the shared
// list, 16 columns per MFMA accumulator:
//
//     D[c][r] = sum_k B[col_c][k] * A[row0+r][k]      c = 0..15, r = 0..7 (8..15 unused)
//
// The 16 gathered B rows are the "row" operand (lane l: B row of column l&15,
// 16-byte unit 4s + (l>>4) in step s), the 8 A rows of the panel the "column"
// operand, held in registers for the whole item.  Result register i of lane l is
// D[4*(l>>4)+i][l&15]: four consecutive entries of row (l&15).  The column indices
// are read once for the 8 rows, each gathered B unit serves 8 rows.
//
// The vector memory pipeline spends its time per instruction (address cycles for 64
// lanes) and per line segment that neighbouring lanes touch (one cache lookup each),
// not per byte, so memory is accessed in a layout of its own, four neighbouring
// lanes on 64 contiguous bytes, and values change layout inside the wave through
// the LDS crossbar (ds_bpermute: no memory traffic):
//   * B:   load lane l reads gathered row l>>2, unit 4s + (l&3): 16 segments per
//          instruction instead of the 64 a load in operand layout would touch;
//          operand lane (n,q) then takes its unit from load lane 4n+q;
//   * S,P: two groups of 16 columns share one access: lane l reads / writes the four
//          consecutive entries 4(l&7).. (of the 32) of row l>>3 as one 16-byte access
//          (rows start at arbitrary 4-byte offsets; global 16-byte accesses need no
//          more alignment than that): 8 rows x 128 bytes per instruction.  Lanes 8..15
//          of every 16 hold the panel's rows a second time, so the second group's
//          results are already in place there: a select merges the two accumulators,
//          the merged one is moved into the memory layout (lane l takes from result
//          lane 16(l&3) + (l>>3) + 8((l>>2)&1)) and multiplied by S there.
//
// Pipeline: the entries are walked in chunks of 64 = 4 groups of 16 columns.  While
// chunk c computes, the B units and S values of chunk c+1 are in flight (a group is
// re-requested as soon as its registers have been consumed) and the column indices
// of chunk c+2 are being read; every load is issued whatever the position (clamped),
// so the wait counts stay exact and a group only waits for loads issued four groups
// earlier.
//
// fp32 rows of 128 bytes and more use v_mfma_f32_4x4x1_16b_f32 instead of the 16x16x4
// shape, whose accumulator the 8 panel rows fill only by half (fp32 MFMA runs at the rate
// of two plain FMAs per lane, so a half-used 16x16 accumulator is no faster than vector
// FMAs).  The instruction computes 16 independent 4x4 outer products, block b = lanes
// 4b..4b+3:  D_b[i][j] += srcA[lane 4b+i] * srcB[lane 4b+j]  (result register i of lane
// 4b+j).  Blocks are numbered (q, cg): q = k quarter (the 16-byte unit 4s+q of a row, as
// above), cg = four of the 16 gathered columns.  srcB is the gathered B row of column
// 4cg+j -- the operand layout of the 16x16 shape, unchanged.  srcA is the panel: with
// cbsz = 2 the four blocks of one q take srcA from the block that abid names, so the four
// blocks of a q hold four different things -- block cg: panel rows 4(cg&1).. of unit
// 4(2s'+(cg>>1))+q -- and one register covers two steps and both row halves: the panel
// costs STEPS/2 registers of 16 bytes (the 16x16 layout needs STEPS and repeats every
// row).  Every MFMA does 256 useful multiply-adds.  Results: register i of lane (q,cg,j)
// is (row i or 4+i, column 4cg+j), partial over q; v_permlane32_swap and
// v_permlane16_swap add the four k quarters while they deal the row halves and the two
// groups of a pair out to the lanes, a 4x4 transpose inside every quad (two DPP stages)
// turns (register = row, lane = column) into (lane = row, register = column): four
// consecutive entries of a row per lane, which then move to the memory layout as above.
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

template <int ABID>
__device__ __forceinline__ f32x4_t mfma_blocks(float a, float b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 2, ABID, 0);
}
// both row halves of the panel against one component of a gathered unit; AB = 2 * (step parity)
template <int AB>
__device__ __forceinline__ void mfma_blocks_unit(const uint4 &r, const uint4 &b, f32x4_t &lo, f32x4_t &hi) {
    lo = mfma_blocks<AB>(__builtin_bit_cast(float, r.x), __builtin_bit_cast(float, b.x), lo);
    hi = mfma_blocks<AB + 1>(__builtin_bit_cast(float, r.x), __builtin_bit_cast(float, b.x), hi);
    lo = mfma_blocks<AB>(__builtin_bit_cast(float, r.y), __builtin_bit_cast(float, b.y), lo);
    hi = mfma_blocks<AB + 1>(__builtin_bit_cast(float, r.y), __builtin_bit_cast(float, b.y), hi);
    lo = mfma_blocks<AB>(__builtin_bit_cast(float, r.z), __builtin_bit_cast(float, b.z), lo);
    hi = mfma_blocks<AB + 1>(__builtin_bit_cast(float, r.z), __builtin_bit_cast(float, b.z), hi);
    lo = mfma_blocks<AB>(__builtin_bit_cast(float, r.w), __builtin_bit_cast(float, b.w), lo);
    hi = mfma_blocks<AB + 1>(__builtin_bit_cast(float, r.w), __builtin_bit_cast(float, b.w), hi);
}
// a + b where lane l of the result pairs (first, second) as the swap instruction deals them:
// permlane32_swap: lanes 0..31 get first[l] + first[l+32], lanes 32..63 second[l-32] + second[l]
__device__ __forceinline__ float swap32_add(float first, float second) {
    const u32x2_t r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned int, first),
                                                       __builtin_bit_cast(unsigned int, second), false, false);
    // (element values first: a bit cast applied to a vector element expression reads element 0)
    const unsigned int x = r.x, y = r.y;
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
}
// permlane16_swap: even 16-lane rows get first[row] + first[row+1], odd rows second[row-1] + second[row]
__device__ __forceinline__ float swap16_add(float first, float second) {
    const u32x2_t r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(unsigned int, first),
                                                       __builtin_bit_cast(unsigned int, second), false, false);
    const unsigned int x = r.x, y = r.y;
    return __builtin_bit_cast(float, x) + __builtin_bit_cast(float, y);
}
// 4x4 transpose inside every quad of lanes: f[i] of lane j  <->  f[j] of lane i
__device__ __forceinline__ void quad_transpose(float (&f)[4], int lane) {
    const bool b0 = (lane & 1) != 0, b1 = (lane & 2) != 0;
    {
        const float t01 = dpp_f32<DPP_QUAD_XOR1>(b0 ? f[0] : f[1]);
        const float t23 = dpp_f32<DPP_QUAD_XOR1>(b0 ? f[2] : f[3]);
        f[0] = b0 ? t01 : f[0]; f[1] = b0 ? f[1] : t01;
        f[2] = b0 ? t23 : f[2]; f[3] = b0 ? f[3] : t23;
    }
    {
        const float t02 = dpp_f32<DPP_QUAD_XOR2>(b1 ? f[0] : f[2]);
        const float t13 = dpp_f32<DPP_QUAD_XOR2>(b1 ? f[1] : f[3]);
        f[0] = b1 ? t02 : f[0]; f[2] = b1 ? f[2] : t02;
        f[1] = b1 ? t13 : f[1]; f[3] = b1 ? f[3] : t13;
    }
}

// Wavefronts per workgroup: the launch is a few workgroups per CU (one work item per
// 8-row panel), so small workgroups spread more evenly over the CUs; measured 2 % faster
// with 2 than with 4 at rows of 128-256 bytes, 2-5 % slower at 512 bytes.
constexpr int panel_mfma_waves(int steps) { return steps <= 4 ? 2 : 4; }

// FUSED (rows of 128 to 512 bytes in fp32, 64 to 256 bytes in bf16 / fp16): the kernel also adds the panel's part of
//
//     O[row0+r][:] += sum over the item's columns c of P[row0+r][c] * B[col_c][:]
//
// with the same instruction in another role: block b = gathered column b of the group,
// srcA = the P values of rows 4h.. in that column (lane 4b+i: row 4h+i), srcB = the B
// unit as it was loaded (lane 4b+j: components 4j.. of unit 4s+j, no layout change), so
// register i of lane 4b+j of accumulator (h,s,comp) collects O[4h+i][16s+4j+comp] over
// the columns that block b has seen.  The P values of a pair move from the memory layout
// to srcA through a tile of LDS (one 16-byte write, four 4-byte reads per lane).  After
// the last column the 16 blocks are added with lane swaps and row rotations and every
// lane adds 2*STEPS values to O atomically (O is cleared before the launch; a row may
// be cut into several items).  Columns past the end of the item enter with srcB = 0,
// whatever their B rows hold.  16-bit operands: a B unit holds 8 components, widened to fp32 for
// the second product (P and O are fp32 whatever the operands are), so there are 8 accumulators
// per (h, s) and register i of lane 4b+j of accumulator (h,s,comp) collects O[4h+i][32s+8j+comp].
constexpr int DPP_ROW_ROR4 = 0x124, DPP_ROW_ROR8 = 0x128;   // rotation by 4 / 8 lanes inside every row of 16
constexpr int PANEL_TILE_PITCH = 48;                        // floats per row of the P tile: conflict-free 4-byte reads

// waves per SIMD the register allocation aims at: the fused kernel keeps 2 * K accumulators of the
// output rows, K = 16 * STEPS in fp32 and 32 * STEPS in 16 bits (3 waves at K = 32 -- 4 were no
// faster --, 2 at K = 64, measured 89 us against 114 us with 1; at K = 128 the accumulators leave
// room for one)
constexpr int panel_mfma_min_waves(int steps, bool fused, bool half_width = false) {
    const int k = steps * (half_width ? 32 : 16);
    return fused ? (k <= 32 ? 3 : k == 64 ? 2 : 1) : steps == 8 ? 4 : 1;
}

template <int DT, int STEPS, bool FUSED = false>
__global__ __launch_bounds__(panel_mfma_waves(STEPS) * WAVE, panel_mfma_min_waves(STEPS, FUSED, DT != DT_F32)) void k_panel_mfma(const void *__restrict__ A, const void *__restrict__ B,
                                                      const int32_t *__restrict__ rowptr,
                                                      const int32_t *__restrict__ col,
                                                      const float *__restrict__ sval, float *__restrict__ P,
                                                      const RowItem *__restrict__ items, int64_t n_items,
                                                      int64_t nblocks, float *__restrict__ O) {
    static_assert(!FUSED || (DT == DT_F32 ? (STEPS == 2 || STEPS == 4 || STEPS == 8) : (STEPS == 1 || STEPS == 2 || STEPS == 4)),
                  "fused panels: 32, 64 or 128 components per row");
    __shared__ __attribute__((aligned(16))) float p_tiles[FUSED ? panel_mfma_waves(STEPS) : 1][FUSED ? PANEL_ROWS * PANEL_TILE_PITCH : 4];
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t w = blk * panel_mfma_waves(STEPS) + wave_in_block();
    if (w >= n_items) return;
    const RowItem it = items[w];
    const int row0 = __builtin_amdgcn_readfirstlane(it.row);
    const int start = __builtin_amdgcn_readfirstlane(it.start);
    const int end = __builtin_amdgcn_readfirstlane(it.end);
    if (start >= end) return;
    const int lane = lane_id();
    const int n = lane & 15, q = lane >> 4;          // operand / result layout
    const int lrow = lane >> 2, lunit = lane & 3;    // memory layout: row, 16-byte unit inside 64 bytes
    const int to_operand_from = (4 * n + q) << 2;    // ds_bpermute address: operand lane (n,q) <- memory lane 4n+q
    // S/P layout of a pair of groups: row l>>3, 16-byte unit l&7 of the 128 bytes; units 4..7 are the
    // second group's, whose results sit in lanes 8..15 of every 16
    const int prow = lane >> 3, punit = lane & 7;
    // fp32 rows of 128 bytes and more: 4x4 blocks, every multiply-add useful (see above)
    constexpr bool BLOCKS = DT == DT_F32 && STEPS % 2 == 0;
    // the 8 rows of a panel have one length and follow each other in the CSR arrays
    const int rs0 = __builtin_amdgcn_readfirstlane(it.pad);
    const int row_len = __builtin_amdgcn_readfirstlane(rowptr[row0 + 1]) - rs0;
    const int64_t out_row = (int64_t)rs0 + (int64_t)prow * row_len;   // this lane's S/P row starts here
    // ROTATE: the S/P window of a row lags the compute window by `rot` 16-byte units, chosen so
    // that the 128 bytes which the 8 lanes of a row read and write per pair are one whole line of
    // the output array (rows start wherever the CSR arrays put them).  A lane takes unit
    // (punit - rot) mod 8 of every pair; lanes with punit < rot store it one pair later, next to
    // the first units of that pair (`held` keeps it until then), and one more store-only step
    // follows the last pair.  Unrotated accesses straddle two lines each: every line of S is then
    // requested twice and every line of P written in two halves, and both wait in L2 in between.
    constexpr bool ROTATE = !FUSED;
    int rot = 0, src_unit = punit;
    if constexpr (ROTATE) {
        rot = (int)(((((uintptr_t)P) >> 2) + (uint64_t)(out_row + start)) & 31u) >> 2;
        src_unit = (punit - rot) & 7;
    }
    const bool use_now = punit >= rot;
    const bool any_rot = ROTATE && __ballot(rot != 0) != 0;
    const int to_memory_from =
        (BLOCKS ? 32 * (prow >> 2) + 16 * (src_unit >> 2) + 4 * (src_unit & 3) + (prow & 3)
                : 16 * (src_unit & 3) + prow + 8 * (src_unit >> 2)) << 2;
    constexpr int ROW_UNITS = STEPS * 4;
    // groups of 16 columns in flight; rows of 512 bytes and more leave registers for two
    constexpr int GROUPS = STEPS >= 8 ? 2 : 4;
    const uint4 *__restrict__ Au = (const uint4 *)A;
    const uint4 *__restrict__ Bu = (const uint4 *)B;
    constexpr int A_REGS = BLOCKS ? STEPS / 2 : STEPS;
    uint4 a[A_REGS];
    if constexpr (BLOCKS) {
        // block cg of every k quarter: rows 4(cg&1).. of the units 4(2s'+(cg>>1))+q
        const int cg = (lane >> 2) & 3, t = lane & 3;
        const uint4 *src = Au + (int64_t)(row0 + 4 * (cg & 1) + t) * ROW_UNITS + 4 * (cg >> 1) + q;
#pragma unroll
        for (int s2 = 0; s2 < A_REGS; ++s2) a[s2] = src[s2 * 8];
    } else {
        // panel rows: lanes 8..15 of every 16 repeat rows 0..7, their results are not stored
        const uint4 *src = Au + (int64_t)(row0 + (n & 7)) * ROW_UNITS + q;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) a[s] = src[s * 4];
    }
    const int last = end - 1;
    auto cols_of_chunk = [&](int base) {                        // column of entry base + lane (clamped)
        const int e = base + lane < last ? base + lane : last;
        return col[rs0 + e];
    };
    struct Oper {
        uint4 b[STEPS];
    };
    auto load_oper = [&](int cc, int u) {                       // group u of the chunk whose columns are in cc
        Oper o;
        const int c = __shfl(cc, u * 16 + lrow, WAVE);
        const uint4 *src = Bu + (int64_t)c * ROW_UNITS + lunit;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) o.b[s] = src[s * 4];
        return o;
    };
    // The S values of entries g0+4*(punit-rot) .. +3 of this lane's row: one access for the pair of
    // groups that starts at g0.  The window is clamped into the row (rows of a panel hold at
    // least 4 entries); a clamped window is never used: lanes whose four entries are not all
    // inside the item fetch their S values again.  (Requested one chunk ahead of its products;
    // two chunks ahead was measured slower, in a loop 34 against 30 us and cold 53 against 48 us
    // at 128-byte rows: a request that waits for HBM holds its place in the vector memory queue.)
    auto load_s = [&](int g0) {
        int e = g0 + 4 * (punit - rot);
        e = e < row_len - 4 ? e : row_len - 4;
        e = e > 0 ? e : 0;
        return *reinterpret_cast<const F4u *>(sval + out_row + e);
    };
    auto permute4 = [&](int from, uint32_t x, uint32_t y, uint32_t z, uint32_t w_) {
        uint4 r;
        r.x = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)x);
        r.y = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)y);
        r.z = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)z);
        r.w = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)w_);
        return r;
    };
    // 4x4 blocks: both row halves of 16 columns, partial over the k quarters
    auto compute_blocks = [&](const Oper &o, f32x4_t &lo, f32x4_t &hi) {
        lo = f32x4_t{0.f, 0.f, 0.f, 0.f};
        hi = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if constexpr (BLOCKS) {
#pragma unroll
            for (int s2 = 0; s2 < A_REGS; ++s2) {
                {
                    const uint4 b = permute4(to_operand_from, o.b[2 * s2].x, o.b[2 * s2].y, o.b[2 * s2].z, o.b[2 * s2].w);
                    mfma_blocks_unit<0>(a[s2], b, lo, hi);
                    __builtin_amdgcn_sched_group_barrier(0x080, 4, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
                }
                {
                    const uint4 b = permute4(to_operand_from, o.b[2 * s2 + 1].x, o.b[2 * s2 + 1].y, o.b[2 * s2 + 1].z,
                                             o.b[2 * s2 + 1].w);
                    mfma_blocks_unit<2>(a[s2], b, lo, hi);
                    __builtin_amdgcn_sched_group_barrier(0x080, 4, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
                }
            }
        }
    };
    auto compute = [&](const Oper &o) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < (BLOCKS ? 0 : STEPS); ++s) {
            const uint4 b = permute4(to_operand_from, o.b[s].x, o.b[s].y, o.b[s].z, o.b[s].w);
            if constexpr (DT == DT_BF16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, b),
                                                              __builtin_bit_cast(bf16x8_t, a[s]), acc, 0, 0, 0);
            } else if constexpr (DT == DT_F16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, b),
                                                             __builtin_bit_cast(half8_t, a[s]), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, b.x),
                                                           __builtin_bit_cast(float, a[s].x), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, b.y),
                                                           __builtin_bit_cast(float, a[s].y), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, b.z),
                                                           __builtin_bit_cast(float, a[s].z), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, b.w),
                                                           __builtin_bit_cast(float, a[s].w), acc, 0, 0, 0);
                // Order of issue: the four permutes of a step, then its four MFMAs.  Left alone the
                // compiler pairs every MFMA with one permute and a wait for it (16 LDS round trips
                // per 16 columns in the wave's dependency chain instead of 4); whole groups of 8 or
                // 16 permutes ahead of their MFMAs were measured slower than either.
                __builtin_amdgcn_sched_group_barrier(0x080, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
            }
        }
        return acc;
    };
    // FUSED: accumulator (h, s, comp) of the output rows, see above
    constexpr int COMPS = DT == DT_F32 ? 4 : 8;                 // components of a 16-byte unit
    f32x4_t oacc[2][STEPS][COMPS];
    if constexpr (FUSED) {
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int s = 0; s < STEPS; ++s)
#pragma unroll
                for (int k = 0; k < COMPS; ++k) oacc[h][s][k] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    auto fused_accumulate = [&](const Oper &o, float p_lo, float p_hi, int gbase) {
        const bool live = gbase + lrow < end;                    // this block's column belongs to the item
#pragma unroll
        for (int s = 0; s < (FUSED ? STEPS : 0); ++s) {
            const uint4 b = o.b[s];
            const unsigned int ux = live ? b.x : 0u, uy = live ? b.y : 0u, uz = live ? b.z : 0u, uw = live ? b.w : 0u;
            float bv[COMPS];
            if constexpr (DT == DT_F32) {
                bv[0] = __builtin_bit_cast(float, ux); bv[1] = __builtin_bit_cast(float, uy);
                bv[2] = __builtin_bit_cast(float, uz); bv[3] = __builtin_bit_cast(float, uw);
            } else {
                using U16 = std::conditional_t<DT == DT_BF16, UnitBF16x8, UnitF16x8>;
                bv[0] = U16::lo(ux); bv[1] = U16::hi(ux); bv[2] = U16::lo(uy); bv[3] = U16::hi(uy);
                bv[4] = U16::lo(uz); bv[5] = U16::hi(uz); bv[6] = U16::lo(uw); bv[7] = U16::hi(uw);
            }
#pragma unroll
            for (int k = 0; k < COMPS; ++k) {
                oacc[0][s][k] = __builtin_amdgcn_mfma_f32_4x4x1f32(p_lo, bv[k], oacc[0][s][k], 0, 0, 0);
                oacc[1][s][k] = __builtin_amdgcn_mfma_f32_4x4x1f32(p_hi, bv[k], oacc[1][s][k], 0, 0, 0);
            }
        }
    };
    // groups o0 (entries g0..g0+15) and o1 (g0+16..g0+31) of the shared column list
    float held[4] = {0.f, 0.f, 0.f, 0.f};                        // ROTATE: the unit taken from the previous pair
    auto compute_store_pair = [&](const Oper &o0, const Oper &o1, const F4u &sw, int g0) {
        if (g0 >= end + (any_rot ? 32 : 0)) return;              // wave-uniform
        const bool past = g0 >= end;                             // the store-only step after the last pair
        float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 0.f;
        if (past) {
        } else if constexpr (BLOCKS) {
            f32x4_t lo0, hi0, lo1, hi1;
            compute_blocks(o0, lo0, hi0);
            compute_blocks(o1, lo1, hi1);                        // columns clamped past the end: computed, not stored
            // register i of lane (q,cg,j): row i (lo) / 4+i (hi), column 4cg+j of its group, partial
            // over q = (bit 5, bit 4) of the lane.  First swap: the two lane halves add up, the lower
            // keeps rows 0..3, the upper rows 4..7; second swap: the 16-lane rows add up, even rows
            // keep the first group, odd rows the second.  Lane (b5,b4,cg,j), register i is then
            // (row 4 b5 + i, column 16 b4 + 4 cg + j of the pair); the transpose makes it
            // (row 4 b5 + j, columns 16 b4 + 4 cg + i).
            float f[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float g_first = swap32_add(lo0[i], hi0[i]);
                const float g_second = swap32_add(lo1[i], hi1[i]);
                f[i] = swap16_add(g_first, g_second);
            }
            quad_transpose(f, lane);
            r0 = f[0]; r1 = f[1]; r2 = f[2]; r3 = f[3];
        } else {
            const f32x4_t acc0 = compute(o0);
            const f32x4_t acc1 = compute(o1);                    // columns clamped past the end: computed, not stored
            // result lane (n,q) holds entries 4q.. of its group for row n&7: lanes with n < 8 keep
            // the first group's, lanes with n >= 8 the second group's; memory lane l wants row l>>3,
            // entries g0+4(l&7)..
            // (element values first: a bit cast applied to a vector element expression reads element 0)
            const bool second = (n & 8) != 0;
            r0 = second ? acc1[0] : acc0[0]; r1 = second ? acc1[1] : acc0[1];
            r2 = second ? acc1[2] : acc0[2]; r3 = second ? acc1[3] : acc0[3];
        }
        const uint4 m = permute4(to_memory_from, __builtin_bit_cast(uint32_t, r0), __builtin_bit_cast(uint32_t, r1),
                                 __builtin_bit_cast(uint32_t, r2), __builtin_bit_cast(uint32_t, r3));
        float d0 = __builtin_bit_cast(float, m.x), d1 = __builtin_bit_cast(float, m.y);
        float d2 = __builtin_bit_cast(float, m.z), d3 = __builtin_bit_cast(float, m.w);
        if constexpr (ROTATE) {
            const float n0 = d0, n1 = d1, n2 = d2, n3 = d3;
            d0 = use_now ? n0 : held[0]; d1 = use_now ? n1 : held[1];
            d2 = use_now ? n2 : held[2]; d3 = use_now ? n3 : held[3];
            held[0] = n0; held[1] = n1; held[2] = n2; held[3] = n3;
        }
        const int e = g0 + 4 * (punit - rot);
        float p[4] = {0.f, 0.f, 0.f, 0.f};                       // FUSED: the P values, 0 past the end of the item
        if (e < start) {
            // ROTATE, first pair: these lanes' first unit comes with the next pair
        } else if (e + 4 <= end) {
            // four consecutive entries inside the item (so the S window was not clamped)
            F4u out{d0 * sw.x, d1 * sw.y, d2 * sw.z, d3 * sw.w};
            *reinterpret_cast<F4u *>(P + out_row + e) = out;
            p[0] = out.x; p[1] = out.y; p[2] = out.z; p[3] = out.w;
        } else {
            // the item ends inside these four: entry by entry, S values fetched again
            const float d[4] = {d0, d1, d2, d3};
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (e + i < end) {
                    p[i] = d[i] * sval[out_row + e + i];
                    P[out_row + e + i] = p[i];
                }
        }
        if constexpr (FUSED) {
            float *tile = p_tiles[wave_in_block()];
            const f32x4_t pv = {p[0], p[1], p[2], p[3]};
            *reinterpret_cast<f32x4_t *>(tile + prow * PANEL_TILE_PITCH + 4 * punit) = pv;
            wave_lds_order();
            // lane 4b+i: row 4h+i, column b of the first / second group
            const float *src = tile + (lane & 3) * PANEL_TILE_PITCH + lrow;
            const float p0_lo = src[0], p0_hi = src[4 * PANEL_TILE_PITCH];
            const float p1_lo = src[16], p1_hi = src[4 * PANEL_TILE_PITCH + 16];
            wave_lds_order();
            fused_accumulate(o0, p0_lo, p0_hi, g0);
            fused_accumulate(o1, p1_lo, p1_hi, g0 + 16);
        }
    };

    constexpr int CHUNK = GROUPS * 16;                          // columns per loop iteration (<= 64)
    Oper o[GROUPS];
    // Loads complete in issue order and a wait names how many of the most recent ones
    // may still be in flight.  The waits inside the loop must hold on the way in from
    // this prologue too, so the prologue issues its loads in the order the loop does
    // (both column loads first, then the groups in the order they are consumed);
    // otherwise the loop would wait for almost everything it has just requested.
    F4u s_cur[GROUPS / 2];
    const int cc0 = cols_of_chunk(start);
    int cc_nxt = cols_of_chunk(start + CHUNK);                  // columns of the next chunk
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < GROUPS; ++u) {
        o[u] = load_oper(cc0, u);
        if ((u & 1) == 0) s_cur[u / 2] = load_s(start + 16 * u);
        __builtin_amdgcn_sched_barrier(0);
    }
    const int walk_end = end + (any_rot ? 32 : 0);
    for (int base = start; base < walk_end; base += CHUNK) {
        const int cc_nn = cols_of_chunk(base + 2 * CHUNK);
#pragma unroll
        for (int u = 0; u < GROUPS; u += 2) {
            compute_store_pair(o[u], o[u + 1], s_cur[u / 2], base + 16 * u);
            o[u] = load_oper(cc_nxt, u);
            o[u + 1] = load_oper(cc_nxt, u + 1);
            s_cur[u / 2] = load_s(base + CHUNK + 16 * u);
        }
        cc_nxt = cc_nn;
    }
    if constexpr (FUSED) {
        // Register i of lane 4b+j of accumulator (h,s,comp) is O[4h+i][(4s+j) COMPS + comp] over block
        // b's columns.  The swaps add the four rows of 16 lanes while dealing the registers out: row r
        // of the wave keeps register {0,2,1,3}[r]; the rotations add the four blocks of a row.  All
        // four blocks then hold the same 16 sums; block cg adds the ones of components cg (and 4+cg) to O.
        const int r16 = lane >> 4, cg = (lane >> 2) & 3;
        const int orow = row0 + ((r16 & 1) << 1 | (r16 >> 1));
        constexpr int K = STEPS * 4 * COMPS;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
#pragma unroll
                for (int c4 = 0; c4 < COMPS; c4 += 4) {
                    float w4[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const f32x4_t v = oacc[h][s][c4 + k];
                        const float t0 = swap32_add(v[0], v[1]);
                        const float t1 = swap32_add(v[2], v[3]);
                        float x = swap16_add(t0, t1);
                        x += dpp_f32<DPP_ROW_ROR4>(x);
                        x += dpp_f32<DPP_ROW_ROR8>(x);
                        w4[k] = x;
                    }
                    const float mine = cg == 0 ? w4[0] : cg == 1 ? w4[1] : cg == 2 ? w4[2] : w4[3];
                    atomicAdd(O + (int64_t)(orow + 4 * h) * K + (4 * s + (lane & 3)) * COMPS + c4 + cg, mine);
                }
            }
        }
    }
}

}  // namespace sddmm
