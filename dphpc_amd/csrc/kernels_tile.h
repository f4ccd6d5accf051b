// Dense-tile path: 16-row strips of S whose 16x16 tiles are well filled are
// computed on the matrix cores, one MFMA accumulator per tile, instead of one
// gathered B row per stored entry.
//
//   * a strip is rows [16*ti, 16*ti+16); a tile is the strip's entries whose
//     column lies in [16*tj, 16*tj+16);
//   * the classifier (k_tile_count / k_tile_fill, plan phase, device only) walks
//     the sorted column lists of the 16 rows of a strip in step and emits one
//     TileDesc per non-empty tile: for every row the CSR position of its first
//     entry inside the tile and a 16-bit mask of the columns present;
//   * a strip goes to this path as a whole (then every one of its entries is
//     computed here, sparse tiles included) or not at all, so the gather kernels
//     and this one never share a row;
//   * k_tile computes the full 16x16 product A[strip rows] * B[tile cols]^T with
//     fp32 accumulation (bf16: v_mfma_f32_16x16x32_bf16, fp32: v_mfma_f32_16x16x4_f32,
//     both exact products of the stored inputs), multiplies by the S values and
//     writes only the positions the masks name -- P keeps S's order.
//
// The B tile costs 16 rows per tile whatever its fill, a gathered entry costs one
// row each: the tile path moves fewer bytes once a tile holds more than 16
// entries, and far fewer at the 25-100 % fill it is used for.
#pragma once
#include "device_utils.h"
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

// pass 1: tiles and entries per strip; a strip qualifies when all its rows are
// sorted and it holds at least min_fill entries per tile on average.
// strip_ntiles[s] = number of tiles (0: strip stays on the gather kernels).
__global__ __launch_bounds__(256) void k_tile_count(const int32_t *__restrict__ rowptr,
                                                    const int32_t *__restrict__ col, int M, int64_t n_strips,
                                                    int min_fill, unsigned int *__restrict__ strip_ntiles,
                                                    unsigned char *__restrict__ owner8, DevCounters *pc) {
    const int64_t strip = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int sub = threadIdx.x & 15;
    if (strip >= n_strips) return;   // whole 16-lane rows leave together
    // entries of the strip, known from rowptr alone: the walk can stop as soon as the
    // strip has more tiles than that many entries could fill to the threshold
    const int64_t r_lo = strip * 16, r_hi = r_lo + 16 < M ? r_lo + 16 : M;
    const int64_t strip_entries = (int64_t)rowptr[r_hi] - (int64_t)rowptr[r_lo];
    const int64_t max_tiles = strip_entries / min_fill;
    int tiles = 0, entries = 0;
    const bool sorted = walk_strip(rowptr, col, M, strip, sub, [&](int, int, unsigned int mask) {
        ++tiles;
        entries += __builtin_popcount(mask);
        return (int64_t)tiles <= max_tiles;
    });
    const int all_entries = sum16(entries);
    const int unsorted = sum16(sorted ? 0 : 1);
    const bool take = unsorted == 0 && tiles > 0 && (int64_t)tiles <= max_tiles &&
                      (int64_t)all_entries >= (int64_t)min_fill * tiles;
    if (sub == 0) {
        strip_ntiles[strip] = take ? (unsigned int)tiles : 0u;
        if (take) {
            owner8[2 * strip] = 1;         // both 8-row halves (the array is padded to an even length)
            owner8[2 * strip + 1] = 1;
            spread_add(pc, K_TILES, (unsigned long long)tiles);
            spread_add(pc, K_NNZ_TILES, (unsigned long long)all_entries);
        }
    }
}

// pass 2 (after the exclusive scan of strip_ntiles into strip_off): descriptors
__global__ __launch_bounds__(256) void k_tile_fill(const int32_t *__restrict__ rowptr,
                                                   const int32_t *__restrict__ col, int M, int64_t n_strips,
                                                   const unsigned int *__restrict__ strip_ntiles,
                                                   const unsigned int *__restrict__ strip_off,
                                                   TileDesc *__restrict__ tiles) {
    const int64_t strip = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 4;
    const int sub = threadIdx.x & 15;
    if (strip >= n_strips) return;
    if (strip_ntiles[strip] == 0) return;
    int64_t at = strip_off[strip];
    (void)walk_strip(rowptr, col, M, strip, sub, [&](int tj, int first, unsigned int mask) {
        TileDesc *d = tiles + at;
        d->off[sub] = first;
        d->mask[sub] = (uint16_t)mask;
        if (sub == 0) { d->strip = (int32_t)strip; d->tj = tj; d->pad[0] = 0; d->pad[1] = 0; }
        ++at;
        return true;
    });
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
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

// One wavefront computes `tiles_per_wave` consecutive tiles.  Operand layout of
// both MFMA shapes used: lane l supplies row (l & 15) of its operand and the k
// positions selected by (l >> 4); the result register i of lane l is row
// 4*(l >> 4) + i, column (l & 15).  A and B are read in 16-byte units: in load
// step s lane l reads unit 4*s + (l >> 4) of its row, so the four lane groups
// cover 64 contiguous bytes of each of 16 rows per instruction; which k positions
// end up in which MFMA does not matter as long as A and B agree.
// STEPS = row bytes / 64.
//
// Software pipeline, three tiles deep, every load unconditional so that the wait
// counts stay exact (loads return in issue order):
//   iteration t issues   B rows + S values of tile t+1   (needs descriptor t+1)
//                        descriptor of tile t+2
//   and then computes    MFMAs of tile t, scale, scatter (operands landed during t-1)
// The A panel of the current strip stays in registers and is reloaded only when
// the strip changes (a wave-uniform branch placed before the iteration's loads).
template <bool BF16, int STEPS>
__global__ __launch_bounds__(BLOCK) void k_tile(const void *__restrict__ A, const void *__restrict__ B, int M, int N,
                                                const TileDesc *__restrict__ tiles, int64_t n_tiles,
                                                int tiles_per_wave, const float *__restrict__ sval,
                                                float *__restrict__ P, int64_t nblocks) {
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t w = blk * WAVES_PER_BLOCK + wave_in_block();
    int64_t t = w * tiles_per_wave;
    if (t >= n_tiles) return;
    int64_t t_end = t + tiles_per_wave;
    t_end = t_end < n_tiles ? t_end : n_tiles;
    const int64_t t_last = t_end - 1;
    const int lane = lane_id();
    const int r16 = lane & 15, q = lane >> 4;
    constexpr uint32_t ROW_UNITS = STEPS * 4;
    const uint4 *__restrict__ Au = (const uint4 *)A;
    const uint4 *__restrict__ Bu = (const uint4 *)B;
    const unsigned int below = (1u << r16) - 1u;

    struct Desc {
        int strip, tj;
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
        r.tj = d->tj;
        r.off = *(const int4 *)&d->off[q * 4];
        r.mask = *(const uint2 *)&d->mask[q * 4];
        return r;
    };
    auto load_oper = [&](const Desc &d) {
        Oper o;
        int64_t brow = (int64_t)d.tj * 16 + r16;
        brow = brow < N ? brow : N - 1;   // columns past N are never in a mask
        const uint4 *src = Bu + brow * ROW_UNITS + q;
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
            int64_t arow = (int64_t)strip * 16 + r16;
            arow = arow < M ? arow : M - 1;   // rows past M are never in a mask
            const uint4 *src = Au + arow * ROW_UNITS + q;
#pragma unroll
            for (int s = 0; s < STEPS; ++s) a[s] = src[s * 4];
        }
        const Oper o_nxt = load_oper(d_nxt);
        const Desc d_nn = load_desc(t + 2);
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            if constexpr (BF16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a[s]),
                                                              __builtin_bit_cast(bf16x8_t, o_cur.b[s]), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].x),
                                                           __builtin_bit_cast(float, o_cur.b[s].x), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].y),
                                                           __builtin_bit_cast(float, o_cur.b[s].y), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].z),
                                                           __builtin_bit_cast(float, o_cur.b[s].z), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, a[s].w),
                                                           __builtin_bit_cast(float, o_cur.b[s].w), acc, 0, 0, 0);
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
// D[4*(l>>4)+i][l&15]: four CONSECUTIVE entries of row (l&15), so S values and P
// move as one 16-byte access per lane (rows start at arbitrary 4-byte offsets;
// global 16-byte accesses need no more alignment than that).  The column indices
// are read once for the 8 rows, each gathered B unit serves 8 rows.
// Pipeline: the entries are walked in chunks of 64 = 4 groups of 16 columns.  While
// chunk c computes, the B units and S values of chunk c+1 are in flight (a group is
// re-requested as soon as its registers have been consumed) and the column indices
// of chunk c+2 are being read; every load is unconditional (clamped), so the wait
// counts stay exact and a group only ever waits for loads issued four groups earlier.
struct __attribute__((packed, aligned(4))) F4u { float x, y, z, w; };

template <bool BF16, int STEPS>
__global__ __launch_bounds__(BLOCK) void k_panel_mfma(const void *__restrict__ A, const void *__restrict__ B,
                                                      const int32_t *__restrict__ rowptr,
                                                      const int32_t *__restrict__ col,
                                                      const float *__restrict__ sval, float *__restrict__ P,
                                                      const RowItem *__restrict__ items, int64_t n_items,
                                                      int64_t nblocks) {
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
    const int n = lane & 15, q = lane >> 4;
    constexpr int ROW_UNITS = STEPS * 4;
    // groups of 16 columns in flight; 1, 2 and 4 measured the same (47-50 us on the
    // FEM shape at K=32): the kernel is not bound by its own prefetch depth
    constexpr int GROUPS = 4;
    const uint4 *__restrict__ Au = (const uint4 *)A;
    const uint4 *__restrict__ Bu = (const uint4 *)B;
    // panel rows: lanes 8..15 of every 16 repeat rows 0..7, their results are not stored
    uint4 a[STEPS];
    {
        const uint4 *src = Au + (int64_t)(row0 + (n & 7)) * ROW_UNITS + q;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) a[s] = src[s * 4];
    }
    // the 8 rows of a panel have one length and follow each other in the CSR arrays
    const int rs0 = __builtin_amdgcn_readfirstlane(it.pad);
    const int row_len = __builtin_amdgcn_readfirstlane(rowptr[row0 + 1]) - rs0;
    const int64_t out_row = (int64_t)rs0 + (int64_t)(n & 7) * row_len;   // this lane's output row starts here
    const int last = end - 1;
    auto cols_of_chunk = [&](int base) {                        // column of entry base + lane (clamped)
        const int e = base + lane < last ? base + lane : last;
        return col[rs0 + e];
    };
    struct Oper {
        uint4 b[STEPS];
        F4u s;
    };
    auto load_oper = [&](int c, int g0) {
        Oper o;
        const uint4 *src = Bu + (int64_t)c * ROW_UNITS + q;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) o.b[s] = src[s * 4];
        // S values of entries g0+4q .. g0+4q+3 of this lane's row.  The window is clamped
        // into the row (rows of a panel hold at least 4 entries); a clamped window is
        // only ever read for the tail group, which fetches its S values again.
        const int e = g0 + 4 * q < row_len - 4 ? g0 + 4 * q : row_len - 4;
        o.s = *reinterpret_cast<const F4u *>(sval + out_row + e);
        return o;
    };
    auto compute_store = [&](const Oper &o, int g0) {
        if (g0 >= end) return;                                   // wave-uniform
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            if constexpr (BF16) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, o.b[s]),
                                                              __builtin_bit_cast(bf16x8_t, a[s]), acc, 0, 0, 0);
            } else {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, o.b[s].x),
                                                           __builtin_bit_cast(float, a[s].x), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, o.b[s].y),
                                                           __builtin_bit_cast(float, a[s].y), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, o.b[s].z),
                                                           __builtin_bit_cast(float, a[s].z), acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(__builtin_bit_cast(float, o.b[s].w),
                                                           __builtin_bit_cast(float, a[s].w), acc, 0, 0, 0);
            }
        }
        if (n < 8) {
            const int e = g0 + 4 * q;
            if (g0 + 16 <= end) {
                // full group: four consecutive entries per lane
                F4u out{acc[0] * o.s.x, acc[1] * o.s.y, acc[2] * o.s.z, acc[3] * o.s.w};
                *reinterpret_cast<F4u *>(P + out_row + e) = out;
            } else {
                // tail group: the S values were read from a clamped window, fetch them again
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (e + i < end) P[out_row + e + i] = acc[i] * sval[out_row + e + i];
            }
        }
    };

    constexpr int CHUNK = GROUPS * 16;                          // columns per loop iteration (<= 64)
    Oper o[GROUPS];
    {
        const int cc0 = cols_of_chunk(start);
#pragma unroll
        for (int u = 0; u < GROUPS; ++u) o[u] = load_oper(__shfl(cc0, u * 16 + n, WAVE), start + 16 * u);
    }
    int cc_nxt = cols_of_chunk(start + CHUNK);                  // columns of the next chunk
    for (int base = start; base < end; base += CHUNK) {
        const int cc_nn = cols_of_chunk(base + 2 * CHUNK);
#pragma unroll
        for (int u = 0; u < GROUPS; ++u) {
            compute_store(o[u], base + 16 * u);
            o[u] = load_oper(__shfl(cc_nxt, u * 16 + n, WAVE), base + CHUNK + 16 * u);
        }
        cc_nxt = cc_nn;
    }
}

}  // namespace sddmm
