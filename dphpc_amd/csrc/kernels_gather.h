// Gather kernels: every stored entry (i,j) of S reads row i of A and row j of B.
//
// Lane layout (all kernels below).  A wavefront works on a "chunk" of up to 64
// consecutive stored entries.  Lane l loads the column index / S value of entry
// l of the chunk and finally stores its P value: plain coalesced 64-wide
// accesses.  For the dot products the 64 lanes are cut into G = 64/LPN groups of
// LPN lanes, LPN being the power of two >= K/ELEMS (capped at 64): at K=32 fp32 a
// group is 8 lanes, each lane owning one 16-byte piece of a row, so a group reads
// one contiguous 128-byte row of B.  In step t group g computes entry t*G+g, i.e.
// a step covers G consecutive entries and a chunk of n entries needs ceil(n/G)
// steps (a short chunk costs proportionally less).  Steps are issued in batches:
// all gathers of a batch are in flight before the first FMA.  Lane (g*LPN+t)
// keeps the group total of step t; one permute at the end brings entry l back to
// lane l.
//
// Per-entry arithmetic is the same everywhere (FMA chain over the lane's pieces
// in k order, then the fixed tree of group_sum), so all strategies built from
// these kernels return bit-identical values.
#pragma once
#include "device_utils.h"

namespace sddmm {

constexpr int BLOCK = 256;                 // 4 wavefronts
constexpr int WAVES_PER_BLOCK = BLOCK / WAVE;

// Accumulates the dot products of up to 64 entries.
//   U, LPN     unit type and lanes per entry
//   WITH_ROWS  true: the A row differs per entry (r holds it per lane);
//              false: `a` already holds this lane's piece of the one A row
template <class U, int LPN, bool WITH_ROWS>
struct ChunkSingle {
    using T = typename U::T;
    static constexpr int G = WAVE / LPN;
    static constexpr int BIG = LPN < 8 ? LPN : 8;
    static constexpr int SMALL = LPN < 2 ? LPN : 2;

    template <int NB>
    static __device__ __forceinline__ void batch(int t0, const T *__restrict__ A, const T *__restrict__ B,
                                                 int KU, int jj, bool lane_on, const T &a, int c, int r,
                                                 int lane, float &out) {
        const int g = lane / LPN, j = lane & (LPN - 1);
        T bf[NB];
        T af[WITH_ROWS ? NB : 1];
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            const int src = ((t0 + u) * G + g) & (WAVE - 1);
            const int cc = __shfl(c, src, WAVE);
            bf[u] = B[(int64_t)cc * KU + jj];
            if constexpr (WITH_ROWS) {
                const int rr = __shfl(r, src, WAVE);
                af[u] = A[(int64_t)rr * KU + jj];
            }
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            float p;
            if constexpr (WITH_ROWS) p = U::dot(af[u], bf[u], 0.f);
            else p = U::dot(a, bf[u], 0.f);
            p = group_sum<LPN>(lane_on ? p : 0.f);
            if (j == t0 + u) out = p;
        }
    }

    // c (and r) must be valid indices in every lane (0 for lanes past the end of
    // the chunk); count = number of entries in the chunk (1..64).
    static __device__ __forceinline__ float run(const T *__restrict__ A, const T *__restrict__ B, int KU,
                                                const T &a, int c, int r, int count, int lane) {
        const int j = lane & (LPN - 1);
        const bool lane_on = j < KU;             // KU < LPN when K/ELEMS is not a power of two
        const int jj = lane_on ? j : 0;
        int steps = (count + G - 1) / G;
        steps = steps < LPN ? steps : LPN;
        float out = 0.f;
        int t0 = 0;
        for (; t0 + BIG <= steps; t0 += BIG) batch<BIG>(t0, A, B, KU, jj, lane_on, a, c, r, lane, out);
        for (; t0 < steps; t0 += SMALL) batch<SMALL>(t0, A, B, KU, jj, lane_on, a, c, r, lane, out);
        // entry l = t*G+g was kept by lane g*LPN+t
        return __shfl(out, (lane % G) * LPN + lane / G, WAVE);
    }
};

// K too long for one piece per lane (more than 64 units per row): one entry per
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

// ---------------------------------------------------------------------------
// FLAT: entries [0,nnz) in order, row index per entry read from rowidx (the COO
// row array, or the expansion of rowptr built by the plan).  Perfectly balanced
// whatever the row lengths are; A pieces are gathered per entry like B pieces
// (L1/L2 hits while the row does not change).
template <class U, int LPN, bool SINGLE>
__global__ __launch_bounds__(BLOCK) void k_flat(const typename U::T *__restrict__ A,
                                                const typename U::T *__restrict__ B, int KU,
                                                const int32_t *__restrict__ rowidx,
                                                const int32_t *__restrict__ col,
                                                const float *__restrict__ sval,
                                                float *__restrict__ P, int64_t nnz,
                                                int chunks_per_wave, int64_t nblocks) {
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int lane = lane_id();
    const int64_t wave = blk * WAVES_PER_BLOCK + wave_in_block();
    int64_t base = wave * (int64_t)chunks_per_wave * WAVE;
    for (int ch = 0; ch < chunks_per_wave && base < nnz; ++ch, base += WAVE) {
        const int64_t n = base + lane;
        const bool valid = n < nnz;
        const int c = valid ? col[n] : 0;
        const int r = valid ? rowidx[n] : 0;
        const float s = valid ? sval[n] : 0.f;
        const int64_t left = nnz - base;
        const int count = left < WAVE ? (int)left : WAVE;
        float res;
        if constexpr (SINGLE) res = ChunkSingle<U, LPN, true>::run(A, B, KU, U::zero(), c, r, count, lane);
        else res = chunk_long<U>(A, B, KU, c, r, count, lane);
        if (valid) P[n] = res * s;
    }
}

// ---------------------------------------------------------------------------
// ROW_WAVE: one wavefront per work item = a segment [start,end) of one row.
// With items == nullptr item w is the whole row w.  The lane's piece of the A
// row stays in a register for the whole segment; no row index is read.
struct RowItem {
    int32_t row;
    int32_t start;
    int32_t end;
    int32_t pad;
};

template <class U, int LPN, bool SINGLE>
__global__ __launch_bounds__(BLOCK) void k_row_wave(const typename U::T *__restrict__ A,
                                                    const typename U::T *__restrict__ B, int KU,
                                                    const int32_t *__restrict__ rowptr,
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
    if (start >= end) return;
    const int lane = lane_id();
    const int j = lane & (LPN - 1);
    typename U::T a = U::zero();
    if constexpr (SINGLE) { if (j < KU) a = A[(int64_t)row * KU + j]; }
    for (int base = start; base < end; base += WAVE) {
        const int n = base + lane;
        const bool valid = n < end;
        const int c = valid ? col[n] : 0;
        const float s = valid ? sval[n] : 0.f;
        const int left = end - base;
        const int count = left < WAVE ? left : WAVE;
        float res;
        if constexpr (SINGLE) res = ChunkSingle<U, LPN, false>::run(A, B, KU, a, c, 0, count, lane);
        else res = chunk_long<U>(A, B, KU, c, row, count, lane);
        if (valid) P[n] = res * s;
    }
}

// ---------------------------------------------------------------------------
// EXACT: one lane per entry, k ascending, separate fp32 multiply and add (the
// translation unit is compiled with -ffp-contract=off), then the multiply by S:
// the operation sequence of the CPU loop, hence bit-identical to it.
template <bool IS_BF16>
__global__ __launch_bounds__(BLOCK) void k_exact(const void *__restrict__ Av, const void *__restrict__ Bv,
                                                 int K, const int32_t *__restrict__ rowidx,
                                                 const int32_t *__restrict__ col,
                                                 const float *__restrict__ sval,
                                                 float *__restrict__ P, int64_t nnz) {
    const int64_t n = (int64_t)blockIdx.x * BLOCK + threadIdx.x;
    if (n >= nnz) return;
    const int64_t r = rowidx[n], c = col[n];
    float acc = 0.f;
    if constexpr (IS_BF16) {
        const uint16_t *a = (const uint16_t *)Av + r * K;
        const uint16_t *b = (const uint16_t *)Bv + c * K;
        for (int k = 0; k < K; ++k) {
            const float x = __builtin_bit_cast(float, (uint32_t)a[k] << 16);
            const float y = __builtin_bit_cast(float, (uint32_t)b[k] << 16);
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
