// SDDMM followed by SpMM over the same pattern ("FusedMM"):
//
//     P[i,j] = S[i,j] * <A[i,:], B[j,:]>          (what the SDDMM kernels compute)
//     O[i,:] = sum over stored (i,j) of P[i,j] * B[j,:]
//
// The step that consumes an SDDMM result in the applications the reference names
// (attention-like updates in graph learning); the reference itself stops at P.
// The gathered B row of an entry is used twice while it sits in registers, so the
// second product costs no memory traffic beyond the M x K output.  A and B may be fp32,
// bf16 or fp16 (16-byte units of 4 or 8 elements); P and O are fp32.
//
// k_fusedmm: one wavefront per work item = entries [start,end) of one row (rows longer
// than FUSED_ROW_MAX entries; shorter ones go to k_fusedmm_rows), in the lane layout
// of the gather kernels: groups of LPN lanes, lane j of a group holds units
// j, j+LPN, ... of the A row, of the entry's B row and of the group's partial output
// row.  After the last entry the partial rows of the 64/LPN groups are added with
// lane permutes; group 0 writes the output row, or adds it atomically when the row
// was split into several items (O is cleared before the launch).
#pragma once
#include "kernels_gather.h"

namespace sddmm {

constexpr int FUSED_ROW_MAX = 64;   // rows up to this length: one row per lane group

template <class L>
__global__ __launch_bounds__(BLOCK) void k_fusedmm(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                   const int32_t *__restrict__ rowptr,
                                                   const int32_t *__restrict__ col,
                                                   const float *__restrict__ sval, float *__restrict__ P,
                                                   float *__restrict__ O, const RowItem *__restrict__ items,
                                                   int64_t n_items, int64_t nblocks) {
    using U = typename L::U;
    using T = typename U::T;                          // 16 bytes: 4 fp32 or 8 bf16 / fp16
    constexpr int E = U::ELEMS;
    using C = Chunk<U, L::LPN, L::UPL, L::FULLK, false, L::WIDE>;
    using Off_t = typename C::O;
    constexpr int LPN = L::LPN, UPL = L::UPL, G = WAVE / LPN;
    constexpr int NB = C::BIG;                        // steps whose gathers are in flight together
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t w = blk * WAVES_PER_BLOCK + wave_in_block();
    if (w >= n_items) return;
    const RowItem it = items[w];
    const int row = __builtin_amdgcn_readfirstlane(it.row);
    const int start = __builtin_amdgcn_readfirstlane(it.start);
    const int end = __builtin_amdgcn_readfirstlane(it.end);
    if (start >= end) return;
    const int lane = lane_id();
    const int g = lane / LPN, j = lane & (LPN - 1);
    const Off_t rb = (Off_t)KU * (Off_t)sizeof(T);
    const typename C::Areg a = C::load_a(A, (Off_t)row * rb, j, KU);
    float acc[UPL][E];                                // the lane's units of the output row, fp32
#pragma unroll
    for (int i = 0; i < UPL; ++i)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[i][e] = 0.f;
    const int last = end - 1;
    for (int base = start; base < end; base += WAVE) {
        const int n = base + lane;
        const bool valid = n < end;
        const int c = col[n < last ? n : last];
        const float s = valid ? sval[n] : 0.f;        // entries past the end contribute p = 0
        const Off_t boff = (Off_t)c * rb;
        const int count = end - base < WAVE ? end - base : WAVE;
        int steps = (count + G - 1) / G;
        steps = steps < LPN ? steps : LPN;
        float out = 0.f;
        for (int t0 = 0; t0 < steps; t0 += NB) {
            T bf[NB][UPL];
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                const int src = ((t0 + q) * G + g) & (WAVE - 1);
                const Off_t bo = shfl_off<Off_t>(boff, src);
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    const int u = C::unit_on(j, i, KU) ? j + i * LPN : 0;
                    bf[q][i] = load_at<T, Off_t>(B, bo + (Off_t)(u * (int)sizeof(T)));
                }
            }
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                if (t0 + q >= steps) break;               // wave-uniform
                const int src = ((t0 + q) * G + g) & (WAVE - 1);
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    const float d = U::dot(a.u[i], bf[q][i], p);
                    p = C::unit_on(j, i, KU) ? d : p;
                }
                // a step past the end of the row works on a clamped position: it must leave the
                // output row alone whatever that position's B row holds (0 * inf is not 0)
                const bool live = __shfl((int)valid, src, WAVE) != 0;
                p = group_sum<LPN>(p) * __shfl(s, src, WAVE);     // every lane takes part in the lane exchange
                p = live ? p : 0.f;
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    float next[E];
#pragma unroll
                    for (int e = 0; e < E; ++e) next[e] = acc[i][e];
                    U::axpy(p, bf[q][i], next);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[i][e] = live ? next[e] : acc[i][e];
                }
                if (j == t0 + q) out = p;
            }
        }
        // entry l = t*G+g was kept by lane g*LPN+t
        const float res = __shfl(out, (lane % G) * LPN + lane / G, WAVE);
        if (valid) P[n] = res;
    }
    // add the partial output rows of the G groups: lanes with the same j
#pragma unroll
    for (int off = LPN; off < WAVE; off <<= 1) {
#pragma unroll
        for (int i = 0; i < UPL; ++i)
#pragma unroll
            for (int e = 0; e < E; ++e) acc[i][e] += __shfl_xor(acc[i][e], off, WAVE);
    }
    if (g == 0) {
        const bool whole_row = start == rowptr[row] && end == rowptr[row + 1];
        float *orow = O + (int64_t)row * KU * E;
#pragma unroll
        for (int i = 0; i < UPL; ++i) {
            const int u = j + i * LPN;
            if (!C::unit_on(j, i, KU)) continue;
            if (whole_row) {
#pragma unroll
                for (int e = 0; e < E; e += 4)
                    *reinterpret_cast<float4 *>(orow + E * u + e) =
                        make_float4(acc[i][e], acc[i][e + 1], acc[i][e + 2], acc[i][e + 3]);
            } else {
#pragma unroll
                for (int e = 0; e < E; ++e) atomicAdd(orow + E * u + e, acc[i][e]);
            }
        }
    }
}

// Rows of at most max_len entries, one row per lane group: a wavefront takes 64/LPN
// consecutive rows, group g walks row r0+g.  Lane j of a group reads column index and
// S value of entry t0+j, so LPN entries of each row are gathered back to back; the
// P value of entry t0+j ends up in lane j, and the output row needs no reduction
// across groups.  Longer rows are left to k_fusedmm and the rows of 8-row panels
// (panel_owner[row] == 2, when the array is given) to the panel kernel (they count as
// empty here); every other row, empty ones included, gets its output row written.
template <class L>
__global__ __launch_bounds__(BLOCK) void k_fusedmm_rows(const void *__restrict__ A, const void *__restrict__ B, int KU,
                                                        const int32_t *__restrict__ rowptr,
                                                        const int32_t *__restrict__ col,
                                                        const float *__restrict__ sval, float *__restrict__ P,
                                                        float *__restrict__ O, int M, int max_len, int64_t nblocks,
                                                        const unsigned char *__restrict__ panel_owner) {
    using U = typename L::U;
    using T = typename U::T;
    constexpr int E = U::ELEMS;
    using C = Chunk<U, L::LPN, L::UPL, L::FULLK, false, L::WIDE>;
    using Off_t = typename C::O;
    constexpr int LPN = L::LPN, UPL = L::UPL, G = WAVE / LPN;
    constexpr int NB = C::BIG;
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t r0 = (blk * WAVES_PER_BLOCK + wave_in_block()) * G;
    if (r0 >= M) return;
    const int lane = lane_id();
    const int g = lane / LPN, j = lane & (LPN - 1);
    const int64_t row = r0 + g;
    int rs = 0, len = 0;
    bool mine = false;
    if (row < M) {
        rs = rowptr[row];
        len = rowptr[row + 1] - rs;
        mine = len <= max_len && !(panel_owner && panel_owner[row] == 2);
        if (!mine) len = 0;
    }
    int longest = len;
    for (int off = LPN; off < WAVE; off <<= 1) {
        const int o = __shfl_xor(longest, off, WAVE);
        longest = o > longest ? o : longest;
    }
    longest = __builtin_amdgcn_readfirstlane(longest);
    const Off_t rb = (Off_t)KU * (Off_t)sizeof(T);
    const typename C::Areg a = C::load_a(A, (Off_t)(row < M ? row : 0) * rb, j, KU);
    float acc[UPL][E];                                // the lane's units of the output row, fp32
#pragma unroll
    for (int i = 0; i < UPL; ++i)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[i][e] = 0.f;
    for (int t0 = 0; t0 < longest; t0 += LPN) {
        const int e = t0 + j;
        const bool has = e < len;
        const int at = has ? rs + e : (len > 0 ? rs + len - 1 : 0);   // a valid position in every lane
        const int c = col[at];
        const float s = has ? sval[at] : 0.f;
        const Off_t boff = (Off_t)c * rb;
        const int steps = longest - t0 < LPN ? longest - t0 : LPN;
        float out = 0.f;
        for (int q0 = 0; q0 < steps; q0 += NB) {
            T bf[NB][UPL];
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                const int src = g * LPN + ((q0 + q) & (LPN - 1));
                const Off_t bo = shfl_off<Off_t>(boff, src);
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    const int u = C::unit_on(j, i, KU) ? j + i * LPN : 0;
                    bf[q][i] = load_at<T, Off_t>(B, bo + (Off_t)(u * (int)sizeof(T)));
                }
            }
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                if (q0 + q >= steps) break;               // wave-uniform
                const int src = g * LPN + ((q0 + q) & (LPN - 1));
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    const float d = U::dot(a.u[i], bf[q][i], p);
                    p = C::unit_on(j, i, KU) ? d : p;
                }
                // a step past the end of the row works on a clamped position: it must leave the
                // output row alone whatever that position's B row holds (0 * inf is not 0)
                const bool live = __shfl((int)has, src, WAVE) != 0;
                p = group_sum<LPN>(p) * __shfl(s, src, WAVE);     // every lane takes part in the lane exchange
                p = live ? p : 0.f;
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    float next[E];
#pragma unroll
                    for (int e = 0; e < E; ++e) next[e] = acc[i][e];
                    U::axpy(p, bf[q][i], next);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[i][e] = live ? next[e] : acc[i][e];
                }
                if (j == q0 + q) out = p;
            }
        }
        if (has) P[at] = out;
    }
    if (mine) {
        float *orow = O + row * KU * E;
#pragma unroll
        for (int i = 0; i < UPL; ++i) {
            const int u = j + i * LPN;
            if (!C::unit_on(j, i, KU)) continue;
#pragma unroll
            for (int e = 0; e < E; e += 4)
                *reinterpret_cast<float4 *>(orow + E * u + e) =
                    make_float4(acc[i][e], acc[i][e + 1], acc[i][e + 2], acc[i][e + 3]);
        }
    }
}

}  // namespace sddmm
