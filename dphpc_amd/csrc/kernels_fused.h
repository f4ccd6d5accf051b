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
    struct Ent { int n, c; float s; bool valid; };
    auto entry = [&](int base) {                      // entry base + lane of the item (clamped past its end)
        Ent x;
        x.n = base + lane;
        x.valid = x.n < end;
        x.c = col[x.n < last ? x.n : last];
        x.s = x.valid ? sval[x.n] : 0.f;              // entries past the end contribute p = 0
        return x;
    };
    // steps t0 .. t0+NB-1 of a chunk: group g gathers the B rows of entries t*G+g
    auto gather = [&](const Ent &x, int t0, T (&bf)[NB][UPL]) {
        const Off_t boff = (Off_t)x.c * rb;
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
    };
    auto consume = [&](const Ent &x, int t0, int steps, const T (&bf)[NB][UPL], float &out) {
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
            const bool live = __shfl((int)x.valid, src, WAVE) != 0;
            p = group_sum<LPN>(p) * __shfl(x.s, src, WAVE);   // every lane takes part in the lane exchange
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
    };
    auto steps_of = [&](int base) {
        const int count = end - base < WAVE ? end - base : WAVE;
        const int st = (count + G - 1) / G;
        return st < LPN ? st : LPN;
    };
    // entry l = t*G+g was kept by lane g*LPN+t
    auto store_p = [&](const Ent &x, float out) {
        const float res = __shfl(out, (lane % G) * LPN + lane / G, WAVE);
        if (x.valid) P[x.n] = res;
    };
    // Batches of NB steps, LPN / NB of them per chunk of 64 entries: the gathers of the next batch (of
    // the next chunk after a chunk's last) and the indices of the chunk after the next are in flight
    // while a batch is multiplied, one round trip per batch instead of one per batch and one per chunk.
    constexpr int BPC = LPN / NB;
    static_assert(LPN % NB == 0, "whole batches per chunk");
    // (Rows of more than one unit per lane keep one batch in flight: the second buffer costs them a
    // third of their wavefronts per SIMD, 171 against 153 us on banded rows of 256 bytes.)
    constexpr bool AHEAD = UPL == 1;
    Ent cur = entry(start);
    T bcur[NB][UPL];
    if constexpr (AHEAD) gather(cur, 0, bcur);
    Ent nxt = entry(start + WAVE);
    for (int base = start; base < end; base += WAVE) {
        const int steps = steps_of(base);
        const bool more = base + WAVE < end;
        const Ent after = entry(base + 2 * WAVE);
        float out = 0.f;
#pragma unroll
        for (int bq = 0; bq < BPC; ++bq) {
            const int t0 = bq * NB;
            if (t0 >= steps) break;                           // wave-uniform
            if constexpr (AHEAD) {
                T bnxt[NB][UPL];
                if (bq + 1 < BPC && t0 + NB < steps) gather(cur, t0 + NB, bnxt);
                else if (more) gather(nxt, 0, bnxt);
                consume(cur, t0, steps, bcur, out);
#pragma unroll
                for (int q = 0; q < NB; ++q)
#pragma unroll
                    for (int i = 0; i < UPL; ++i) bcur[q][i] = bnxt[q][i];
            } else {
                gather(cur, t0, bcur);
                consume(cur, t0, steps, bcur, out);
            }
        }
        store_p(cur, out);
        cur = nxt;
        nxt = after;
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
// (panel_owner[row] == 2, when the array is given) to the panel kernel: those rows count
// as empty here and get a row of zeros, which the kernels launched after this one add to.
// Every row below M gets its output row written, so O needs no clearing before the launch.
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
    struct Ent { int at, c; float s; bool has; };
    auto entry = [&](int t0) {                        // entry t0 + j of this group's row
        Ent x;
        const int e = t0 + j;
        x.has = e < len;
        x.at = x.has ? rs + e : (len > 0 ? rs + len - 1 : 0);   // a valid position in every lane
        x.c = col[x.at];
        x.s = x.has ? sval[x.at] : 0.f;
        return x;
    };
    auto gather = [&](const Ent &x, int q0, T (&bf)[NB][UPL]) {
        const Off_t boff = (Off_t)x.c * rb;
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
    };
    auto consume = [&](const Ent &x, int q0, int steps, const T (&bf)[NB][UPL], float &out) {
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
            const bool live = __shfl((int)x.has, src, WAVE) != 0;
            p = group_sum<LPN>(p) * __shfl(x.s, src, WAVE);   // every lane takes part in the lane exchange
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
    };
    // Batches of NB steps, LPN / NB of them per LPN entries of a row: the gathers of the next batch and
    // the indices of the entries after the next LPN are in flight while a batch is multiplied.
    constexpr int BPC = LPN / NB;
    static_assert(LPN % NB == 0, "whole batches per LPN entries");
    constexpr bool AHEAD = UPL <= 2;                 // (rows of more units per lane: measured the same either way)
    Ent cur = entry(0);
    T bcur[NB][UPL];
    if constexpr (AHEAD) {
        if (longest > 0) gather(cur, 0, bcur);                // wave-uniform
    }
    Ent nxt = entry(LPN);
    for (int t0 = 0; t0 < longest; t0 += LPN) {
        const int steps = longest - t0 < LPN ? longest - t0 : LPN;
        const bool more = t0 + LPN < longest;
        const Ent after = entry(t0 + 2 * LPN);
        float out = 0.f;
#pragma unroll
        for (int bq = 0; bq < BPC; ++bq) {
            const int q0 = bq * NB;
            if (q0 >= steps) break;                           // wave-uniform
            if constexpr (AHEAD) {
                T bnxt[NB][UPL];
                if (bq + 1 < BPC && q0 + NB < steps) gather(cur, q0 + NB, bnxt);
                else if (more) gather(nxt, 0, bnxt);
                consume(cur, q0, steps, bcur, out);
#pragma unroll
                for (int q = 0; q < NB; ++q)
#pragma unroll
                    for (int i = 0; i < UPL; ++i) bcur[q][i] = bnxt[q][i];
            } else {
                gather(cur, q0, bcur);
                consume(cur, q0, steps, bcur, out);
            }
        }
        if (cur.has) P[cur.at] = out;
        cur = nxt;
        nxt = after;
    }
    if (row < M) {                                    // (the accumulators of a row left to other kernels are zero)
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

// The same rows as k_fusedmm_rows when their lengths differ a lot (a power-law graph: most
// rows hold one to three entries, a few dozens): there a lane group that waits for the longest
// of a wavefront's 64/LPN rows idles four steps out of five.  Here a wavefront takes 64
// consecutive rows, numbers their entries across the rows (prefix sum of the lengths, kept in
// LDS with the rows' CSR positions) and deals whole rows out to its lane groups so that every
// group gets about an equal share of the entries.  A group walks its entries LPN at a time: lane
// j finds the row of its entry by bisection over the prefix sums, loads column index and S
// value; step q then takes entry q with all lanes of the group, gathers the entry's A row with
// its B row (the rows change inside a group, as in the flat kernel), and the group's partial
// output row is written whenever the row changes.  Rows without entries of their own (empty,
// left to other kernels) get zeros, as in k_fusedmm_rows.
template <class L>
__global__ __launch_bounds__(BLOCK) void k_fusedmm_rows_balanced(const void *__restrict__ A, const void *__restrict__ B,
                                                                 int KU, const int32_t *__restrict__ rowptr,
                                                                 const int32_t *__restrict__ col,
                                                                 const float *__restrict__ sval, float *__restrict__ P,
                                                                 float *__restrict__ O, int M, int max_len,
                                                                 int64_t nblocks,
                                                                 const unsigned char *__restrict__ panel_owner) {
    using U = typename L::U;
    using T = typename U::T;
    constexpr int E = U::ELEMS;
    using C = Chunk<U, L::LPN, L::UPL, L::FULLK, false, L::WIDE>;
    using Off_t = typename C::O;
    constexpr int LPN = L::LPN, UPL = L::UPL, G = WAVE / LPN;
    constexpr int NB = C::BIG > 4 ? 4 : C::BIG;       // A and B rows of a batch of steps in flight together
    __shared__ int pre_all[WAVES_PER_BLOCK][WAVE], pos_all[WAVES_PER_BLOCK][WAVE];
    const int64_t blk = xcd_remap(blockIdx.x, nblocks);
    if (blk < 0) return;
    const int64_t r0 = (blk * WAVES_PER_BLOCK + wave_in_block()) * WAVE;
    if (r0 >= M) return;
    const int lane = lane_id();
    const int g = lane / LPN, j = lane & (LPN - 1);
    int *pre = pre_all[wave_in_block()], *pos = pos_all[wave_in_block()];
    // lane l: row r0 + l
    const bool inside = r0 + lane < M;
    int rs = 0, len = 0;
    if (inside) {
        rs = rowptr[r0 + lane];
        len = rowptr[r0 + lane + 1] - rs;
        if (len > max_len || (panel_owner && panel_owner[r0 + lane] == 2)) len = 0;
    }
    int incl = len;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const int up = __shfl_up(incl, o, WAVE);
        if (lane >= o) incl += up;
    }
    const int total = __builtin_amdgcn_readlane(incl, WAVE - 1);
    pre[lane] = incl - len;
    pos[lane] = rs;
    wave_lds_order();
    // whole rows per group: group gg starts at the first row whose prefix reaches gg/G of the entries
    int b_lo = 0, b_hi = WAVE;
#pragma unroll
    for (int gg = 1; gg < G; ++gg) {
        const int target = (int)((int64_t)gg * total / G);
        const int first = __popcll(__ballot(incl - len < target));
        if (g == gg) b_lo = first;
        if (g + 1 == gg) b_hi = first;
    }
    const int v_lo = b_lo < WAVE ? pre[b_lo] : total, v_hi = b_hi < WAVE ? pre[b_hi] : total;
    int longest = v_hi - v_lo;
#pragma unroll
    for (int o = LPN; o < WAVE; o <<= 1) {
        const int other = __shfl_xor(longest, o, WAVE);
        longest = other > longest ? other : longest;
    }
    longest = __builtin_amdgcn_readfirstlane(longest);
    const Off_t rb = (Off_t)KU * (Off_t)sizeof(T);
    // rows with nothing of their own: zeros (lane group g takes rows g, g + G, ..)
    {
        const unsigned long long empty = __ballot(inside && len == 0);
#pragma unroll
        for (int k = 0; k < WAVE / G; ++k) {
            const int rr = k * G + g;
            if (!((empty >> rr) & 1ull)) continue;
            float *orow = O + (r0 + rr) * (int64_t)KU * E;
#pragma unroll
            for (int i = 0; i < UPL; ++i) {
                const int u = j + i * LPN;
                if (!C::unit_on(j, i, KU)) continue;
#pragma unroll
                for (int e = 0; e < E; e += 4)
                    *reinterpret_cast<float4 *>(orow + E * u + e) = make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
    }
    float acc[UPL][E];
#pragma unroll
    for (int i = 0; i < UPL; ++i)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[i][e] = 0.f;
    int cur_row = -1;                                 // the row the group's partial sums belong to (the same in its lanes)
    auto flush = [&](bool on) {
        if (!on) return;
        float *orow = O + (r0 + cur_row) * (int64_t)KU * E;
#pragma unroll
        for (int i = 0; i < UPL; ++i) {
            const int u = j + i * LPN;
            if (!C::unit_on(j, i, KU)) continue;
#pragma unroll
            for (int e = 0; e < E; e += 4)
                *reinterpret_cast<float4 *>(orow + E * u + e) =
                    make_float4(acc[i][e], acc[i][e + 1], acc[i][e + 2], acc[i][e + 3]);
        }
    };
    for (int t0 = 0; t0 < longest; t0 += LPN) {
        const int v = v_lo + t0 + j;
        const bool has = v < v_hi;
        // the row of entry v: the last row whose prefix does not exceed v (rows without entries
        // share their prefix with the row after them and are never the last such row)
        const int vv = has ? v : (v_hi > v_lo ? v_hi - 1 : 0);
        int lo = 0, hi = WAVE;
#pragma unroll
        for (int it = 0; it < 6; ++it) {
            const int mid = (lo + hi) >> 1;
            if (pre[mid] <= vv) lo = mid; else hi = mid;
        }
        const int row = v_hi > v_lo ? lo : 0;                            // (a group without entries: row 0, position 0)
        const int at = v_hi > v_lo ? pos[row] + (vv - pre[row]) : 0;      // a valid position in every lane
        const int c = col[at];
        const float s = has ? sval[at] : 0.f;
        const Off_t boff = (Off_t)c * rb, aoff = (Off_t)(r0 + row) * rb;
        const int steps = longest - t0 < LPN ? longest - t0 : LPN;
        float out = 0.f;
        for (int q0 = 0; q0 < steps; q0 += NB) {
            T bf[NB][UPL], af[NB][UPL];
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                const int src = g * LPN + ((q0 + q) & (LPN - 1));
                const Off_t bo = shfl_off<Off_t>(boff, src), ao = shfl_off<Off_t>(aoff, src);
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    const int u = C::unit_on(j, i, KU) ? j + i * LPN : 0;
                    bf[q][i] = load_at<T, Off_t>(B, bo + (Off_t)(u * (int)sizeof(T)));
                    af[q][i] = load_at<T, Off_t>(A, ao + (Off_t)(u * (int)sizeof(T)));
                }
            }
#pragma unroll
            for (int q = 0; q < NB; ++q) {
                if (q0 + q >= steps) break;               // wave-uniform
                const int src = g * LPN + ((q0 + q) & (LPN - 1));
                const bool live = __shfl((int)has, src, WAVE) != 0;
                const int row_q = __shfl(row, src, WAVE);
                const bool change = live && row_q != cur_row;
                flush(change && cur_row >= 0);
                cur_row = change ? row_q : cur_row;
                float p = 0.f;
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    const float d = U::dot(af[q][i], bf[q][i], p);
                    p = C::unit_on(j, i, KU) ? d : p;
                }
                // a step past the end of the group's entries works on a clamped position: it must leave
                // the output row alone whatever that position's B row holds (0 * inf is not 0)
                p = group_sum<LPN>(p) * __shfl(s, src, WAVE);     // every lane takes part in the lane exchange
                p = live ? p : 0.f;
#pragma unroll
                for (int i = 0; i < UPL; ++i) {
                    float next[E];
#pragma unroll
                    for (int e = 0; e < E; ++e) next[e] = change ? 0.f : acc[i][e];
                    U::axpy(p, bf[q][i], next);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[i][e] = live ? next[e] : acc[i][e];
                }
                if (j == q0 + q) out = p;
            }
        }
        if (has) P[at] = out;
    }
    flush(cur_row >= 0);
}

}  // namespace sddmm
