// Structure kernels of the plan phase: validation, CSR<->COO index expansion,
// row statistics.  Everything that looks at S's pattern runs here, on the
// device; the host reads back only the small PlanCounters block.
#pragma once
#include "device_utils.h"

namespace sddmm {

struct PlanCounters {
    unsigned int bad_pattern;      // != 0: malformed CSR/COO
    unsigned int coo_unsorted;     // != 0: COO rows not non-decreasing
    unsigned int max_len;          // longest row
    unsigned int pad;
    unsigned long long rows_nonempty;
    unsigned long long rows_short, rows_medium, rows_long;
    unsigned long long nnz_short, nnz_medium, nnz_long;
    unsigned long long n_items;    // work items of the wave-per-segment kernel
    unsigned long long spare[6];
};

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

// rowptr[0]==0, rowptr[M]==nnz, non-decreasing; also counts non-empty rows and the
// longest row.  One lane per row.
__global__ __launch_bounds__(256) void k_check_rowptr(const int32_t *__restrict__ rowptr, int M,
                                                      int64_t nnz, PlanCounters *pc) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned int bad = 0, len = 0;
    if (i < M) {
        const int32_t s = rowptr[i], e = rowptr[i + 1];
        if (e < s || s < 0) bad = 1; else len = (unsigned int)(e - s);
        if (i == 0 && s != 0) bad = 1;
        if (i == M - 1 && (int64_t)e != nnz) bad = 1;
    }
    const unsigned long long ne = wave_sum_u64(len > 0 ? 1ull : 0ull);
    const unsigned int mx = wave_max_u32(len);
    const unsigned long long anybad = __ballot(bad != 0);
    if (lane_id() == 0) {
        if (ne) atomicAdd(&pc->rows_nonempty, ne);
        if (mx) atomicMax(&pc->max_len, mx);
        if (anybad) atomicOr(&pc->bad_pattern, 1u);
    }
}

// every column index in [0,N)
__global__ __launch_bounds__(256) void k_check_index(const int32_t *__restrict__ idx, int64_t n,
                                                     int bound, PlanCounters *pc) {
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
// whole wavefront.
__global__ __launch_bounds__(256) void k_expand_rows(const int32_t *__restrict__ rowptr, int M,
                                                     int32_t *__restrict__ rowidx) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int lane = lane_id();
    int32_t s = 0, e = 0;
    if (i < M) { s = rowptr[i]; e = rowptr[i + 1]; }
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
                                                          PlanCounters *pc) {
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
