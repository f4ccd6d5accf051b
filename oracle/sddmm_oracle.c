/*
 * CPU oracle for SDDMM  P = S o (A * B^T)  -- TEST INFRASTRUCTURE ONLY.
 *
 * Plain-C restatement of the reference's CPU path.  Nothing in the product
 * (the HIP library, its C++ host adapter, the Python binding) links, loads or
 * calls this file; only tests/, __graft_entry__.smoke() and the cpu_baseline
 * leg of bench.py do, and only as the checker / the reported CPU baseline.
 *
 * What each function follows in the reference (paths under src/):
 *   oracle_sddmm_csr_f32      competitors/cpu/cpu_basic.hpp:18-36
 *   oracle_sddmm_coo_f32      competitors/cpu/cpu_basic.hpp:38-51
 *   oracle_sddmm_csr_f32_omp  same loop as :18-36, rows split over threads
 *                             (rows are independent, per-entry arithmetic unchanged)
 *   oracle_triplets_sort_unique, oracle_csr_from_triplets, oracle_coo_from_triplets
 *                             matrices/CSR.hpp:169-194, matrices/COO.hpp:27-49,
 *                             matrices/triplet.h:12-19
 *   oracle_coo_from_csr       matrices/COO.hpp:55-74
 *   oracle_dispatch           matrices/CSR.hpp:196-264
 *   oracle_density            matrices/CSR.hpp:157-159 (in 64-bit; the reference
 *                             multiplies rows*cols in int and overflows above 46340^2)
 *   oracle_compare            no counterpart (a comparator, not arithmetic): the value
 *                             test of oracle.check_values over large arrays, held to
 *                             the numpy version by tests/test_oracle.py
 *   oracle_fusedmm_csr_f32/_f64   no counterpart: the reference stops at P.  SpMM of
 *                             the SDDMM result with B, written in the reference's
 *                             style (multiply, then add, entries in storage order);
 *                             pinned by numpy identities only (tests/test_oracle.py)
 *
 * Arithmetic contract of the reference loop: fp32 multiply, then fp32 add into
 * the running value, k ascending, then one fp32 multiply by the S value.  The
 * reference is built -O3 for baseline x86-64 (no FMA instructions exist there),
 * so this file must be compiled with -ffp-contract=off.
 *
 * Pinning status: every function here is pinned by tests/test_oracle.py against
 * closed forms of the reference's own test cases (tests/matrix_test.cc:124-182,
 * 354-425, 460-477; benchmark/dataset.hpp:183-204), against numpy identities
 * (all-ones S == GEMM, K=1 outer product, brute-force dense), and against
 * oracle/_ref (the reference's own headers compiled in place) where that is built.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- SDDMM, CSR (cpu_basic.hpp:18-36) ---------------------------------- */
void oracle_sddmm_csr_f32(int M, int K,
                          const int32_t *rowptr, const int32_t *col, const float *sval,
                          const float *A, const float *B, float *P)
{
    for (int i = 0; i < M; i++) {
        const float *a = A + (size_t)i * (size_t)K;
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++) {
            const float *b = B + (size_t)col[j] * (size_t)K;
            P[j] = 0.0f;                          /* accumulates in the output slot, as the reference does */
            for (int k = 0; k < K; k++)
                P[j] += a[k] * b[k];
        }
    }
    /* second pass of the reference: scale by S */
    for (int i = 0; i < M; i++)
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++)
            P[j] = P[j] * sval[j];
}

/* Same arithmetic per entry, rows split over OpenMP threads. */
void oracle_sddmm_csr_f32_omp(int M, int K,
                              const int32_t *rowptr, const int32_t *col, const float *sval,
                              const float *A, const float *B, float *P, int threads)
{
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#else
    (void)threads;
#endif
#pragma omp parallel for schedule(dynamic, 64)
    for (int i = 0; i < M; i++) {
        const float *a = A + (size_t)i * (size_t)K;
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++) {
            const float *b = B + (size_t)col[j] * (size_t)K;
            float acc = 0.0f;
            for (int k = 0; k < K; k++) {
                float prod = a[k] * b[k];
                acc = acc + prod;
            }
            P[j] = acc * sval[j];
        }
    }
}

int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---- SDDMM, COO (cpu_basic.hpp:38-51) ---------------------------------- */
void oracle_sddmm_coo_f32(int64_t nnz, int K,
                          const int32_t *row, const int32_t *col, const float *sval,
                          const float *A, const float *B, float *P)
{
    for (int64_t i = 0; i < nnz; i++) {
        const float *a = A + (size_t)row[i] * (size_t)K;
        const float *b = B + (size_t)col[i] * (size_t)K;
        float acc = 0.0f;
        for (int k = 0; k < K; k++) {
            float prod = a[k] * b[k];
            acc = acc + prod;
        }
        P[i] = acc;
    }
    for (int64_t i = 0; i < nnz; i++)
        P[i] = P[i] * sval[i];
}

/* ---- error-analysis helpers (no counterpart in the reference) ----------
 * dot64[j]  = S_j * sum_k a_k*b_k        accumulated in double
 * mag64[j]  = |S_j| * sum_k |a_k*b_k|    the cancellation-free magnitude a
 *                                        tolerance floor is scaled with        */
void oracle_sddmm_csr_f64(int M, int K,
                          const int32_t *rowptr, const int32_t *col, const float *sval,
                          const float *A, const float *B, double *dot64, double *mag64)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int i = 0; i < M; i++) {
        const float *a = A + (size_t)i * (size_t)K;
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++) {
            const float *b = B + (size_t)col[j] * (size_t)K;
            double acc = 0.0, mag = 0.0;
            for (int k = 0; k < K; k++) {
                double p = (double)a[k] * (double)b[k];
                acc += p;
                mag += fabs(p);
            }
            if (dot64) dot64[j] = acc * (double)sval[j];
            if (mag64) mag64[j] = mag * fabs((double)sval[j]);
        }
    }
}

/* ---- SDDMM followed by SpMM over the same pattern (no counterpart) ------
 * P as oracle_sddmm_csr_f32; O[i,:] = sum_j P[i,j] * B[col_j,:], fp32 multiply then
 * fp32 add, entries in storage order. */
void oracle_fusedmm_csr_f32(int M, int K,
                            const int32_t *rowptr, const int32_t *col, const float *sval,
                            const float *A, const float *B, float *P, float *O)
{
    oracle_sddmm_csr_f32(M, K, rowptr, col, sval, A, B, P);
    for (int i = 0; i < M; i++) {
        float *o = O + (size_t)i * (size_t)K;
        for (int k = 0; k < K; k++) o[k] = 0.0f;
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++) {
            const float *b = B + (size_t)col[j] * (size_t)K;
            for (int k = 0; k < K; k++)
                o[k] += P[j] * b[k];
        }
    }
}

/* O64 = the same in double from the double SDDMM values; mag64[i,k] = sum_j
 * |S_j| (sum_k' |a b|) |b_k|, the cancellation-free magnitude for a tolerance floor */
void oracle_fusedmm_csr_f64(int M, int K,
                            const int32_t *rowptr, const int32_t *col, const float *sval,
                            const float *A, const float *B, double *O64, double *mag64)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (int i = 0; i < M; i++) {
        const float *a = A + (size_t)i * (size_t)K;
        double *o = O64 + (size_t)i * (size_t)K, *m = mag64 + (size_t)i * (size_t)K;
        for (int k = 0; k < K; k++) { o[k] = 0.0; m[k] = 0.0; }
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++) {
            const float *b = B + (size_t)col[j] * (size_t)K;
            double acc = 0.0, mag = 0.0;
            for (int k = 0; k < K; k++) {
                double p = (double)a[k] * (double)b[k];
                acc += p;
                mag += fabs(p);
            }
            acc *= (double)sval[j];
            mag *= fabs((double)sval[j]);
            for (int k = 0; k < K; k++) {
                o[k] += acc * (double)b[k];
                m[k] += mag * fabs((double)b[k]);
            }
        }
    }
}

/* ---- containers -------------------------------------------------------- */
typedef struct { int32_t row, col; float val; int64_t seq; } trip_t;

static int trip_cmp(const void *pa, const void *pb)
{
    const trip_t *a = (const trip_t *)pa, *b = (const trip_t *)pb;
    if (a->row != b->row) return a->row < b->row ? -1 : 1;
    if (a->col != b->col) return a->col < b->col ? -1 : 1;
    /* the reference's std::sort leaves the order of equal (row,col) keys
       unspecified; this restatement fixes it to input order */
    return a->seq < b->seq ? -1 : (a->seq > b->seq);
}

/* Sort by (row,col) (triplet.h:16-19) and drop an element when it equals its
 * kept predecessor under triplet.h:12-14: same row, same col AND both values
 * non-zero (so an explicit zero never merges).  In place; returns the new count. */
int64_t oracle_triplets_sort_unique(int64_t n, int32_t *row, int32_t *col, float *val)
{
    if (n <= 0) return 0;
    trip_t *t = (trip_t *)malloc((size_t)n * sizeof(trip_t));
    for (int64_t i = 0; i < n; i++) { t[i].row = row[i]; t[i].col = col[i]; t[i].val = val[i]; t[i].seq = i; }
    qsort(t, (size_t)n, sizeof(trip_t), trip_cmp);
    int64_t w = 0;
    for (int64_t i = 0; i < n; i++) {
        if (w > 0 && t[w - 1].row == t[i].row && t[w - 1].col == t[i].col &&
            t[w - 1].val != 0.0f && t[i].val != 0.0f)
            continue;                              /* std::unique keeps the first of a run */
        t[w++] = t[i];
    }
    for (int64_t i = 0; i < w; i++) { row[i] = t[i].row; col[i] = t[i].col; val[i] = t[i].val; }
    free(t);
    return w;
}

/* CSR.hpp:169-194: after sort/unique, walk rows 0..rows-1 and consume the
 * triplets whose row equals i.  A triplet whose row is outside [0,rows) stops
 * the walk exactly as in the reference (everything after it is dropped).
 * Inputs are overwritten by the sorted/unique triplets; returns nnz stored. */
int64_t oracle_csr_from_triplets(int rows, int64_t n, int32_t *row, int32_t *col, float *val,
                                 int32_t *rowptr /* rows+1 */, int32_t *out_col, float *out_val)
{
    int64_t m = oracle_triplets_sort_unique(n, row, col, val);
    int64_t idx = 0;
    for (int i = 0; i < rows; i++) {
        rowptr[i] = (int32_t)idx;
        while (idx < m && row[idx] == i) { out_val[idx] = val[idx]; out_col[idx] = col[idx]; idx++; }
    }
    rowptr[rows] = (int32_t)idx;
    return idx;
}

/* COO.hpp:27-49: sorted, de-duplicated triplets kept as three parallel arrays. */
int64_t oracle_coo_from_triplets(int64_t n, int32_t *row, int32_t *col, float *val)
{
    return oracle_triplets_sort_unique(n, row, col, val);
}

/* COO.hpp:55-74 */
void oracle_coo_from_csr(int rows, const int32_t *rowptr, int32_t *out_row)
{
    for (int i = 0; i < rows; i++)
        for (int32_t j = rowptr[i]; j < rowptr[i + 1]; j++) out_row[j] = i;
}

double oracle_density(int rows, int cols, int64_t nnz)
{
    return (double)nnz / ((double)rows * (double)cols);
}

/* ---- nnz-balanced contiguous row partition (CSR.hpp:196-264) ----------- */
static int dispatch_test(const int32_t *sizes, int64_t ns, int64_t val, int parts)
{
    int64_t mx = 0;
    for (int64_t i = 0; i < ns; i++) if (sizes[i] > mx) mx = sizes[i];
    if (mx > val) return 0;
    int64_t cnt = 1, sum = 0;
    for (int64_t i = 0; i < ns; i++) {
        sum += sizes[i];
        if (sum > val) { cnt++; sum = sizes[i]; }
    }
    return cnt <= parts;
}

/* start_idx must hold parts+1 ints.  rows must be a multiple of stride. Returns
 * the number of entries written (parts+1), or -1 on bad arguments. */
int oracle_dispatch(int rows, const int32_t *rowptr, int parts, int stride, int32_t *start_idx)
{
    if (rows <= 0 || parts <= 0 || stride <= 0 || rows % stride) return -1;
    int64_t ns = rows / stride;
    int32_t *sizes = (int32_t *)malloc((size_t)ns * sizeof(int32_t));
    for (int64_t s = 0; s < ns; s++) sizes[s] = rowptr[(s + 1) * stride] - rowptr[s * stride];
    int64_t lo = 1, hi = rowptr[rows], seg = 0;
    while (lo <= hi) {                              /* smallest feasible maximum load */
        int64_t mid = (lo + hi) / 2;
        if (dispatch_test(sizes, ns, mid, parts)) { seg = mid; hi = mid - 1; }
        else lo = mid + 1;
    }
    int w = 0;
    int64_t cur = 0;
    start_idx[w++] = 0;
    for (int64_t i = 0; i < ns; i++) {
        cur += sizes[i];
        if (cur > seg) {
            if (w > parts) { free(sizes); return -1; }
            start_idx[w++] = (int32_t)(i * stride);
            cur = sizes[i];
        }
    }
    while (w <= parts) start_idx[w++] = rows;       /* idle parts */
    free(sizes);
    return w;
}

/* ---- comparator --------------------------------------------------------- */
/* ratio[i] = 0 when got[i] == ref[i], else |got-ref| / (rtol * max(|ref|, floor*mag[i]))
 * (mag may be NULL); a NaN ratio counts as infinite.  Returns the largest ratio and
 * the first position that attains it: the test passes when it is <= 1. */
double oracle_compare(int64_t n, const float *got, const float *ref, const double *mag,
                      double rtol, double floor_, int64_t *worst_at)
{
    double worst = -1.0;
    int64_t at = -1;
#pragma omp parallel
    {
        double w = -1.0;
        int64_t a = -1;
#pragma omp for schedule(static) nowait
        for (int64_t i = 0; i < n; i++) {
            const double g = (double)got[i], r = (double)ref[i];
            double scale = fabs(r);
            if (mag && floor_ * mag[i] > scale) scale = floor_ * mag[i];
            const double err = fabs(g - r);
            double ratio = err == 0.0 ? 0.0 : err / (rtol * scale);
            if (isnan(ratio)) ratio = INFINITY;
            if (ratio > w) { w = ratio; a = i; }
        }
#pragma omp critical
        {
            if (w > worst || (w == worst && a >= 0 && (at < 0 || a < at))) { worst = w; at = a; }
        }
    }
    if (worst_at) *worst_at = at;
    return n > 0 ? worst : 0.0;
}
