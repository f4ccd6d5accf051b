/*
 * C-ABI wrapper around the REFERENCE's own headers, compiled where they lie
 * (-I/root/reference/src).  TEST INFRASTRUCTURE ONLY: it validates
 * oracle/sddmm_oracle.c and may serve as the CPU baseline (kind "reference").
 * No reference source is copied here; this file only calls into
 *   competitors/cpu/cpu_basic.hpp  (CPUBasic<float>::run_csr / run_coo)
 *   matrices/{CSR,COO,Dense}.hpp   (constructors, conversions, _dispatch)
 * Output goes to oracle/_ref/ only (see oracle/Makefile).
 */
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include "matrices/matrices.h"
#include "competitors/cpu/cpu_basic.hpp"

namespace {
Dense<float> make_dense(int rows, int cols, const float *p)
{
    std::vector<std::vector<float>> m((size_t)rows, std::vector<float>((size_t)cols));
    for (int r = 0; r < rows; r++) std::memcpy(m[(size_t)r].data(), p + (size_t)r * cols, sizeof(float) * (size_t)cols);
    return Dense<float>(m);
}
std::vector<Triplet<float>> make_triplets(int64_t n, const int32_t *row, const int32_t *col, const float *val)
{
    std::vector<Triplet<float>> t((size_t)n);
    for (int64_t i = 0; i < n; i++) t[(size_t)i] = Triplet<float>{row[i], col[i], val[i]};
    return t;
}
}

extern "C" {

/* S given as already-sorted unique triplets (any order is accepted; the
 * reference constructor sorts).  P_out receives CSR-ordered values; returns nnz. */
int64_t ref_cpu_basic_csr(int M, int N, int K, int64_t n, const int32_t *row, const int32_t *col,
                          const float *val, const float *A, const float *B,
                          int32_t *rowptr_out, int32_t *col_out, float *P_out)
{
    Dense<float> dA = make_dense(M, K, A), dB = make_dense(N, K, B);
    CSR<float> S(M, N, make_triplets(n, row, col, val));
    CSR<float> P(S);
    P.clearValues();
    Competitors::CPUBasic<float> c;
    c.run_csr(dA, dB, S, P);
    const size_t nnz = P.getValues().size();
    std::memcpy(P_out, P.getValues().data(), nnz * sizeof(float));
    if (rowptr_out) std::memcpy(rowptr_out, S.getRowPositions().data(), sizeof(int32_t) * (size_t)(M + 1));
    if (col_out) std::memcpy(col_out, S.getColPositions().data(), sizeof(int32_t) * nnz);
    return (int64_t)nnz;
}

int64_t ref_cpu_basic_coo(int M, int N, int K, int64_t n, const int32_t *row, const int32_t *col,
                          const float *val, const float *A, const float *B,
                          int32_t *row_out, int32_t *col_out, float *sval_out, float *P_out)
{
    Dense<float> dA = make_dense(M, K, A), dB = make_dense(N, K, B);
    COO<float> S(M, N, make_triplets(n, row, col, val));
    COO<float> P(S);
    P.clearValues();
    Competitors::CPUBasic<float> c;
    c.run_coo(dA, dB, S, P);
    const size_t nnz = P.getValues().size();
    std::memcpy(P_out, P.getValues().data(), nnz * sizeof(float));
    if (row_out) std::memcpy(row_out, S.getRowPositions().data(), sizeof(int32_t) * nnz);
    if (col_out) std::memcpy(col_out, S.getColPositions().data(), sizeof(int32_t) * nnz);
    if (sval_out) std::memcpy(sval_out, S.getValues().data(), sizeof(float) * nnz);
    return (int64_t)nnz;
}

/* Timed leg for the CPU baseline: the containers are built outside the clock,
 * only CPUBasic::run_csr is inside (benchmark/benchmark.hpp:166-168 times the
 * same call).  Returns seconds per run (best of reps). */
double ref_cpu_basic_csr_seconds(int M, int N, int K, int64_t n, const int32_t *row, const int32_t *col,
                                 const float *val, const float *A, const float *B, int reps, float *P_out)
{
    Dense<float> dA = make_dense(M, K, A), dB = make_dense(N, K, B);
    CSR<float> S(M, N, make_triplets(n, row, col, val));
    CSR<float> P(S);
    Competitors::CPUBasic<float> c;
    double best = 1e300;
    for (int r = 0; r < reps; r++) {
        P.clearValues();
        auto t0 = std::chrono::steady_clock::now();
        c.run_csr(dA, dB, S, P);
        auto t1 = std::chrono::steady_clock::now();
        double s = std::chrono::duration<double>(t1 - t0).count();
        if (s < best) best = s;
    }
    if (P_out) std::memcpy(P_out, P.getValues().data(), P.getValues().size() * sizeof(float));
    return best;
}

/* CSR(COO(triplets)) and COO(CSR(triplets)) round trips (tests/matrix_test.cc:93-122). */
int64_t ref_csr_build(int M, int N, int64_t n, const int32_t *row, const int32_t *col, const float *val,
                      int via_coo, int32_t *rowptr_out, int32_t *col_out, float *val_out)
{
    auto t = make_triplets(n, row, col, val);
    CSR<float> S = [&] {
        if (via_coo) { COO<float> c(M, N, t); return CSR<float>(c); }
        return CSR<float>(M, N, t);
    }();
    const size_t nnz = S.getValues().size();
    std::memcpy(rowptr_out, S.getRowPositions().data(), sizeof(int32_t) * (size_t)(M + 1));
    std::memcpy(col_out, S.getColPositions().data(), sizeof(int32_t) * nnz);
    std::memcpy(val_out, S.getValues().data(), sizeof(float) * nnz);
    return (int64_t)nnz;
}

/* CSR::computeDispatcher / computeDispatcherTensorCores (CSR.hpp:149-155). */
int ref_dispatch(int M, int N, int64_t n, const int32_t *row, const int32_t *col, const float *val,
                 int parts, int stride, int32_t *start_idx, int cap)
{
    CSR<float> S(M, N, make_triplets(n, row, col, val));
    if (stride == 16) S.computeDispatcherTensorCores(parts);
    else if (stride == 1) S.computeDispatcher(parts);
    else return -1;
    const auto &v = S.getStartIdx();
    if ((int)v.size() > cap) return -2;
    std::memcpy(start_idx, v.data(), sizeof(int32_t) * v.size());
    return (int)v.size();
}

}  /* extern "C" */
