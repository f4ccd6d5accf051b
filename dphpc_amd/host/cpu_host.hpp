// Competitors::CPUHost -- the ground truth of the benchmark driver: the plain host
// loop of the reference's CPU-Basic competitor (src/competitors/cpu/cpu_basic.hpp:18-51),
// which the reference's harness takes as expected result for every other competitor
// (src/benchmark/benchmark.hpp:50-61, src/main.cpp:18-22).
//
// Operation order per stored entry: fp32 multiply, fp32 add, k ascending from an
// accumulator of 0, then one fp32 multiply by the entry's S value.  The translation
// unit that includes this header must be compiled with -ffp-contract=off so that the
// multiply and the add stay two roundings; GPU-AMD-Exact then has to agree bit for bit.
//
// It also returns, on request, the cancellation-free magnitude |S| * sum_k |a_k b_k|
// of every entry (in double), the floor of the driver's tolerance.
#pragma once

#include <cmath>
#include <cstdint>
#include <string>
#include <vector>

#include "benchmark/competitor.hpp"
#include "matrices/matrices.h"

namespace Competitors {

class CPUHost : public SDDMM::Competitor<float> {
public:
    CPUHost() : SDDMM::Competitor<float>("CPU-Basic") {}

    void run_csr(Dense<float> &A, Dense<float> &B, CSR<float> &S, CSR<float> &P) override {
        const auto &rp = S.getRowPositions();
        std::vector<float> out(S.getValues().size());
        for (size_t row = 0; row + 1 < rp.size(); ++row)
            for (int32_t n = rp[row]; n < rp[row + 1]; ++n)
                out[(size_t)n] = entry(A, B, (int)row, S.getColPositions()[(size_t)n], S.getValues()[(size_t)n]);
        P.setValues(out);
        P.setColPositions(S.getColPositions());
        P.setRowPositions(S.getRowPositions());
    }
    void run_coo(Dense<float> &A, Dense<float> &B, COO<float> &S, COO<float> &P) override {
        const size_t nnz = S.getValues().size();
        std::vector<float> out(nnz);
        for (size_t n = 0; n < nnz; ++n)
            out[n] = entry(A, B, S.getRowPositions()[n], S.getColPositions()[n], S.getValues()[n]);
        P.setValues(out);
        P.setColPositions(S.getColPositions());
        P.setRowPositions(S.getRowPositions());
    }
    bool csr_supported() override { return true; }
    bool coo_supported() override { return true; }

    // |S| * sum_k |a_k * b_k| per stored entry of a CSR pattern
    static std::vector<double> magnitudes(Dense<float> &A, Dense<float> &B, CSR<float> &S) {
        const auto &rp = S.getRowPositions();
        const int K = (int)A.getCols();
        std::vector<double> mag(S.getValues().size());
        for (size_t row = 0; row + 1 < rp.size(); ++row) {
            const float *a = A.get_pointer() + row * (size_t)K;
            for (int32_t n = rp[row]; n < rp[row + 1]; ++n) {
                const float *b = B.get_pointer() + (size_t)S.getColPositions()[(size_t)n] * (size_t)K;
                double acc = 0.0;
                for (int k = 0; k < K; ++k) acc += std::fabs((double)a[k] * (double)b[k]);
                mag[(size_t)n] = acc * std::fabs((double)S.getValues()[(size_t)n]);
            }
        }
        return mag;
    }

private:
    static float entry(Dense<float> &A, Dense<float> &B, int row, int col, float s) {
        const int K = (int)A.getCols();
        const float *a = A.get_pointer() + (size_t)row * (size_t)K;
        const float *b = B.get_pointer() + (size_t)col * (size_t)K;
        float acc = 0.0f;
        for (int k = 0; k < K; ++k) {
            const float prod = a[k] * b[k];
            acc = acc + prod;
        }
        return acc * s;
    }
};

}  // namespace Competitors
