/*
 * Drop-in check, built only where the reference tree is mounted (oracle/Makefile,
 * output oracle/_ref/ref_adapter_check).  TEST INFRASTRUCTURE ONLY.
 *
 * Compiles this repository's competitor adapter (dphpc_amd/host/gpu_amd.hpp)
 * against the REFERENCE's own headers -- src/benchmark/competitor.hpp,
 * src/matrices/{Dense,CSR,COO}.hpp -- and runs it next to the reference's
 * CPUBasic (src/competitors/cpu/cpu_basic.hpp) on the reference's own containers,
 * the way tests/matrix_test.cc:40-82 compares competitors: P1 from CPU-Basic, P2
 * from the competitor, compared with the reference's operator== and, stricter,
 * value by value.  Inputs are positive like the reference's generateDense /
 * sampleTriplets (benchmark/dataset.hpp:35-43, utils/random_generator.hpp:56), the
 * only regime in which the reference's signed-relative operator== is meaningful.
 */
#include <cassert>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>
#include <vector>

#include "benchmark/competitor.hpp"      /* the reference's, via -I<reference>/src */
#include "matrices/matrices.h"
#include "competitors/cpu/cpu_basic.hpp"
#include "gpu_amd.hpp"                   /* this repository's adapter */

static int failures = 0;
#define CHECK(c) do { if (!(c)) { ++failures; std::printf("FAIL %s:%d %s\n", __FILE__, __LINE__, #c); } } while (0)

static Dense<float> random_dense(std::mt19937_64 &rng, int rows, int cols, float lo, float hi) {
    std::uniform_real_distribution<float> v(lo, hi);
    std::vector<std::vector<float>> m((size_t)rows, std::vector<float>((size_t)cols));
    for (auto &r : m) for (auto &x : r) x = v(rng);
    return Dense<float>(m);
}
static std::vector<Triplet<float>> random_triplets(std::mt19937_64 &rng, int rows, int cols, double density) {
    std::uniform_real_distribution<double> u(0.0, 1.0);
    std::uniform_real_distribution<float> v(0.05f, 1.0f);
    std::vector<Triplet<float>> t;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c)
            if (u(rng) < density) t.push_back(Triplet<float>{r, c, v(rng)});
    if (t.empty()) t.push_back(Triplet<float>{0, 0, 1.0f});
    return t;
}

static void compare(std::vector<std::shared_ptr<SDDMM::Competitor<float>>> &comps, Dense<float> &A, Dense<float> &B,
                    COO<float> &S_coo, const char *what) {
    CSR<float> S_csr(S_coo);
    COO<float> P1c(S_coo);
    CSR<float> P1r(S_csr);
    comps[0]->run_coo(A, B, S_coo, P1c);
    comps[0]->run_csr(A, B, S_csr, P1r);
    for (size_t i = 1; i < comps.size(); ++i) {
        auto &c = comps[i];
        COO<float> P2c(S_coo);
        P2c.clearValues();
        c->init_coo(A, B, S_coo, P2c);
        c->run_coo(A, B, S_coo, P2c);
        c->cleanup_coo(A, B, S_coo, P2c);
        CHECK(P1c == P2c);
        CSR<float> P2r(S_csr);
        P2r.clearValues();
        c->init_csr(A, B, S_csr, P2r);
        c->run_csr(A, B, S_csr, P2r);
        c->cleanup_csr(A, B, S_csr, P2r);
        CHECK(P1r == P2r);
        double worst = 0;
        for (size_t e = 0; e < P1r.getValues().size(); ++e) {
            const double ref = P1r.getValues()[e], got = P2r.getValues()[e];
            worst = std::max(worst, std::fabs(got - ref) / std::max(std::fabs(ref), 1e-30));
        }
        CHECK(worst <= 1e-5);
        const bool exact = c->name == "GPU-AMD-Exact";
        if (exact) CHECK(std::memcmp(P1r.getValues().data(), P2r.getValues().data(), P1r.getValues().size() * sizeof(float)) == 0);
        std::printf("%-28s %-18s nnz %8zu worst rel err %.3g%s\n", what, c->name.c_str(), P1r.getValues().size(), worst,
                    exact ? " (bitwise equal)" : "");
    }
}

int main() {
    std::vector<std::shared_ptr<SDDMM::Competitor<float>>> comps;
    comps.push_back(std::make_shared<Competitors::CPUBasic<float>>());
    for (int st : {SDDMM_AUTO, SDDMM_FLAT, SDDMM_ROW_WAVE, SDDMM_SHORT_ROWS, SDDMM_LDS_TILED, SDDMM_MFMA_TILE, SDDMM_EXACT})
        comps.push_back(std::make_shared<Competitors::GPUAmd>(st));
    std::mt19937_64 rng(2024);
    {
        std::vector<std::vector<float>> a{{1, 2}, {3, 4}, {5, 6}}, b{{-1, -3}, {2, 2}, {3, 1}};
        Dense<float> A(a), B(b);
        std::vector<Triplet<float>> t{{0, 0, 1.0f}, {1, 0, -1.0f}, {2, 0, 1.0f}, {2, 2, 1.0f}};
        COO<float> S(3, 3, t);
        compare(comps, A, B, S, "sddmm_coo4");
    }
    struct R { const char *name; int rows, cols, K; double d; };
    for (const R &r : {R{"random 500^2 d=0.3", 500, 500, 32, 0.3}, R{"random 250^2 d=0.7", 250, 250, 32, 0.7},
                       R{"random 10000^2 d=0.001", 10000, 10000, 32, 0.001}, R{"random 300x200 K=3", 300, 200, 3, 0.2},
                       R{"random 400^2 K=128", 400, 400, 128, 0.2}}) {
        Dense<float> A = random_dense(rng, r.rows, r.K, 0.f, 100.f), B = random_dense(rng, r.cols, r.K, 0.f, 100.f);
        COO<float> S(r.rows, r.cols, random_triplets(rng, r.rows, r.cols, r.d));
        compare(comps, A, B, S, r.name);
    }
    std::printf("ref_adapter_check: %d failure(s)\n", failures);
    return failures ? 1 : 0;
}
