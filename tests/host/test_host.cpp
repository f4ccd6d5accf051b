// The reference's test cases (tests/matrix_test.cc) re-expressed against this
// repository's host layer: containers, row partition, and the GPUAmd competitor
// driven exactly like test_all_competitors_{coo,csr} drives a competitor
// (tests/matrix_test.cc:40-82).  Expected values come from closed forms and from
// the CPU oracle (oracle/sddmm_oracle.c), never from the code under test.
//
//   test_host cpu   containers, conversions, partition vectors (no GPU needed)
//   test_host gpu   everything that launches kernels
#include <cstdio>
#include <cstdlib>
#include <unistd.h>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "cpu_host.hpp"
#include "gpu_amd.hpp"
#include "datasets.hpp"

extern "C" {
void oracle_sddmm_csr_f32(int M, int K, const int32_t *rowptr, const int32_t *col, const float *sval,
                          const float *A, const float *B, float *P);
void oracle_sddmm_coo_f32(int64_t nnz, int K, const int32_t *row, const int32_t *col, const float *sval,
                          const float *A, const float *B, float *P);
void oracle_sddmm_csr_f64(int M, int K, const int32_t *rowptr, const int32_t *col, const float *sval,
                          const float *A, const float *B, double *dot64, double *mag64);
}

static int g_checks = 0, g_failed = 0;
static const char *g_case = "";
#define CHECK(cond)                                                                         \
    do {                                                                                    \
        ++g_checks;                                                                         \
        if (!(cond)) { ++g_failed; std::printf("FAIL [%s] %s:%d: %s\n", g_case, __FILE__, __LINE__, #cond); } \
    } while (0)
#define CASE(name) g_case = name; std::printf("case %s\n", name); std::fflush(stdout)

using Trips = std::vector<Triplet<float>>;

static Dense<float> dense_of(std::vector<std::vector<float>> v) { return Dense<float>(v); }

// seeded stand-in for the reference's unseeded sampleTriplets / generate_data
static Trips random_triplets(std::mt19937_64 &rng, int rows, int cols, double density, float lo, float hi) {
    std::uniform_real_distribution<double> u(0.0, 1.0);
    std::uniform_real_distribution<float> v(lo, hi);
    Trips t;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c)
            if (u(rng) < density) t.push_back({r, c, v(rng)});
    if (t.empty()) t.push_back({0, 0, 1.0f});
    return t;
}
static Trips sample_triplets(std::mt19937_64 &rng, int rows, int cols, int n) {
    std::uniform_int_distribution<int> ur(0, rows - 1), uc(0, cols - 1);
    std::uniform_real_distribution<float> v(0.1f, 1.0f);
    Trips t;
    for (int i = 0; i < n; ++i) t.push_back({ur(rng), uc(rng), v(rng)});
    return t;
}
static Dense<float> random_dense(std::mt19937_64 &rng, int rows, int cols, float lo, float hi) {
    std::uniform_real_distribution<float> v(lo, hi);
    std::vector<float> flat((size_t)rows * cols);
    for (auto &x : flat) x = v(rng);
    return Dense<float>((unsigned)rows, (unsigned)cols, std::move(flat));
}

// |got-ref| <= 1e-5 * max(|ref|, 0.25*mag)
static bool close_to_oracle(const std::vector<float> &got, const std::vector<float> &ref, const std::vector<double> &mag) {
    if (got.size() != ref.size()) return false;
    for (size_t i = 0; i < got.size(); ++i) {
        const double scale = std::max(std::fabs((double)ref[i]), 0.25 * mag[i]);
        if (!(std::fabs((double)got[i] - (double)ref[i]) <= 1e-5 * scale)) {
            std::printf("  entry %zu got %.9g ref %.9g\n", i, got[i], ref[i]);
            return false;
        }
    }
    return true;
}

// ---------------------------------------------------------------- CPU cases
static void cpu_cases() {
    {
        CASE("COO");   // tests/matrix_test.cc:84-91
        Trips t{{0, 0, 1.0f}, {0, 1, 1.0f}, {1, 0, 1.0f}, {1, 1, 1.0f}};
        COO<float> coo(2, 2, t);
        CHECK(coo.getValues().size() == 4 && coo.getRowPositions().size() == 4 && coo.getColPositions().size() == 4);
    }
    {
        CASE("RepresentationConversion");   // :93-106
        Trips tc{{0, 0, 1.0f}, {1, 0, 1.0f}, {0, 1, 1.0f}, {1, 1, 1.0f}};
        CSR<float> csr(2, 2, tc);
        Trips t{{0, 0, 1.0f}, {0, 1, 1.0f}, {1, 0, 1.0f}, {1, 1, 1.0f}};
        COO<float> coo(2, 2, t);
        CSR<float> csr2(coo);
        COO<float> coo2(csr);
        CHECK(csr == csr2);
        CHECK(coo == coo2);
        CHECK((csr.getRowPositions() == std::vector<int>{0, 2, 4}));
        CHECK((csr.getColPositions() == std::vector<int>{0, 1, 0, 1}));
    }
    {
        CASE("BiggerConversion");   // :108-122
        std::mt19937_64 rng(1234);
        for (int i = 100; i <= 1500; i += 25) {
            const int cols = i, rows = 2 * i;
            Trips t = sample_triplets(rng, rows, cols, i);
            CSR<float> s_csr(rows, cols, t);
            COO<float> s_coo(rows, cols, t);
            CSR<float> back_csr(s_coo);
            COO<float> back_coo(s_csr);
            CHECK(s_csr == back_csr);
            CHECK(s_coo == back_coo);
        }
    }
    {
        CASE("triplet_rules");   // triplet.h:12-19
        Trips t{{1, 0, 5.f}, {0, 1, 2.f}, {1, 0, 6.f}, {0, 0, 1.f}, {1, 1, 0.f}, {0, 1, 3.f}, {2, 2, 0.f}, {2, 2, 7.f}};
        COO<float> coo(3, 3, t);
        CHECK((coo.getRowPositions() == std::vector<int>{0, 0, 1, 1, 2, 2}));
        CHECK((coo.getColPositions() == std::vector<int>{0, 1, 0, 1, 2, 2}));
        CHECK((coo.getValues() == std::vector<float>{1.f, 2.f, 5.f, 0.f, 0.f, 7.f}));   // zeros never merge
        CSR<float> csr(4, 3, Trips{{1, 0, 1.f}});
        CHECK((csr.getRowPositions() == std::vector<int>{0, 0, 1, 1, 1}));
    }
    {
        CASE("dispatcher");   // :354-425, :460-477
        Trips sq{{0, 0, 1.f}, {1, 0, 1.f}, {0, 1, 1.f}, {1, 1, 1.f}};
        CSR<float> a(2, 2, sq);
        a.computeDispatcher(4);
        CHECK((a.getStartIdx() == std::vector<int>{0, 1, 2, 2, 2}));
        a.computeDispatcher(2);
        CHECK((a.getStartIdx() == std::vector<int>{0, 1, 2}));
        CSR<float> b(4, 2, Trips{{0, 0, 1.f}, {1, 0, 1.f}, {2, 1, 1.f}, {3, 1, 1.f}});
        b.computeDispatcher(2);
        CHECK((b.getStartIdx() == std::vector<int>{0, 2, 4}));
        CSR<float> c(4, 2, Trips{{1, 0, 1.f}});
        c.computeDispatcher(2);
        CHECK((c.getStartIdx() == std::vector<int>{0, 4, 4}));
        const int n = 150000;
        Trips diag;
        for (int i = 0; i < n; ++i) diag.push_back({i, i, 4.f});
        CSR<float> d(n, n, diag);
        d.computeDispatcher(n / 2);
        bool okd = d.getStartIdx().size() == (size_t)n / 2 + 1;
        for (int i = 0; okd && i <= n / 2; ++i) okd = d.getStartIdx()[(size_t)i] == 2 * i;
        CHECK(okd);
        Trips d64;
        for (int i = 0; i < 64; ++i) d64.push_back({i, i, 1.f});
        CSR<float> e(64, 64, d64);
        e.computeDispatcherTensorCores(4);
        CHECK((e.getStartIdx() == std::vector<int>{0, 16, 32, 48, 64}));
        CHECK(std::fabs(d.getDensity() - 1.0 / n) < 1e-12);   // 150000^2 overflows int in the reference
    }
    {
        CASE("tolerant_equality");
        CSR<float> x(2, 2, Trips{{0, 0, 1.f}, {1, 1, -2.f}});
        CSR<float> y(x), z(x), w(x);
        y.getValues()[0] = 1.0005f;
        CHECK(y == x);                      // within 1e-3
        z.getValues()[1] = -2.1f;
        CHECK(!(z == x));                   // the reference's signed test would accept this
        w.getValues()[1] = 2.f;
        CHECK(!(w == x));
        CSR<float> zero(x), zero2(x);
        zero.clearValues(); zero2.clearValues();
        CHECK(zero == zero2);               // 0/0 is NaN in the reference
    }
    {
        CASE("file_readers");   // src/benchmark/dataset.hpp:123-181 (Matrix Market), :271-313 (SNAP edge list)
        char dir[] = "/tmp/sddmm_host_XXXXXX";
        CHECK(mkdtemp(dir) != nullptr);
        const std::string base(dir);
        auto put = [&](const char *name, const char *text) {
            std::ofstream f(base + "/" + name);
            f << text;
            return base + "/" + name;
        };
        sddmm_host::Dataset d;
        std::string err;
        // four header lines, TAB-separated 0-based pairs, a repeated edge, directed as written
        const std::string snap = put("edges.txt", "# Directed graph\n# tiny\n# Nodes: 5 Edges: 5\n# FromNodeId\tToNodeId\n"
                                                  "0\t1\n3\t0\n1\t4\n0\t1\n4\t4\n");
        CHECK(sddmm_host::read_snap_edge_list(snap, 0, 8, 7, d, err));
        CHECK(d.S_csr.getRows() == 5 && d.S_csr.getCols() == 5 && d.A.getRows() == 5 && d.B.getCols() == 8);
        CHECK((d.S_csr.getRowPositions() == std::vector<int>{0, 1, 2, 2, 3, 4}));   // the repeated edge is stored once
        CHECK((d.S_csr.getColPositions() == std::vector<int>{1, 4, 0, 4}));
        CHECK((d.S_csr.getValues() == std::vector<float>{1.f, 1.f, 1.f, 1.f}));
        CHECK(d.S_coo.getRowPositions() == (std::vector<int>{0, 1, 3, 4}));
        CHECK(sddmm_host::read_snap_edge_list(snap, 36, 4, 7, d, err) && d.S_csr.getRows() == 36 && d.S_csr.getCols() == 36);
        CHECK(!sddmm_host::read_snap_edge_list(snap, 4, 4, 7, d, err) && err.find("dimension") != std::string::npos);
        CHECK(!sddmm_host::read_snap_edge_list(put("bad.txt", "# x\n1\n"), 0, 4, 7, d, err));
        CHECK(!sddmm_host::read_snap_edge_list(base + "/absent.txt", 0, 4, 7, d, err));
        // Matrix Market: 1-based, symmetric not expanded, pattern -> 1, tiny values dropped
        const std::string mm = put("m.mtx", "%%MatrixMarket matrix coordinate real symmetric\n% c\n3 4 4\n"
                                            "1 1 2.5\n3 4 -1\n2 2 1e-9\n2 1 0.5\n");
        CHECK(sddmm_host::read_matrix_market(mm, 4, 7, d, err));
        CHECK(d.S_csr.getRows() == 3 && d.S_csr.getCols() == 4);
        CHECK((d.S_csr.getRowPositions() == std::vector<int>{0, 1, 2, 3}));
        CHECK((d.S_csr.getColPositions() == std::vector<int>{0, 0, 3}));
        CHECK((d.S_csr.getValues() == std::vector<float>{2.5f, 0.5f, -1.f}));
        const std::string pat = put("p.mtx", "%%MatrixMarket matrix coordinate pattern general\n2 2 2\n2 1\n1 2\n");
        CHECK(sddmm_host::read_matrix_market(pat, 4, 7, d, err));
        CHECK((d.S_csr.getValues() == std::vector<float>{1.f, 1.f}) && (d.S_csr.getColPositions() == std::vector<int>{1, 0}));
        CHECK(!sddmm_host::read_matrix_market(put("a.mtx", "%%MatrixMarket matrix array real general\n2 2\n1\n2\n3\n4\n"), 4, 7, d, err));
        for (const char *n : {"edges.txt", "bad.txt", "m.mtx", "p.mtx", "a.mtx"}) std::remove((base + "/" + n).c_str());
        rmdir(dir);
    }
    {
        CASE("latin_and_unbalanced_shapes");   // src/benchmark/dataset.hpp:358-412
        const sddmm_host::Dataset l = sddmm_host::latin_hypercube(257, 8, 11);
        CHECK(l.S_csr.getRows() == 257 && l.S_csr.getCols() == 257 && l.S_csr.getValues().size() == 257);
        std::vector<int> per_col(257, 0);
        bool one_per_row = true, moved = false;
        for (int r = 0; r < 257; ++r) {
            one_per_row = one_per_row && l.S_csr.getRowPositions()[r + 1] - l.S_csr.getRowPositions()[r] == 1;
            const int c = l.S_csr.getColPositions()[r];
            per_col[c] += 1;
            moved = moved || c != r;
        }
        CHECK(one_per_row && moved);
        CHECK(std::all_of(per_col.begin(), per_col.end(), [](int n) { return n == 1; }));
        CHECK(std::all_of(l.S_csr.getValues().begin(), l.S_csr.getValues().end(), [](float v) { return v >= 0.f && v < 1.f; }));
        const sddmm_host::Dataset u = sddmm_host::unbalanced(40, 24, 8, 0.26, 12);   // floor(0.26 * 40) = 10 full rows
        CHECK(u.S_csr.getRows() == 40 && u.S_csr.getCols() == 24 && u.S_csr.getValues().size() == 240);
        bool shape = true;
        for (int r = 0; r <= 40; ++r) shape = shape && u.S_csr.getRowPositions()[r] == std::min(r, 10) * 24;
        for (int j = 0; j < 240; ++j) shape = shape && u.S_csr.getColPositions()[j] == j % 24 && u.S_csr.getValues()[j] == 1.f;
        CHECK(shape);
        CHECK(u.S_coo.getRowPositions()[239] == 9 && u.A.getRows() == 40 && u.B.getRows() == 24);
    }
    {
        CASE("the driver's CPU-Basic competitor equals the oracle bit for bit (CSR and COO)");
        // the ground truth of sddmm_driver (cpu_host.hpp) against the closed form of the
        // reference's sddmm_coo1 (tests/matrix_test.cc:124-137) and against the oracle on
        // signed random inputs, through the competitor interface like any other competitor
        Competitors::CPUHost cpu;
        CHECK(cpu.name == "CPU-Basic" && cpu.csr_supported() && cpu.coo_supported() && !cpu.is_gpu());
        {
            Dense<float> A = dense_of({{1, 2}, {3, 4}}), B = dense_of({{-1, 2}, {-3, 4}});
            Trips t = {{0, 0, 1.f}, {0, 1, 1.f}, {1, 0, 1.f}, {1, 1, 1.f}};
            COO<float> S(2, 2, t), P(S);
            P.clearValues();
            cpu.init_coo(A, B, S, P); cpu.run_coo(A, B, S, P); cpu.cleanup_coo(A, B, S, P);
            CHECK((P.getValues() == std::vector<float>{3.f, 5.f, 5.f, 7.f}));
        }
        std::mt19937_64 rng(4242);
        for (int K : {1, 7, 32, 100}) {
            Trips t = random_triplets(rng, 57, 43, 0.2, -1.f, 1.f);
            COO<float> S_coo(57, 43, t);
            CSR<float> S(S_coo);
            Dense<float> A = random_dense(rng, 57, K, -1.f, 1.f), B = random_dense(rng, 43, K, -1.f, 1.f);
            std::vector<float> ref(S.getValues().size());
            oracle_sddmm_csr_f32(S.getRows(), K, S.getRowPositions().data(), S.getColPositions().data(), S.getValues().data(),
                                 A.get_pointer(), B.get_pointer(), ref.data());
            CSR<float> P(S);
            P.clearValues();
            cpu.init_csr(A, B, S, P); cpu.run_csr(A, B, S, P); cpu.cleanup_csr(A, B, S, P);
            CHECK(P.getValues().size() == ref.size() &&
                  std::memcmp(P.getValues().data(), ref.data(), ref.size() * sizeof(float)) == 0);
            CHECK(P.getColPositions() == S.getColPositions() && P.getRowPositions() == S.getRowPositions());
            COO<float> Pc(S_coo);
            Pc.clearValues();
            cpu.init_coo(A, B, S_coo, Pc); cpu.run_coo(A, B, S_coo, Pc); cpu.cleanup_coo(A, B, S_coo, Pc);
            CHECK(Pc.getValues().size() == ref.size() &&
                  std::memcmp(Pc.getValues().data(), ref.data(), ref.size() * sizeof(float)) == 0);
            std::vector<double> mag(ref.size());
            oracle_sddmm_csr_f64(S.getRows(), K, S.getRowPositions().data(), S.getColPositions().data(), S.getValues().data(),
                                 A.get_pointer(), B.get_pointer(), nullptr, mag.data());
            const std::vector<double> got_mag = Competitors::CPUHost::magnitudes(A, B, S);
            bool same = got_mag.size() == mag.size();
            for (size_t i = 0; same && i < mag.size(); ++i) same = std::fabs(got_mag[i] - mag[i]) <= 1e-12 * (1.0 + mag[i]);
            CHECK(same);
        }
    }
}

// ---------------------------------------------------------------- GPU cases
static const int kStrategies[] = {SDDMM_AUTO, SDDMM_FLAT, SDDMM_ROW_WAVE, SDDMM_SHORT_ROWS, SDDMM_LDS_TILED, SDDMM_MFMA_TILE, SDDMM_EXACT};

// tests/matrix_test.cc:40-59 with the oracle in the role of float_competitors[0]
// `harness_predicate`: also apply the containers' operator== (1e-3 relative to the
// expected value).  Like the reference's, it is only meaningful when no entry is the
// result of heavy cancellation, i.e. for the positive inputs the reference generates.
static COO<float> all_strategies_coo(Dense<float> &A, Dense<float> &B, COO<float> &S, const std::vector<float> *closed_form,
                                     bool harness_predicate = true) {
    const int K = (int)A.getCols();
    std::vector<float> ref(S.getValues().size());
    oracle_sddmm_coo_f32((int64_t)ref.size(), K, S.getRowPositions().data(), S.getColPositions().data(),
                         S.getValues().data(), A.get_pointer(), B.get_pointer(), ref.data());
    if (closed_form) CHECK(ref == *closed_form);
    CSR<float> S_csr(S);
    std::vector<double> mag(ref.size());
    oracle_sddmm_csr_f64(S_csr.getRows(), K, S_csr.getRowPositions().data(), S_csr.getColPositions().data(),
                         S_csr.getValues().data(), A.get_pointer(), B.get_pointer(), nullptr, mag.data());
    COO<float> P1(S);
    P1.setValues(ref);
    for (int st : kStrategies) {
        Competitors::GPUAmd comp(st);
        COO<float> P2(S);
        P2.clearValues();
        comp.init_coo(A, B, S, P2);
        comp.run_coo(A, B, S, P2);
        comp.cleanup_coo(A, B, S, P2);
        CHECK(comp.last_ok());
        if (harness_predicate) CHECK(P2 == P1);
        CHECK(P2.getRowPositions() == S.getRowPositions() && P2.getColPositions() == S.getColPositions());
        CHECK(close_to_oracle(P2.getValues(), ref, mag)); // the strict one
        if (st == SDDMM_EXACT) CHECK(std::memcmp(P2.getValues().data(), ref.data(), ref.size() * sizeof(float)) == 0);
        if (closed_form) CHECK(P2.getValues() == *closed_form);
    }
    return P1;
}

static CSR<float> all_strategies_csr(Dense<float> &A, Dense<float> &B, CSR<float> &S, bool harness_predicate = true) {
    const int K = (int)A.getCols();
    std::vector<float> ref(S.getValues().size());
    std::vector<double> mag(ref.size());
    oracle_sddmm_csr_f32(S.getRows(), K, S.getRowPositions().data(), S.getColPositions().data(), S.getValues().data(),
                         A.get_pointer(), B.get_pointer(), ref.data());
    oracle_sddmm_csr_f64(S.getRows(), K, S.getRowPositions().data(), S.getColPositions().data(), S.getValues().data(),
                         A.get_pointer(), B.get_pointer(), nullptr, mag.data());
    CSR<float> P1(S);
    P1.setValues(ref);
    for (int st : kStrategies) {
        Competitors::GPUAmd comp(st);
        CSR<float> P2(S);
        P2.clearValues();
        comp.init_csr(A, B, S, P2);
        comp.run_csr(A, B, S, P2);
        comp.cleanup_csr(A, B, S, P2);
        CHECK(comp.last_ok());
        if (harness_predicate) CHECK(P2 == P1);
        CHECK(close_to_oracle(P2.getValues(), ref, mag));
        if (st == SDDMM_EXACT) CHECK(std::memcmp(P2.getValues().data(), ref.data(), ref.size() * sizeof(float)) == 0);
    }
    return P1;
}

static void gpu_cases() {
    {
        CASE("sddmm_coo1");   // :124-138
        auto A = dense_of({{1, 2}, {3, 4}}), B = dense_of({{-1, 2}, {-3, 4}});
        COO<float> S(2, 2, Trips{{0, 0, 1.f}, {0, 1, 1.f}, {1, 0, 1.f}, {1, 1, 1.f}});
        std::vector<float> exp{3, 5, 5, 7};
        all_strategies_coo(A, B, S, &exp);
    }
    {
        CASE("sddmm_coo2");   // :140-152
        auto A = dense_of({{1, 2, 3}, {4, 5, 6}}), B = dense_of({{-1, -3, 5}, {2, 4, -6}});
        COO<float> S(2, 2, Trips{{0, 0, 1.f}, {1, 0, 1.f}, {1, 1, 1.f}});
        std::vector<float> exp{8, 11, -8};
        all_strategies_coo(A, B, S, &exp);
    }
    {
        CASE("sddmm_coo3");   // :154-166 (B has one row; S is declared 2x2 there, only column 0 is used)
        auto A = dense_of({{1, 2, 3}, {4, 5, 6}}), B = dense_of({{-1, -3, 5}});
        COO<float> S(2, 1, Trips{{0, 0, 1.f}, {1, 0, -1.f}});
        std::vector<float> exp{8, -11};
        all_strategies_coo(A, B, S, &exp);
    }
    {
        CASE("sddmm_coo4");   // :168-182
        auto A = dense_of({{1, 2}, {3, 4}, {5, 6}}), B = dense_of({{-1, -3}, {2, 2}, {3, 1}});
        COO<float> S(3, 3, Trips{{0, 0, 1.f}, {1, 0, -1.f}, {2, 0, 1.f}, {2, 2, 1.f}});
        std::vector<float> exp{-7, 15, -23, 21};
        all_strategies_coo(A, B, S, &exp);
    }
    {
        CASE("dummy_dataset");   // benchmark/dataset.hpp:183-204
        auto A = dense_of({{1, 1}, {1, 1}}), B = dense_of({{1, 1}, {1, 1}});
        COO<float> S(2, 2, Trips{{0, 0, 1.f}, {0, 1, 1.f}, {1, 0, 1.f}, {1, 1, 1.f}});
        std::vector<float> exp{2, 2, 2, 2};
        all_strategies_coo(A, B, S, &exp);
    }
    struct R { const char *name; int rows, cols; double d; };
    // :184-227; inputs positive like the reference's generateDense (dataset.hpp:35-43)
    // in the first three, signed in the last
    const R randoms[] = {{"sddmm_random_coo", 500, 500, 0.3}, {"sddmm_random_dense_coo", 250, 250, 0.7},
                         {"sddmm_random_sparse_coo", 10000, 10000, 0.001}};
    std::mt19937_64 rng(42);
    for (const R &r : randoms) {
        CASE(r.name);
        auto A = random_dense(rng, r.rows, 32, 0.f, 100.f), B = random_dense(rng, r.cols, 32, 0.f, 100.f);
        COO<float> S(r.rows, r.cols, random_triplets(rng, r.rows, r.cols, r.d, 0.f, 1.f));
        all_strategies_coo(A, B, S, nullptr);
    }
    {
        CASE("sddmm_csr_coo");   // :229-246
        auto A = random_dense(rng, 500, 32, 0.f, 100.f), B = random_dense(rng, 500, 32, 0.f, 100.f);
        COO<float> S_coo(500, 500, random_triplets(rng, 500, 500, 0.3, 0.f, 1.f));
        CSR<float> S_csr(S_coo);
        CSR<float> P_csr = all_strategies_csr(A, B, S_csr);
        COO<float> P_coo = all_strategies_coo(A, B, S_coo, nullptr);
        COO<float> P_csr_as_coo(P_csr);
        CHECK(P_coo == P_csr_as_coo);
        CHECK(P_coo.getValues() == P_csr_as_coo.getValues());   // same arithmetic: bitwise
    }
    {
        CASE("signed_inputs_csr_coo");   // cancellation: only the floor-scaled comparison applies
        auto A = random_dense(rng, 500, 32, -1.f, 1.f), B = random_dense(rng, 500, 32, -1.f, 1.f);
        COO<float> S_coo(500, 500, random_triplets(rng, 500, 500, 0.3, -1.f, 1.f));
        CSR<float> S_csr(S_coo);
        CSR<float> P_csr = all_strategies_csr(A, B, S_csr, false);
        COO<float> P_coo = all_strategies_coo(A, B, S_coo, nullptr, false);
        COO<float> P_csr_as_coo(P_csr);
        CHECK(P_coo.getValues() == P_csr_as_coo.getValues());
    }
    {
        CASE("competitor_reuse_and_flags");
        Competitors::GPUAmd comp;
        CHECK(comp.is_gpu() && comp.csr_supported() && comp.coo_supported());
        CHECK(comp.name == "GPU-AMD-Dynamic");
        CHECK(comp.get_num_thread_blocks() == 1 && comp.get_num_threads_per_block() == 1);
        for (int round = 0; round < 3; ++round) {   // one object, many runs and datasets (benchmark.hpp:71-99)
            const int M = 200 + 50 * round, N = 300 - 40 * round;
            auto A = random_dense(rng, M, 32, 0.f, 1.f), B = random_dense(rng, N, 32, 0.f, 1.f);
            CSR<float> S(M, N, random_triplets(rng, M, N, 0.1, 0.1f, 1.f));
            CSR<float> P(S);
            P.clearValues();
            comp.init_csr(A, B, S, P);
            comp.run_csr(A, B, S, P);
            comp.cleanup_csr(A, B, S, P);
            std::vector<float> ref(S.getValues().size());
            oracle_sddmm_csr_f32(M, 32, S.getRowPositions().data(), S.getColPositions().data(), S.getValues().data(),
                                 A.get_pointer(), B.get_pointer(), ref.data());
            CSR<float> E(S);
            E.setValues(ref);
            CHECK(P == E);
            CHECK(comp.get_num_threads_per_block() == 256);
        }
    }
    {
        CASE("mismatched_k_is_reported_not_thrown");
        std::mt19937_64 r2(7);
        auto A = random_dense(r2, 10, 8, -1.f, 1.f), B = random_dense(r2, 10, 4, -1.f, 1.f);
        CSR<float> S(10, 10, Trips{{0, 0, 1.f}, {3, 4, 2.f}});
        CSR<float> P(S);
        P.clearValues();
        Competitors::GPUAmd comp;
        comp.init_csr(A, B, S, P);
        comp.run_csr(A, B, S, P);
        comp.cleanup_csr(A, B, S, P);
        CHECK(!comp.last_ok());
        CHECK((P.getValues() == std::vector<float>{0.f, 0.f}));   // P keeps its zeros: correctness 0 in the CSV
        CHECK(P.getColPositions() == S.getColPositions());
    }
}

int main(int argc, char **argv) {
    const std::string mode = argc > 1 ? argv[1] : "cpu";
    if (mode == "cpu" || mode == "all") cpu_cases();
    if (mode == "gpu" || mode == "all") gpu_cases();
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
