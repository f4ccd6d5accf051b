// Seeded synthetic datasets and a Matrix Market reader for the C++ driver.
//
// The reference's datasets (src/benchmark/dataset.hpp) draw from an unseeded
// std::random_device (src/utils/random_generator.hpp:13-14,53-54); these use
// std::mt19937_64 with fixed seeds.  Shapes follow the five benchmark
// configurations; `scale` < 1 shrinks them.
#pragma once

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <random>
#include <sstream>
#include <string>
#include <vector>

#include "sddmm_containers.hpp"

namespace sddmm_host {

struct Dataset {
    std::string name;
    Dense<float> A, B;
    CSR<float> S_csr;
    COO<float> S_coo;
};

inline Dense<float> random_dense(std::mt19937_64 &rng, int rows, int cols, bool normal) {
    std::vector<float> flat((size_t)rows * cols);
    if (normal) {
        std::normal_distribution<float> d(0.f, 1.f);
        for (auto &x : flat) x = d(rng);
    } else {
        std::uniform_real_distribution<float> d(-1.f, 1.f);
        for (auto &x : flat) x = d(rng);
    }
    return Dense<float>((unsigned)rows, (unsigned)cols, std::move(flat));
}

inline Dataset finish(const std::string &name, int M, int N, int K, std::vector<Triplet<float>> t,
                      std::mt19937_64 &rng, bool normal) {
    Dataset d;
    d.name = name;
    d.S_csr = CSR<float>(M, N, std::move(t));
    d.S_coo = COO<float>(d.S_csr);
    d.A = random_dense(rng, M, K, normal);
    d.B = random_dense(rng, N, K, normal);
    return d;
}

// M x N with each position kept with probability `density`, values U[0,1)
// (the shape of RandomWithDensityDataset, src/benchmark/dataset.hpp:331-354).
inline Dataset uniform_random(int M, int N, int K, double density, uint64_t seed) {
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<float> v(0.f, 1.f);
    std::vector<Triplet<float>> t;
    // geometric skips instead of M*N coin flips
    std::geometric_distribution<int64_t> skip(std::min(1.0, std::max(density, 1e-12)));
    const int64_t total = (int64_t)M * N;
    for (int64_t pos = skip(rng); pos < total; pos += 1 + skip(rng))
        t.push_back({(int)(pos / N), (int)(pos % N), v(rng)});
    if (t.empty()) t.push_back({0, 0, 1.f});
    return finish("uniform", M, N, K, std::move(t), rng, false);
}

// dense 8x8 blocks inside a band of half-width `half_width` around the diagonal
inline Dataset fem_banded(int M, int K, int half_width, double blocks_per_row, uint64_t seed) {
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<float> v(0.f, 1.f);
    std::uniform_real_distribution<double> u(0.0, 1.0);
    const int nbr = M / 8, hw = std::max(1, half_width / 8);
    std::vector<Triplet<float>> t;
    std::vector<int> window;
    for (int b = 0; b < nbr; ++b) {
        const int lo = std::max(0, b - hw), hi = std::min(nbr - 1, b + hw);
        window.resize((size_t)(hi - lo + 1));
        for (int i = 0; i < (int)window.size(); ++i) window[(size_t)i] = lo + i;
        int nb = (int)blocks_per_row + (u(rng) < blocks_per_row - std::floor(blocks_per_row) ? 1 : 0);
        nb = std::min<int>(nb, (int)window.size());
        for (int i = 0; i < nb; ++i) {   // partial Fisher-Yates
            std::uniform_int_distribution<int> pick(i, (int)window.size() - 1);
            std::swap(window[(size_t)i], window[(size_t)pick(rng)]);
            for (int r = 0; r < 8; ++r)
                for (int c = 0; c < 8; ++c) t.push_back({b * 8 + r, window[(size_t)i] * 8 + c, v(rng)});
        }
    }
    return finish("fem_banded", nbr * 8, nbr * 8, K, std::move(t), rng, false);
}

// `dense_frac` of the rows near-dense inside a column window, the rest 5..20 entries
inline Dataset mixed_density(int M, int K, double dense_frac, int window, double fill, uint64_t seed) {
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<float> v(0.f, 1.f);
    std::uniform_real_distribution<double> u(0.0, 1.0);
    window = std::min(window, M);
    std::vector<Triplet<float>> t;
    for (int r = 0; r < M; ++r) {
        if (u(rng) < dense_frac) {
            std::uniform_int_distribution<int> s(0, M - window);
            const int s0 = s(rng);
            for (int c = 0; c < window; ++c)
                if (u(rng) < fill) t.push_back({r, s0 + c, v(rng)});
        } else {
            std::uniform_int_distribution<int> len(5, 20), col(0, M - 1);
            const int l = len(rng);
            for (int i = 0; i < l; ++i) t.push_back({r, col(rng), v(rng)});
        }
    }
    return finish("mixed_density", M, M, K, std::move(t), rng, false);
}

// Zipf row lengths and Zipf-skewed column popularity; values 1, A,B ~ N(0,1)
inline Dataset power_law(int M, int K, double mean_len, int trunc, uint64_t seed) {
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<double> u(0.0, 1.0);
    trunc = std::min(trunc, M);
    double alpha = 1.8;
    for (double lo = 1.01, hi = 4.0; hi - lo > 1e-6;) {   // fit alpha to the wanted truncated mean
        alpha = 0.5 * (lo + hi);
        double num = 0, den = 0;
        for (int k = 1; k <= trunc; ++k) { const double w = std::pow(k, -alpha); num += k * w; den += w; }
        if (num / den > mean_len) lo = alpha; else hi = alpha;
    }
    std::vector<double> cdf((size_t)trunc);
    double acc = 0;
    for (int k = 1; k <= trunc; ++k) { acc += std::pow(k, -alpha); cdf[(size_t)k - 1] = acc; }
    std::vector<int> perm((size_t)M);
    for (int i = 0; i < M; ++i) perm[(size_t)i] = i;
    std::shuffle(perm.begin(), perm.end(), rng);
    const double beta = 0.8, one_m = 1.0 - beta, top = std::pow(M + 1.0, one_m) - 1.0;
    std::vector<Triplet<float>> t;
    for (int r = 0; r < M; ++r) {
        const int len = (int)(std::lower_bound(cdf.begin(), cdf.end(), u(rng) * acc) - cdf.begin()) + 1;
        for (int i = 0; i < len; ++i) {
            int rank = (int)std::floor(std::pow(u(rng) * top + 1.0, 1.0 / one_m)) - 1;
            rank = std::min(std::max(rank, 0), M - 1);
            t.push_back({r, perm[(size_t)rank], 1.f});
        }
    }
    return finish("power_law", M, M, K, std::move(t), rng, true);
}

// fully dense 16x16 tiles at random tile positions
inline Dataset dense_tiles(int M, int N, int K, double tile_frac, uint64_t seed) {
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<float> v(0.f, 1.f);
    std::uniform_real_distribution<double> u(0.0, 1.0);
    std::vector<Triplet<float>> t;
    for (int ti = 0; ti < M / 16; ++ti)
        for (int tj = 0; tj < N / 16; ++tj)
            if (u(rng) < tile_frac)
                for (int r = 0; r < 16; ++r)
                    for (int c = 0; c < 16; ++c) t.push_back({ti * 16 + r, tj * 16 + c, v(rng)});
    if (t.empty()) t.push_back({0, 0, 1.f});
    return finish("dense_tiles", M, N, K, std::move(t), rng, false);
}

// One entry per row and per column at a random permutation, values U[0,1): the
// shape of LatinHypercubeDataset (src/benchmark/dataset.hpp:358-378, sampler
// src/utils/random_generator.hpp:82-107; the sampler there shuffles the row list
// twice and leaves the columns in order, which is still a permutation matrix).
inline Dataset latin_hypercube(int M, int K, uint64_t seed) {
    std::mt19937_64 rng(seed);
    std::uniform_real_distribution<float> v(0.f, 1.f);
    std::vector<int> perm((size_t)M);
    for (int i = 0; i < M; ++i) perm[(size_t)i] = i;
    std::shuffle(perm.begin(), perm.end(), rng);
    std::vector<Triplet<float>> t;
    t.reserve((size_t)M);
    for (int i = 0; i < M; ++i) t.push_back({perm[(size_t)i], i, v(rng)});
    return finish("latin_hypercube", M, M, K, std::move(t), rng, false);
}

// The first floor(density * M) rows completely filled with ones, every other row
// empty: the shape of UnbalancedDataset (src/benchmark/dataset.hpp:380-412).
inline Dataset unbalanced(int M, int N, int K, double density, uint64_t seed) {
    std::mt19937_64 rng(seed);
    const int full_rows = (int)(std::min(1.0, std::max(density, 0.0)) * M);
    std::vector<Triplet<float>> t;
    t.reserve((size_t)full_rows * N);
    for (int r = 0; r < full_rows; ++r)
        for (int c = 0; c < N; ++c) t.push_back({r, c, 1.f});
    if (t.empty()) t.push_back({0, 0, 1.f});
    return finish("unbalanced", M, N, K, std::move(t), rng, false);
}

// Matrix Market coordinate reader with the reference's conventions
// (src/benchmark/dataset.hpp:123-181): 1-based indices, the `symmetric`
// qualifier is NOT expanded, `pattern` files get value 1, and entries with
// |v| < 1e-7 are dropped.  Returns false when the file cannot be parsed.
inline bool read_matrix_market(const std::string &path, int K, uint64_t seed, Dataset &out, std::string &err) {
    std::ifstream in(path);
    if (!in) { err = "cannot open " + path; return false; }
    std::string line;
    bool pattern = false;
    if (!std::getline(in, line) || line.rfind("%%MatrixMarket", 0) != 0) { err = "missing %%MatrixMarket banner"; return false; }
    if (line.find("coordinate") == std::string::npos) { err = "only coordinate format is supported"; return false; }
    pattern = line.find("pattern") != std::string::npos;
    while (std::getline(in, line) && (line.empty() || line[0] == '%')) {}
    long long M = 0, N = 0, nz = 0;
    { std::istringstream h(line); if (!(h >> M >> N >> nz) || M <= 0 || N <= 0 || nz < 0) { err = "bad size line"; return false; } }
    std::vector<Triplet<float>> t;
    t.reserve((size_t)nz);
    for (long long i = 0; i < nz; ++i) {
        if (!std::getline(in, line)) { err = "file ends before all entries were read"; return false; }
        std::istringstream e(line);
        long long r, c;
        double v = 1.0;
        if (!(e >> r >> c)) { err = "bad entry line"; return false; }
        if (!pattern && !(e >> v)) { err = "entry without a value"; return false; }
        if (r < 1 || r > M || c < 1 || c > N) { err = "index out of range"; return false; }
        if (std::fabs(v) < 1e-7) continue;
        t.push_back({(int)(r - 1), (int)(c - 1), (float)v});
    }
    if (t.empty()) { err = "no entries"; return false; }
    std::mt19937_64 rng(seed);
    const size_t slash = path.find_last_of('/');
    out = finish(slash == std::string::npos ? path : path.substr(slash + 1), (int)M, (int)N, K, std::move(t), rng, false);
    return true;
}

// SNAP edge list reader (the format of EMailEnronDataset,
// src/benchmark/dataset.hpp:271-313): leading '#' comment lines (the reference
// skips the first four lines, which is what SNAP files carry), then one
// "row<TAB>col" pair per line with 0-based indices; every edge gets value 1 and
// the edge list is taken as directed, exactly as written.  dim > 0 fixes the
// square dimension (36692 for email-Enron in the reference); dim == 0 takes
// 1 + the largest index seen.  Returns false when the file cannot be parsed.
inline bool read_snap_edge_list(const std::string &path, int dim, int K, uint64_t seed, Dataset &out, std::string &err) {
    std::ifstream in(path);
    if (!in) { err = "cannot open " + path; return false; }
    std::vector<Triplet<float>> t;
    std::string line;
    long long top = -1, lineno = 0;
    while (std::getline(in, line)) {
        ++lineno;
        if (line.empty() || line[0] == '#' || line[0] == '%') continue;
        std::istringstream e(line);
        long long r, c;
        if (!(e >> r >> c)) { err = "bad edge at line " + std::to_string(lineno); return false; }
        if (r < 0 || c < 0 || r > 2147483646LL || c > 2147483646LL) { err = "index out of range at line " + std::to_string(lineno); return false; }
        if (dim > 0 && (r >= dim || c >= dim)) { err = "index beyond the given dimension at line " + std::to_string(lineno); return false; }
        top = std::max(top, std::max(r, c));
        t.push_back({(int)r, (int)c, 1.f});
    }
    if (t.empty()) { err = "no edges"; return false; }
    const int n = dim > 0 ? dim : (int)(top + 1);
    std::mt19937_64 rng(seed);
    const size_t slash = path.find_last_of('/');
    out = finish(slash == std::string::npos ? path : path.substr(slash + 1), n, n, K, std::move(t), rng, false);
    return true;
}

}  // namespace sddmm_host
