// Host-side containers with the public interface of the reference's
// src/matrices/{Dense,CSR,COO}.hpp and triplet.h, so that code written against
// the reference (its competitors, its tests) compiles unchanged against these.
// The implementation is independent: one base class carries the index/value
// arrays, construction sorts an index permutation, and the row partition is
// delegated to the library's sddmm_partition_rows.
//
// Deliberate differences from the reference, all on paths where it misbehaves:
//   * operator== divides by |expected| and treats equal values (including two
//     zeros) as matching; the reference divides by the signed expected value
//     (CSR.hpp:92-94), which accepts any error on a negative entry and yields NaN
//     on a zero one;
//   * getDensity() multiplies in double (CSR.hpp:157-159 overflows int above
//     46340 x 46340);
//   * the triplet sort is stable, so which duplicate survives is defined
//     (the first in input order); the reference uses std::sort.
#pragma once

#include <algorithm>
#include <cassert>
#include <cmath>
#include <cstdint>
#include <iostream>
#include <numeric>
#include <type_traits>
#include <vector>

#include "../../include/sddmm_amd.h"

template <typename T>
struct Triplet {
    int row;
    int col;
    T value;
};

// src/matrices/triplet.h:12-14 -- two triplets merge only when both values are non-zero
template <typename T>
bool operator==(const Triplet<T> &a, const Triplet<T> b) {
    return a.row == b.row && a.col == b.col && a.value && b.value;
}
// src/matrices/triplet.h:16-19
template <typename T>
bool operator<(const Triplet<T> &a, const Triplet<T> b) {
    return a.row != b.row ? a.row < b.row : a.col < b.col;
}
template <typename S>
std::ostream &operator<<(std::ostream &os, const Triplet<S> &t) {
    return os << t.row << " " << t.col << " " << t.value;
}

// ---------------------------------------------------------------------------
// Row-major dense matrix (src/matrices/Dense.hpp:21-58).
template <class T>
class Dense {
public:
    Dense() = default;
    explicit Dense(std::vector<std::vector<T>> &in) {
        assert(!in.empty());
        rows_ = (unsigned)in.size();
        cols_ = (unsigned)in.front().size();
        data_.resize((size_t)rows_ * cols_);
        for (unsigned r = 0; r < rows_; ++r) {
            assert(in[r].size() == cols_);
            std::copy(in[r].begin(), in[r].end(), data_.begin() + (size_t)r * cols_);
        }
    }
    // adopt a flat row-major buffer (not in the reference; used by the drivers)
    Dense(unsigned rows, unsigned cols, std::vector<T> flat) : rows_(rows), cols_(cols), data_(std::move(flat)) {
        assert(data_.size() == (size_t)rows * cols);
    }
    T &getValue(int row, int col) { return data_[(size_t)row * cols_ + (size_t)col]; }
    T *get_pointer() { return data_.data(); }
    unsigned int getRows() const { return rows_; }
    unsigned int getCols() const { return cols_; }
    friend std::ostream &operator<<(std::ostream &os, const Dense &d) {
        for (unsigned r = 0; r < d.rows_; ++r) {
            for (unsigned c = 0; c < d.cols_; ++c) os << d.data_[(size_t)r * d.cols_ + c] << " ";
            os << "\n";
        }
        return os;
    }

private:
    unsigned rows_ = 0, cols_ = 0;
    std::vector<T> data_;
};

// ---------------------------------------------------------------------------
namespace sddmm_host {

// Sorted, de-duplicated triplets (CSR.hpp:172-173, COO.hpp:39-40).
template <class T>
std::vector<Triplet<T>> canonical(std::vector<Triplet<T>> t) {
    std::stable_sort(t.begin(), t.end(), [](const Triplet<T> &a, const Triplet<T> &b) { return a < b; });
    t.erase(std::unique(t.begin(), t.end(), [](const Triplet<T> &a, const Triplet<T> &b) { return a == b; }), t.end());
    return t;
}

template <class T>
bool values_match(const std::vector<T> &got, const std::vector<T> &expected) {
    if (got.size() != expected.size()) return false;
    if (std::is_integral<T>::value) return got == expected;
    for (size_t i = 0; i < got.size(); ++i) {
        const double g = (double)got[i], e = (double)expected[i];
        if (g == e) continue;
        if (!(std::fabs(e - g) <= 1e-3 * std::fabs(e))) return false;   // also rejects NaN
    }
    return true;
}

// What CSR and COO share: dimensions, column indices, values.
template <class T>
class SparseBase {
public:
    int getRows() const { return rows; }
    int getCols() const { return cols; }
    void clearValues() { std::fill(values.begin(), values.end(), static_cast<T>(0)); }
    std::vector<T> &getValues() { return values; }
    const std::vector<T> &getValues() const { return values; }
    void setValues(const std::vector<T> &v) { values = v; }
    const std::vector<int> &getColPositions() const { return colPositions; }
    void setColPositions(const std::vector<int> &c) { colPositions = c; }
    const std::vector<int> &getRowPositions() const { return rowPositions; }
    void setRowPositions(const std::vector<int> &r) { rowPositions = r; }
    T *getValue(int j) {
        assert((size_t)j < values.size());
        return &values[(size_t)j];
    }

protected:
    int rows = 0, cols = 0;
    std::vector<int> rowPositions;   // CSR: rows+1 offsets; COO: one row index per entry
    std::vector<int> colPositions;
    std::vector<T> values;

    bool same_as(const SparseBase &o) const {
        const bool pattern = rows == o.rows && cols == o.cols && rowPositions == o.rowPositions &&
                             colPositions == o.colPositions;
        if (!pattern) std::cout << "Cols and Rows don't match" << std::endl;
        return pattern && values_match(values, o.values);
    }
    void print(std::ostream &os, bool values_first) const {
        auto line = [&os](const auto &v) { for (const auto &x : v) os << x << " "; os << std::endl; };
        if (values_first) { line(values); line(colPositions); line(rowPositions); }
        else { line(rowPositions); line(colPositions); line(values); }
    }
};

}  // namespace sddmm_host

template <class T> class CSR;

// ---------------------------------------------------------------------------
// Coordinate format, entries sorted by (row, col) (src/matrices/COO.hpp:27-74).
template <class T>
class COO : public sddmm_host::SparseBase<T> {
    using Base = sddmm_host::SparseBase<T>;

public:
    COO() = default;
    COO(int rows, int cols, std::vector<Triplet<T>> triplets) {
        assert(!triplets.empty());
        this->rows = rows;
        this->cols = cols;
        const auto t = sddmm_host::canonical(std::move(triplets));
        this->rowPositions.reserve(t.size());
        this->colPositions.reserve(t.size());
        this->values.reserve(t.size());
        for (const auto &e : t) {
            assert(e.row >= 0 && e.row < rows && e.col >= 0 && e.col < cols);
            this->rowPositions.push_back(e.row);
            this->colPositions.push_back(e.col);
            this->values.push_back(e.value);
        }
    }
    COO(const COO &) = default;
    COO &operator=(const COO &) = default;
    explicit COO(CSR<T> &csr);   // COO.hpp:55-74, defined below
    // the reference's lhs is the computed result, rhs the expected one (benchmark.hpp:88)
    friend bool operator==(const COO &got, const COO &expected) { return got.same_as(expected); }
    friend std::ostream &operator<<(std::ostream &os, const COO &m) {
        m.print(os, false);
        return os;
    }
};

// ---------------------------------------------------------------------------
// Compressed sparse rows (src/matrices/CSR.hpp:25-50, 162-194) plus the
// nnz-balanced row partition (CSR.hpp:149-155, 196-264).
template <class T>
class CSR : public sddmm_host::SparseBase<T> {
public:
    CSR() = default;
    CSR(int rows, int cols, std::vector<Triplet<T>> triplets) {
        this->rows = rows;
        this->cols = cols;
        build(std::move(triplets));
    }
    CSR(const CSR &) = default;
    CSR &operator=(const CSR &) = default;
    explicit CSR(COO<T> &coo) {
        this->rows = coo.getRows();
        this->cols = coo.getCols();
        const size_t n = coo.getValues().size();
        std::vector<Triplet<T>> t(n);
        for (size_t i = 0; i < n; ++i)
            t[i] = Triplet<T>{coo.getRowPositions()[i], coo.getColPositions()[i], coo.getValues()[i]};
        build(std::move(t));
    }
    friend bool operator==(const CSR &got, const CSR &expected) { return got.same_as(expected); }
    friend std::ostream &operator<<(std::ostream &os, const CSR &m) {
        m.print(os, true);
        return os;
    }

    const std::vector<int> &getStartIdx() const { return startIdx; }
    void computeDispatcher(int numThreads) { partition(numThreads, 1); }
    void computeDispatcherTensorCores(int nbThreads) { partition(nbThreads, 16); }
    double getDensity() const { return (double)this->values.size() / ((double)this->rows * (double)this->cols); }

private:
    std::vector<int> startIdx;

    void build(std::vector<Triplet<T>> triplets) {
        assert(!triplets.empty());
        const auto t = sddmm_host::canonical(std::move(triplets));
        this->rowPositions.assign((size_t)this->rows + 1, 0);
        this->colPositions.clear();
        this->values.clear();
        this->colPositions.reserve(t.size());
        this->values.reserve(t.size());
        // the reference walks rows 0..rows-1 and stops at the first triplet whose row
        // is not the current one, so an out-of-range row ends the matrix there
        size_t idx = 0;
        for (int r = 0; r < this->rows; ++r) {
            this->rowPositions[(size_t)r] = (int)idx;
            while (idx < t.size() && t[idx].row == r) {
                this->colPositions.push_back(t[idx].col);
                this->values.push_back(t[idx].value);
                ++idx;
            }
        }
        this->rowPositions[(size_t)this->rows] = (int)idx;
    }

    void partition(int parts, int stride) {
        startIdx.assign((size_t)parts + 1, this->rows);
        const int rc = sddmm_partition_rows(this->rows, this->rowPositions.data(), parts, stride, startIdx.data());
        assert(rc == 0);
        (void)rc;
    }
};

template <class T>
COO<T>::COO(CSR<T> &csr) {
    this->rows = csr.getRows();
    this->cols = csr.getCols();
    const auto &rp = csr.getRowPositions();
    this->colPositions = csr.getColPositions();
    this->values = csr.getValues();
    this->rowPositions.resize(this->values.size());
    for (int r = 0; r < this->rows; ++r)
        std::fill(this->rowPositions.begin() + rp[(size_t)r], this->rowPositions.begin() + rp[(size_t)r + 1], r);
}
