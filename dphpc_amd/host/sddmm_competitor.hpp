// The plugin interface of the reference harness (src/benchmark/competitor.hpp:12-60),
// restated so that this repository's adapter and tests compile without the
// reference tree.  Same names, same phases, same defaults (1 thread block of 1
// thread, echoed in the CSV columns 13-14 by src/benchmark/benchmark.hpp:95-98).
#pragma once

#include <string>

#include "sddmm_containers.hpp"

namespace SDDMM {

template <typename T>
class Competitor {
public:
    const std::string name;

    explicit Competitor(const std::string &n) : name(n) {}
    Competitor(const std::string &n, int threads_per_block, int thread_blocks)
        : name(n), threads_per_block_(threads_per_block), thread_blocks_(thread_blocks) {}
    virtual ~Competitor() = default;

    // init: allocate, upload, preprocess (timed as init_ns)
    virtual void init_csr(Dense<T> &, Dense<T> &, CSR<T> &, CSR<T> &) {}
    virtual void init_coo(Dense<T> &, Dense<T> &, COO<T> &, COO<T> &) {}
    // run: compute; complete on return (timed as comp_ns)
    virtual void run_csr(Dense<T> &A, Dense<T> &B, CSR<T> &S, CSR<T> &P) = 0;
    virtual void run_coo(Dense<T> &A, Dense<T> &B, COO<T> &S, COO<T> &P) = 0;
    // cleanup: download into P, release (timed as cleanup_ns)
    virtual void cleanup_csr(Dense<T> &, Dense<T> &, CSR<T> &, CSR<T> &) {}
    virtual void cleanup_coo(Dense<T> &, Dense<T> &, COO<T> &, COO<T> &) {}

    virtual bool csr_supported() = 0;
    virtual bool coo_supported() = 0;
    virtual bool is_gpu() { return false; }

    void set_num_threads_per_block(int n) { threads_per_block_ = n; }
    int get_num_threads_per_block() { return threads_per_block_; }
    void set_num_thread_blocks(int n) { thread_blocks_ = n; }
    int get_num_thread_blocks() { return thread_blocks_; }

private:
    int threads_per_block_ = 1;
    int thread_blocks_ = 1;
};

}  // namespace SDDMM
