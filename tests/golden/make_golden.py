#!/usr/bin/env python3
"""Writes the golden fixtures under tests/golden/ from the REFERENCE's own CPU path.

Runs in the build container only (it needs oracle/_ref/libdphpc_ref.so, i.e. the
reference's src/competitors/cpu/cpu_basic.hpp and src/matrices/*.hpp compiled in
place by oracle/Makefile).  Inputs are this repository's seeded workloads; the
expected values are what the reference's CPUBasic<float>::run_csr returns on them.

  small_uniform_K32.npz   benchmark config 1 at full size: complete inputs and P
  sampled_<name>_K<k>.npz scaled-down configs 2-5: 4096 sampled entries (position,
                          expected value) and a float64 sum of all expected values;
                          the inputs are regenerated from the seeds by the tests
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from dphpc_amd import workloads as W  # noqa: E402
from oracle import oracle as O  # noqa: E402

SAMPLED = [("fem_banded", 32), ("fem_banded", 128), ("power_law", 32), ("mixed_density", 32),
           ("mixed_density", 64), ("mixed_density", 256), ("dense_tiles", 128), ("dense_tiles", 512)]


def reference_values(ref, w):
    rp, col, P = ref.cpu_basic_csr(w.M, w.N, w.rows(), w.col, w.sval, w.A, w.B)
    assert np.array_equal(rp, w.rowptr) and np.array_equal(col, w.col), "reference CSR constructor changed the pattern"
    return P


def main():
    ref = O.Ref()
    w = W.make("small_uniform")
    P = reference_values(ref, w)
    np.savez_compressed(os.path.join(HERE, "small_uniform_K32.npz"), rowptr=w.rowptr, col=w.col, sval=w.sval,
                        A=w.A, B=w.B, P=P)
    print("small_uniform_K32: nnz", w.nnz)
    for name, K in SAMPLED:
        w = W.make(name, "small", K=K)
        P = reference_values(ref, w)        # for bf16 workloads A,B are the bf16-rounded values in fp32
        rng = np.random.default_rng(12345)
        pos = np.sort(rng.choice(w.nnz, size=min(4096, w.nnz), replace=False)).astype(np.int64)
        np.savez_compressed(os.path.join(HERE, "sampled_%s_K%d.npz" % (name, K)), nnz=np.int64(w.nnz), pos=pos,
                            val=P[pos], total=np.float64(P.astype(np.float64).sum()),
                            col_sum=np.int64(w.col.astype(np.int64).sum()))
        print("sampled_%s_K%d: nnz %d" % (name, K, w.nnz))


if __name__ == "__main__":
    main()
