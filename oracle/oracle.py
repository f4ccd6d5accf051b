"""ctypes front end of the CPU oracle + a numpy restatement.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module; the product (dphpc_amd) never does.

* `sddmm_csr` / `sddmm_coo` call oracle/liboracle.so (sddmm_oracle.c), the C
  restatement of src/competitors/cpu/cpu_basic.hpp:18-51.
* `sddmm_csr_numpy` is an independent numpy restatement of the same loop
  (fp32 multiply, fp32 add, k ascending, then scale by S) used to cross-check the
  C file; it is bit-identical by construction because numpy performs the same two
  fp32 operations per k on every stored entry.
* `Ref` wraps oracle/_ref/libdphpc_ref.so, the reference's own headers compiled
  in place, when that library has been built.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_REF = os.path.join(_HERE, "_ref", "libdphpc_ref.so")

_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is mounted)."""
    if force or not os.path.exists(_LIB):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        L = C.CDLL(_LIB)
        L.oracle_sddmm_csr_f32.argtypes = [C.c_int, C.c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f32p]
        L.oracle_sddmm_csr_f32.restype = None
        L.oracle_sddmm_csr_f32_omp.argtypes = [C.c_int, C.c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f32p, C.c_int]
        L.oracle_sddmm_csr_f32_omp.restype = None
        L.oracle_sddmm_coo_f32.argtypes = [C.c_int64, C.c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f32p]
        L.oracle_sddmm_coo_f32.restype = None
        L.oracle_sddmm_csr_f64.argtypes = [C.c_int, C.c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f64p, _f64p]
        L.oracle_sddmm_csr_f64.restype = None
        L.oracle_fusedmm_csr_f32.argtypes = [C.c_int, C.c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f32p, _f32p]
        L.oracle_fusedmm_csr_f32.restype = None
        L.oracle_fusedmm_csr_f64.argtypes = [C.c_int, C.c_int, _i32p, _i32p, _f32p, _f32p, _f32p, _f64p, _f64p]
        L.oracle_fusedmm_csr_f64.restype = None
        L.oracle_triplets_sort_unique.argtypes = [C.c_int64, _i32p, _i32p, _f32p]
        L.oracle_triplets_sort_unique.restype = C.c_int64
        L.oracle_csr_from_triplets.argtypes = [C.c_int, C.c_int64, _i32p, _i32p, _f32p, _i32p, _i32p, _f32p]
        L.oracle_csr_from_triplets.restype = C.c_int64
        L.oracle_coo_from_csr.argtypes = [C.c_int, _i32p, _i32p]
        L.oracle_coo_from_csr.restype = None
        L.oracle_dispatch.argtypes = [C.c_int, _i32p, C.c_int, C.c_int, _i32p]
        L.oracle_dispatch.restype = C.c_int
        L.oracle_density.argtypes = [C.c_int, C.c_int, C.c_int64]
        L.oracle_density.restype = C.c_double
        L.oracle_max_threads.restype = C.c_int
        L.oracle_compare.argtypes = [C.c_int64, _f32p, _f32p, C.c_void_p, C.c_double, C.c_double, C.POINTER(C.c_int64)]
        L.oracle_compare.restype = C.c_double
        _lib = L
    return _lib


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def sddmm_csr(rowptr, col, sval, A, B, threads=1):
    """P values in CSR order.  threads=1 is the reference's serial loop."""
    rowptr, col, sval = _c(rowptr, np.int32), _c(col, np.int32), _c(sval, np.float32)
    A, B = _c(A, np.float32), _c(B, np.float32)
    M, K = len(rowptr) - 1, A.shape[1]
    assert A.shape[0] >= M and B.shape[1] == K
    P = np.zeros(len(col), np.float32)
    if threads == 1:
        lib().oracle_sddmm_csr_f32(M, K, rowptr, col, sval, A, B, P)
    else:
        lib().oracle_sddmm_csr_f32_omp(M, K, rowptr, col, sval, A, B, P, threads)
    return P


def sddmm_coo(row, col, sval, A, B):
    row, col, sval = _c(row, np.int32), _c(col, np.int32), _c(sval, np.float32)
    A, B = _c(A, np.float32), _c(B, np.float32)
    P = np.zeros(len(col), np.float32)
    lib().oracle_sddmm_coo_f32(len(col), A.shape[1], row, col, sval, A, B, P)
    return P


def sddmm_csr_f64(rowptr, col, sval, A, B):
    """(S*dot, |S|*sum|a*b|) accumulated in double: error analysis / tolerance floor."""
    rowptr, col, sval = _c(rowptr, np.int32), _c(col, np.int32), _c(sval, np.float32)
    A, B = _c(A, np.float32), _c(B, np.float32)
    d = np.zeros(len(col), np.float64)
    m = np.zeros(len(col), np.float64)
    lib().oracle_sddmm_csr_f64(len(rowptr) - 1, A.shape[1], rowptr, col, sval, A, B, d, m)
    return d, m


def fusedmm_csr(rowptr, col, sval, A, B):
    """(P, O): SDDMM values and O = P @ B over the same pattern, fp32 in storage order."""
    rowptr, col, sval = _c(rowptr, np.int32), _c(col, np.int32), _c(sval, np.float32)
    A, B = _c(A, np.float32), _c(B, np.float32)
    M, K = len(rowptr) - 1, A.shape[1]
    P = np.zeros(len(col), np.float32)
    Out = np.zeros((M, K), np.float32)
    lib().oracle_fusedmm_csr_f32(M, K, rowptr, col, sval, A, B, P, Out)
    return P, Out


def fusedmm_csr_f64(rowptr, col, sval, A, B):
    """(O, magnitude) in double: error analysis / tolerance floor of the fused result."""
    rowptr, col, sval = _c(rowptr, np.int32), _c(col, np.int32), _c(sval, np.float32)
    A, B = _c(A, np.float32), _c(B, np.float32)
    M, K = len(rowptr) - 1, A.shape[1]
    o = np.zeros((M, K), np.float64)
    m = np.zeros((M, K), np.float64)
    lib().oracle_fusedmm_csr_f64(M, K, rowptr, col, sval, A, B, o, m)
    return o, m


def sddmm_csr_numpy(rowptr, col, sval, A, B):
    """numpy restatement of cpu_basic.hpp:18-36 (vectorised over entries, k sequential)."""
    rowptr = np.asarray(rowptr, np.int64)
    col = np.asarray(col, np.int64)
    A = np.asarray(A, np.float32)
    B = np.asarray(B, np.float32)
    rows = np.repeat(np.arange(len(rowptr) - 1, dtype=np.int64), np.diff(rowptr))
    return sddmm_coo_numpy(rows, col, sval, A, B)


def sddmm_coo_numpy(row, col, sval, A, B):
    """numpy restatement of cpu_basic.hpp:38-51."""
    row = np.asarray(row, np.int64)
    col = np.asarray(col, np.int64)
    A = np.asarray(A, np.float32)
    B = np.asarray(B, np.float32)
    acc = np.zeros(len(col), np.float32)
    for k in range(A.shape[1]):
        acc = (acc + (A[row, k] * B[col, k]).astype(np.float32)).astype(np.float32)
    return (acc * np.asarray(sval, np.float32)).astype(np.float32)


def csr_from_triplets(rows, row, col, val):
    row, col, val = _c(row, np.int32).copy(), _c(col, np.int32).copy(), _c(val, np.float32).copy()
    n = len(row)
    rowptr = np.zeros(rows + 1, np.int32)
    oc = np.zeros(max(n, 1), np.int32)
    ov = np.zeros(max(n, 1), np.float32)
    nnz = lib().oracle_csr_from_triplets(rows, n, row, col, val, rowptr, oc, ov)
    return rowptr, oc[:nnz].copy(), ov[:nnz].copy()


def coo_from_triplets(row, col, val):
    row, col, val = _c(row, np.int32).copy(), _c(col, np.int32).copy(), _c(val, np.float32).copy()
    n = lib().oracle_triplets_sort_unique(len(row), row, col, val)
    return row[:n].copy(), col[:n].copy(), val[:n].copy()


def coo_rows_from_csr(rowptr):
    rowptr = _c(rowptr, np.int32)
    out = np.zeros(int(rowptr[-1]), np.int32)
    lib().oracle_coo_from_csr(len(rowptr) - 1, rowptr, out)
    return out


def dispatch(rowptr, parts, stride=1):
    rowptr = _c(rowptr, np.int32)
    out = np.zeros(parts + 1, np.int32)
    n = lib().oracle_dispatch(len(rowptr) - 1, rowptr, parts, stride, out)
    if n < 0:
        raise ValueError("oracle_dispatch: bad arguments")
    return out[:n].copy()


def density(rows, cols, nnz):
    return lib().oracle_density(rows, cols, nnz)


def max_threads():
    return lib().oracle_max_threads()


# --------------------------------------------------------------------------
def check_values(got, ref, mag=None, rtol=1e-5, floor=0.25):
    """The value comparator used by every parity test.

    |got-ref| <= rtol * max(|ref|, floor*mag) where mag = |S|*sum_k|a_k b_k| is the
    cancellation-free magnitude of the entry (from `sddmm_csr_f64`).  With mag=None
    it is the plain relative test.  Unlike the reference's operator== (CSR.hpp:92-94)
    the denominator is |ref|, so negative and zero reference values are handled.
    Returns (ok, worst_ratio, index_of_worst)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    if got.shape != ref.shape:
        return False, np.inf, -1
    if got.size == 0:
        return True, 0.0, -1
    scale = np.abs(ref)
    if mag is not None:
        scale = np.maximum(scale, floor * np.asarray(mag, np.float64))
    err = np.abs(got - ref)
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(err == 0, 0.0, err / (rtol * scale))
    ratio = np.nan_to_num(ratio, nan=np.inf, posinf=np.inf)
    i = int(np.argmax(ratio))
    return bool(ratio[i] <= 1.0), float(ratio[i]), i


def check_values_fast(got, ref, mag=None, rtol=1e-5, floor=0.25):
    """`check_values` for large fp32 arrays: the same test in C on all cores
    (oracle_compare); tests/test_oracle.py holds the two to the same answers."""
    got, ref = _c(got, np.float32), _c(ref, np.float32)
    if got.shape != ref.shape:
        return False, np.inf, -1
    if got.size == 0:
        return True, 0.0, -1
    m = None if mag is None else _c(mag, np.float64)
    at = C.c_int64(-1)
    worst = lib().oracle_compare(got.size, got.ravel(), ref.ravel(), None if m is None else m.ctypes.data_as(C.c_void_p),
                                 float(rtol), float(floor), C.byref(at))
    return bool(worst <= 1.0), float(worst), int(at.value)


class Ref:
    """oracle/_ref/libdphpc_ref.so: the reference's own CPUBasic / CSR / COO."""

    def __init__(self):
        if not os.path.exists(_REF):
            raise FileNotFoundError(_REF)
        L = C.CDLL(_REF)
        L.ref_cpu_basic_csr.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int64, _i32p, _i32p, _f32p, _f32p, _f32p,
                                        _i32p, _i32p, _f32p]
        L.ref_cpu_basic_csr.restype = C.c_int64
        L.ref_cpu_basic_coo.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int64, _i32p, _i32p, _f32p, _f32p, _f32p,
                                        _i32p, _i32p, _f32p, _f32p]
        L.ref_cpu_basic_coo.restype = C.c_int64
        L.ref_cpu_basic_csr_seconds.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int64, _i32p, _i32p, _f32p, _f32p,
                                                _f32p, C.c_int, _f32p]
        L.ref_cpu_basic_csr_seconds.restype = C.c_double
        L.ref_csr_build.argtypes = [C.c_int, C.c_int, C.c_int64, _i32p, _i32p, _f32p, C.c_int, _i32p, _i32p, _f32p]
        L.ref_csr_build.restype = C.c_int64
        L.ref_dispatch.argtypes = [C.c_int, C.c_int, C.c_int64, _i32p, _i32p, _f32p, C.c_int, C.c_int, _i32p, C.c_int]
        L.ref_dispatch.restype = C.c_int
        self.L = L

    @staticmethod
    def available():
        return os.path.exists(_REF)

    def cpu_basic_csr(self, M, N, row, col, val, A, B):
        row, col, val = _c(row, np.int32), _c(col, np.int32), _c(val, np.float32)
        A, B = _c(A, np.float32), _c(B, np.float32)
        n = len(row)
        rp = np.zeros(M + 1, np.int32)
        oc = np.zeros(n, np.int32)
        P = np.zeros(n, np.float32)
        nnz = self.L.ref_cpu_basic_csr(M, N, A.shape[1], n, row, col, val, A, B, rp, oc, P)
        return rp, oc[:nnz].copy(), P[:nnz].copy()

    def cpu_basic_coo(self, M, N, row, col, val, A, B):
        row, col, val = _c(row, np.int32), _c(col, np.int32), _c(val, np.float32)
        A, B = _c(A, np.float32), _c(B, np.float32)
        n = len(row)
        orow = np.zeros(n, np.int32)
        oc = np.zeros(n, np.int32)
        ov = np.zeros(n, np.float32)
        P = np.zeros(n, np.float32)
        nnz = self.L.ref_cpu_basic_coo(M, N, A.shape[1], n, row, col, val, A, B, orow, oc, ov, P)
        return orow[:nnz].copy(), oc[:nnz].copy(), ov[:nnz].copy(), P[:nnz].copy()

    def cpu_basic_csr_seconds(self, M, N, row, col, val, A, B, reps=1):
        row, col, val = _c(row, np.int32), _c(col, np.int32), _c(val, np.float32)
        A, B = _c(A, np.float32), _c(B, np.float32)
        P = np.zeros(len(row), np.float32)
        s = self.L.ref_cpu_basic_csr_seconds(M, N, A.shape[1], len(row), row, col, val, A, B, reps, P)
        return s, P

    def csr_build(self, M, N, row, col, val, via_coo=False):
        row, col, val = _c(row, np.int32), _c(col, np.int32), _c(val, np.float32)
        n = len(row)
        rp = np.zeros(M + 1, np.int32)
        oc = np.zeros(n, np.int32)
        ov = np.zeros(n, np.float32)
        nnz = self.L.ref_csr_build(M, N, n, row, col, val, int(via_coo), rp, oc, ov)
        return rp, oc[:nnz].copy(), ov[:nnz].copy()

    def dispatch(self, M, N, row, col, val, parts, stride=1):
        row, col, val = _c(row, np.int32), _c(col, np.int32), _c(val, np.float32)
        out = np.zeros(parts + 64, np.int32)
        n = self.L.ref_dispatch(M, N, len(row), row, col, val, parts, stride, out, len(out))
        if n < 0:
            raise ValueError("ref_dispatch failed: %d" % n)
        return out[:n].copy()
