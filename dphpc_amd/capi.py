"""ctypes binding of include/sddmm_amd.h.

There is no fallback: if the HIP library is missing `load_library` raises, and if
no GPU is present `Engine()` raises SddmmError(SDDMM_ERR_NO_DEVICE).
"""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
# SDDMM_LIB selects another build of the same library (kernel experiments)
_LIB_PATH = os.environ.get("SDDMM_LIB") or os.path.join(_PKG, "lib", "libsddmm_amd.so")

AUTO, FLAT, ROW_WAVE, SHORT_ROWS, LDS_TILED, MFMA_TILE, EXACT = range(7)
STRATEGY_NAMES = ["AUTO", "FLAT", "ROW_WAVE", "SHORT_ROWS", "LDS_TILED", "MFMA_TILE", "EXACT"]
F32, BF16, F16 = 0, 1, 2

OK, ERR_INVALID, ERR_NULL, ERR_STATE, ERR_ALLOC, ERR_HIP, ERR_UNSUPPORTED, ERR_NO_DEVICE, ERR_PATTERN = (
    0, -1, -2, -3, -4, -5, -6, -7, -8)
ERR_TOO_LARGE = -9
NOALLOC_MAX_NNZ = 1 << 24

# every symbol include/sddmm_amd.h declares
EXPORTS = [
    "sddmm_create", "sddmm_destroy", "sddmm_strerror", "sddmm_last_error", "sddmm_set_stream", "sddmm_get_stream",
    "sddmm_set_dense", "sddmm_set_dense_device", "sddmm_set_csr", "sddmm_set_coo",
    "sddmm_set_csr_device", "sddmm_set_coo_device", "sddmm_update_values", "sddmm_plan", "sddmm_run",
    "sddmm_launch", "sddmm_synchronize", "sddmm_time_runs", "sddmm_time_region", "sddmm_run_fused",
    "sddmm_get_fused", "sddmm_get_fused_device", "sddmm_get_values",
    "sddmm_get_values_device", "sddmm_last_stats", "sddmm_partition_rows", "sddmm_version",
    "sddmm_launch_noalloc",
]


class Stats(C.Structure):
    _fields_ = [
        ("plan_ms", C.c_float), ("run_ms", C.c_float),
        ("strategy_used", C.c_int32), ("kernels_launched", C.c_int32),
        ("nnz", C.c_int64), ("rows_nonempty", C.c_int64),
        ("rows_short", C.c_int64), ("rows_medium", C.c_int64), ("rows_long", C.c_int64),
        ("nnz_short", C.c_int64), ("nnz_medium", C.c_int64), ("nnz_long", C.c_int64),
        ("mfma_tiles", C.c_int64), ("nnz_mfma", C.c_int64), ("cols_touched", C.c_int64),
        ("flops", C.c_double), ("bytes_gathered", C.c_double),
        ("panels", C.c_int64), ("nnz_panel", C.c_int64),
    ]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


class SddmmError(RuntimeError):
    def __init__(self, code, msg=""):
        self.code = code
        super().__init__("sddmm error %d: %s" % (code, msg))


def library_path():
    return _LIB_PATH


_lib = None


def load_library():
    """Load the built HIP library (built on first use only if absent)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        from . import build
        build.build_library()
    L = C.CDLL(_LIB_PATH)
    vp, i32, i64 = C.c_void_p, C.c_int, C.c_int64
    L.sddmm_create.argtypes = [C.POINTER(vp), i32]
    L.sddmm_destroy.argtypes = [vp]
    L.sddmm_destroy.restype = None
    L.sddmm_strerror.argtypes = [i32]
    L.sddmm_strerror.restype = C.c_char_p
    L.sddmm_last_error.argtypes = [vp]
    L.sddmm_last_error.restype = C.c_char_p
    L.sddmm_set_stream.argtypes = [vp, vp, i32]
    L.sddmm_get_stream.argtypes = [vp, C.POINTER(vp)]
    L.sddmm_set_dense.argtypes = [vp, i32, i32, i32, vp, vp, i32]
    L.sddmm_set_dense_device.argtypes = [vp, i32, i32, i32, vp, vp, i32]
    L.sddmm_set_csr.argtypes = [vp, i32, i32, i64, vp, vp, vp]
    L.sddmm_set_coo.argtypes = [vp, i32, i32, i64, vp, vp, vp]
    L.sddmm_set_csr_device.argtypes = [vp, i32, i32, i64, vp, vp, vp]
    L.sddmm_set_coo_device.argtypes = [vp, i32, i32, i64, vp, vp, vp]
    L.sddmm_update_values.argtypes = [vp, vp]
    L.sddmm_plan.argtypes = [vp, i32]
    L.sddmm_run.argtypes = [vp]
    L.sddmm_launch.argtypes = [vp]
    L.sddmm_synchronize.argtypes = [vp]
    L.sddmm_time_runs.argtypes = [vp, i32, i32, i32, vp]
    L.sddmm_time_region.argtypes = [vp, i32, i32, C.POINTER(C.c_float)]
    L.sddmm_run_fused.argtypes = [vp]
    L.sddmm_get_fused.argtypes = [vp, vp]
    L.sddmm_get_fused_device.argtypes = [vp, C.POINTER(vp)]
    L.sddmm_get_values.argtypes = [vp, vp]
    L.sddmm_get_values_device.argtypes = [vp, C.POINTER(vp)]
    L.sddmm_last_stats.argtypes = [vp, C.POINTER(Stats)]
    L.sddmm_partition_rows.argtypes = [i32, vp, i32, i32, vp]
    L.sddmm_version.restype = C.c_char_p
    L.sddmm_launch_noalloc.argtypes = [i32, i32, i32, i64, vp, vp, vp, vp, vp, vp, vp]
    _lib = L
    return L


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def to_bf16(x):
    """fp32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def from_bf16(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_f16(x):
    """fp32 -> IEEE half bit patterns (uint16), round to nearest even."""
    return np.ascontiguousarray(x, np.float32).astype(np.float16).view(np.uint16)


def from_f16(b):
    return np.ascontiguousarray(b, np.uint16).view(np.float16).astype(np.float32)


def partition_rows(rowptr, parts, stride=1):
    """Host helper: nnz-balanced contiguous row ranges (start indices, parts+1)."""
    L = load_library()
    rowptr = np.ascontiguousarray(rowptr, np.int32)
    out = np.zeros(parts + 1, np.int32)
    rc = L.sddmm_partition_rows(len(rowptr) - 1, _ptr(rowptr), parts, stride, _ptr(out))
    if rc:
        raise SddmmError(rc, L.sddmm_strerror(rc).decode())
    return out


class Engine:
    """One sddmm_ctx.  Method names follow the C ABI one to one."""

    def __init__(self, device=0):
        self.L = load_library()
        self.h = C.c_void_p()
        rc = self.L.sddmm_create(C.byref(self.h), device)
        if rc:
            self.h = C.c_void_p()
            raise SddmmError(rc, self.L.sddmm_strerror(rc).decode())
        self.nnz = 0

    def _chk(self, rc):
        if rc:
            raise SddmmError(rc, "%s: %s" % (self.L.sddmm_strerror(rc).decode(),
                                             self.L.sddmm_last_error(self.h).decode()))

    def close(self):
        if self.h:
            self.L.sddmm_destroy(self.h)
            self.h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_dense(self, A, B, dtype=F32):
        if dtype == F32:
            A = np.ascontiguousarray(A, np.float32)
            B = np.ascontiguousarray(B, np.float32)
        else:
            A = np.ascontiguousarray(A, np.uint16)
            B = np.ascontiguousarray(B, np.uint16)
        assert A.ndim == 2 and B.ndim == 2 and A.shape[1] == B.shape[1]
        self._chk(self.L.sddmm_set_dense(self.h, A.shape[0], B.shape[0], A.shape[1], _ptr(A), _ptr(B), dtype))
        self._dense_shape = (A.shape[0], A.shape[1])

    def set_csr(self, M, N, rowptr, col, sval):
        rowptr = np.ascontiguousarray(rowptr, np.int32)
        col = np.ascontiguousarray(col, np.int32)
        sval = np.ascontiguousarray(sval, np.float32)
        self._chk(self.L.sddmm_set_csr(self.h, M, N, len(col), _ptr(rowptr), _ptr(col), _ptr(sval)))
        self.nnz = len(col)

    def set_coo(self, M, N, row, col, sval):
        row = np.ascontiguousarray(row, np.int32)
        col = np.ascontiguousarray(col, np.int32)
        sval = np.ascontiguousarray(sval, np.float32)
        self._chk(self.L.sddmm_set_coo(self.h, M, N, len(col), _ptr(row), _ptr(col), _ptr(sval)))
        self.nnz = len(col)

    def update_values(self, sval):
        sval = np.ascontiguousarray(sval, np.float32)
        assert len(sval) == self.nnz
        self._chk(self.L.sddmm_update_values(self.h, _ptr(sval)))

    def set_stream(self, stream, lent=True):
        """stream: a hipStream_t as an integer (0 = the null stream); lent=False
        returns to the context's own stream."""
        self._chk(self.L.sddmm_set_stream(self.h, C.c_void_p(stream or None), 1 if lent else 0))

    def get_stream(self):
        p = C.c_void_p()
        self._chk(self.L.sddmm_get_stream(self.h, C.byref(p)))
        return p.value or 0

    def plan(self, strategy=AUTO):
        self._chk(self.L.sddmm_plan(self.h, strategy))

    def run(self):
        self._chk(self.L.sddmm_run(self.h))

    def launch(self):
        self._chk(self.L.sddmm_launch(self.h))

    def synchronize(self):
        self._chk(self.L.sddmm_synchronize(self.h))

    def time_runs(self, warmup, reps, include_plan=False):
        ms = np.zeros(max(reps, 1), np.float32)
        self._chk(self.L.sddmm_time_runs(self.h, warmup, reps, int(include_plan), _ptr(ms)))
        return ms[:reps]

    def time_region(self, reps, include_plan=False):
        """Device milliseconds of `reps` launches back to back between one pair of events."""
        total = C.c_float(0.0)
        self._chk(self.L.sddmm_time_region(self.h, reps, int(include_plan), C.byref(total)))
        return float(total.value)

    def run_fused(self, fetch=True):
        """SDDMM followed by SpMM over the same pattern; returns O (M x K, fp32), or nothing
        with fetch=False (stats().run_ms then holds the device time of the launch)."""
        self._chk(self.L.sddmm_run_fused(self.h))
        if not fetch:
            return None
        O = np.empty(self._dense_shape, np.float32)
        self._chk(self.L.sddmm_get_fused(self.h, _ptr(O)))
        return O

    def values(self):
        P = np.empty(self.nnz, np.float32)
        self._chk(self.L.sddmm_get_values(self.h, _ptr(P)))
        return P

    def stats(self):
        s = Stats()
        self._chk(self.L.sddmm_last_stats(self.h, C.byref(s)))
        return s


def sddmm_csr(rowptr, col, sval, A, B, N=None, strategy=AUTO, dtype=F32, device=0):
    """Convenience one-shot: create, upload, plan, run, download, destroy."""
    M = len(rowptr) - 1
    with Engine(device) as e:
        e.set_dense(A, B, dtype)
        e.set_csr(M, B.shape[0] if N is None else N, rowptr, col, sval)
        e.plan(strategy)
        e.run()
        return e.values()


def sddmm_coo(M, row, col, sval, A, B, N=None, strategy=AUTO, dtype=F32, device=0):
    with Engine(device) as e:
        e.set_dense(A, B, dtype)
        e.set_coo(M, B.shape[0] if N is None else N, row, col, sval)
        e.plan(strategy)
        e.run()
        return e.values()
