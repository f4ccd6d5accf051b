"""sddmm_launch_noalloc: the entry point that allocates nothing (the row index per
stored entry lives in a static device array of the library).  Its output must equal,
bit for bit, what the context-based entry points give with the flat strategy on the
same operands (same kernels), and meet the oracle's bar -- on two calls in a row, the
second on a smaller input, so that whatever the first call left in the shared array
cannot leak into the second."""
import ctypes as C

import numpy as np
import pytest

from dphpc_amd import capi, workloads as W
from oracle import oracle as O

pytestmark = pytest.mark.gpu
f32 = np.float32


class Hip:
    def __init__(self):
        self.h = C.CDLL("libamdhip64.so")
        self.h.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.h.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.h.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        self.h.hipFree.argtypes = [C.c_void_p]
        self.live = []

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = C.c_void_p()
        assert self.h.hipMalloc(C.byref(p), max(a.nbytes, 16)) == 0
        assert self.h.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), a.nbytes, 1) == 0     # host to device
        self.live.append(p)
        return p

    def zeros(self, nbytes):
        p = C.c_void_p()
        assert self.h.hipMalloc(C.byref(p), max(nbytes, 16)) == 0
        assert self.h.hipMemset(p, 0, max(nbytes, 16)) == 0
        self.live.append(p)
        return p

    def download(self, p, n, dtype):
        out = np.empty(n, dtype)
        assert self.h.hipDeviceSynchronize() == 0
        assert self.h.hipMemcpy(out.ctypes.data_as(C.c_void_p), p, out.nbytes, 2) == 0  # device to host
        return out

    def free_all(self):
        for p in self.live:
            self.h.hipFree(p)
        self.live = []


def _flat_through_a_context(w):
    with capi.Engine(0) as e:
        e.set_dense(w.A, w.B)
        e.set_csr(w.M, w.N, w.rowptr, w.col, w.sval)
        e.plan(capi.FLAT)
        e.run()
        return e.values()


def _noalloc(L, hip, w):
    dA, dB = hip.upload(w.A), hip.upload(w.B)
    d_rp, d_col, d_val = hip.upload(w.rowptr), hip.upload(w.col), hip.upload(w.sval)
    dP = hip.zeros(4 * w.nnz)
    rc = L.sddmm_launch_noalloc(w.M, w.N, w.K, w.nnz, dA, dB, d_rp, d_col, d_val, dP, None)
    assert rc == 0, L.sddmm_strerror(rc)
    return hip.download(dP, w.nnz, f32)


def test_two_calls_in_a_row_the_second_smaller():
    L = capi.load_library()
    hip = Hip()
    try:
        # first a large input (power-law rows: lengths from 1 to thousands), then a smaller one
        # with another shape and another K; then the first again
        big = W.make("power_law", "small", K=32)
        small = W.make("mixed_density", "small", K=48)
        assert small.nnz < big.nnz
        for w in (big, small, big):
            got = _noalloc(L, hip, w)
            want = _flat_through_a_context(w)
            np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
            ref = O.sddmm_csr(w.rowptr, w.col, w.sval, w.A, w.B, threads=0)
            _, mag = O.sddmm_csr_f64(w.rowptr, w.col, w.sval, w.A, w.B)
            ok, worst, i = O.check_values(got, ref, mag=mag)
            assert ok, (w.name, i, worst)
            hip.free_all()
    finally:
        hip.free_all()


def test_rows_of_any_width_and_empty_input():
    """K not a multiple of 4 (one fp32 per lane) and K beyond the register layout take
    the same flat kernel variants as a context does; nnz = 0 launches nothing."""
    L = capi.load_library()
    hip = Hip()
    rng = np.random.default_rng(12)
    try:
        for K in (5, 100, 260):
            M, N = 180, 150
            mask = rng.random((M, N)) < 0.07
            mask[3] = False
            r, c = np.nonzero(mask)
            v = rng.uniform(-1, 1, len(r)).astype(f32)
            rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
            w = W.Workload("random", M, N, K, rowptr, col, val, rng.uniform(-1, 1, (M, K)).astype(f32),
                           rng.uniform(-1, 1, (N, K)).astype(f32))
            got = _noalloc(L, hip, w)
            np.testing.assert_array_equal(got.view(np.uint32), _flat_through_a_context(w).view(np.uint32))
            ok, worst, i = O.check_values(got, O.sddmm_csr(rowptr, col, val, w.A, w.B),
                                          mag=O.sddmm_csr_f64(rowptr, col, val, w.A, w.B)[1])
            assert ok, (K, i, worst)
            hip.free_all()
        d_rp = hip.upload(np.zeros(11, np.int32))
        assert L.sddmm_launch_noalloc(10, 10, 8, 0, None, None, d_rp, None, None, None, None) == 0
    finally:
        hip.free_all()


def test_sizes_beyond_the_static_buffer_and_bad_arguments_are_refused():
    """Refused on the host, before anything is launched: the pointers are never touched."""
    L = capi.load_library()
    hip = Hip()
    try:
        d = hip.zeros(64)
        too_many = capi.NOALLOC_MAX_NNZ + 1
        assert L.sddmm_launch_noalloc(10, 10, 32, too_many, d, d, d, d, d, d, None) == capi.ERR_TOO_LARGE
        assert b"SDDMM_NOALLOC_MAX_NNZ" in L.sddmm_strerror(capi.ERR_TOO_LARGE)
        assert L.sddmm_launch_noalloc(10, 10, 0, 5, d, d, d, d, d, d, None) == capi.ERR_INVALID
        assert L.sddmm_launch_noalloc(-1, 10, 8, 5, d, d, d, d, d, d, None) == capi.ERR_INVALID
        assert L.sddmm_launch_noalloc(10, 10, 8, 5, d, d, None, d, d, d, None) == capi.ERR_NULL
        assert L.sddmm_launch_noalloc(10, 10, 8, 5, d, d, d, d, d, None, None) == capi.ERR_NULL
        assert L.sddmm_launch_noalloc(10, 10, 8, 5, C.c_void_p(d.value + 4), d, d, d, d, d, None) == capi.ERR_INVALID
    finally:
        hip.free_all()


def test_row_pointer_beyond_nnz_writes_nothing_outside_the_output():
    """A row pointer whose tail runs past the nnz argument (the structure is not validated by
    this entry point) must not make the library write outside its own array or outside
    P[0, nnz): the entries below nnz come out as usual, a guard area behind P stays untouched."""
    L = capi.load_library()
    hip = Hip()
    try:
        w = W.make("mixed_density", "small", K=32)
        cut = int(w.rowptr[w.M // 2])                  # entries of the first half of the rows
        assert 0 < cut < w.nnz
        bad_rowptr = w.rowptr.copy()
        bad_rowptr[w.M // 2 + 1:] += 1 << 26           # far beyond nnz and beyond the static array
        bad_rowptr[-1] = np.iinfo(np.int32).max
        dA, dB = hip.upload(w.A), hip.upload(w.B)
        d_rp, d_col, d_val = hip.upload(bad_rowptr), hip.upload(w.col), hip.upload(w.sval)
        guard = 4096
        sentinel = np.full(cut + guard, -123.25, f32)
        dP = hip.upload(sentinel)
        # first a good call, so that every row index the flat kernel may read below is a valid row
        good = _noalloc(L, hip, w)
        rc = L.sddmm_launch_noalloc(w.M, w.N, w.K, cut, dA, dB, d_rp, d_col, d_val, dP, None)
        assert rc == 0, L.sddmm_strerror(rc)
        got = hip.download(dP, cut + guard, f32)
        np.testing.assert_array_equal(got[cut:], sentinel[cut:])
        np.testing.assert_array_equal(got[:cut].view(np.uint32), good[:cut].view(np.uint32))
    finally:
        hip.free_all()


def test_under_graph_capture_and_without_allocating():
    """What the entry point is for: after the warm-up call (nnz = 0, outside the capture) one call
    is captured into a HIP graph -- kernels only -- and the graph launched twice, with eager work
    in between; both replays give the flat strategy's values.  The free device memory is the same
    before and after an eager call."""
    L = capi.load_library()
    hip = Hip()
    h = hip.h
    vp = C.c_void_p
    h.hipStreamCreate.argtypes = [C.POINTER(vp)]
    h.hipStreamDestroy.argtypes = [vp]
    h.hipStreamSynchronize.argtypes = [vp]
    h.hipStreamBeginCapture.argtypes = [vp, C.c_int]
    h.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
    h.hipGraphInstantiate.argtypes = [C.POINTER(vp), vp, vp, vp, C.c_size_t]
    h.hipGraphLaunch.argtypes = [vp, vp]
    h.hipGraphExecDestroy.argtypes = [vp]
    h.hipGraphDestroy.argtypes = [vp]
    h.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    h.hipMemsetAsync.argtypes = [vp, C.c_int, C.c_size_t, vp]
    stream, graph, gexec = vp(), vp(), vp()
    try:
        w = W.make("power_law", "small", K=32)
        want = _flat_through_a_context(w)
        dA, dB = hip.upload(w.A), hip.upload(w.B)
        d_rp, d_col, d_val = hip.upload(w.rowptr), hip.upload(w.col), hip.upload(w.sval)
        dP = hip.zeros(4 * w.nnz)
        assert h.hipStreamCreate(C.byref(stream)) == 0
        assert L.sddmm_launch_noalloc(w.M, w.N, w.K, 0, None, None, d_rp, None, None, None, stream) == 0   # warm-up
        assert L.sddmm_launch_noalloc(w.M, w.N, w.K, w.nnz, dA, dB, d_rp, d_col, d_val, dP, stream) == 0   # code loaded
        assert h.hipStreamSynchronize(stream) == 0
        free0, free1, total = C.c_size_t(), C.c_size_t(), C.c_size_t()
        assert h.hipMemGetInfo(C.byref(free0), C.byref(total)) == 0
        assert L.sddmm_launch_noalloc(w.M, w.N, w.K, w.nnz, dA, dB, d_rp, d_col, d_val, dP, stream) == 0
        assert h.hipStreamSynchronize(stream) == 0
        assert h.hipMemGetInfo(C.byref(free1), C.byref(total)) == 0
        assert free0.value == free1.value

        assert h.hipStreamBeginCapture(stream, 0) == 0                       # hipStreamCaptureModeGlobal
        rc = L.sddmm_launch_noalloc(w.M, w.N, w.K, w.nnz, dA, dB, d_rp, d_col, d_val, dP, stream)
        assert h.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert rc == 0, L.sddmm_strerror(rc)
        assert h.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for replay in range(2):
            assert h.hipMemsetAsync(dP, 0, 4 * w.nnz, stream) == 0           # eager work between the replays
            assert h.hipStreamSynchronize(stream) == 0
            assert h.hipGraphLaunch(gexec, stream) == 0
            assert h.hipStreamSynchronize(stream) == 0
            got = hip.download(dP, w.nnz, f32)
            np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32), err_msg="replay %d" % replay)
    finally:
        if gexec:
            h.hipGraphExecDestroy(gexec)
        if graph:
            h.hipGraphDestroy(graph)
        if stream:
            h.hipStreamDestroy(stream)
        hip.free_all()
