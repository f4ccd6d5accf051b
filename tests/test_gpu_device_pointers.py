"""Device-resident operands (the *_device entry points) and operands of 4 GiB and
more (64-bit byte offsets in the gather kernels).  HIP memory is managed here with
a few direct runtime calls; the library only borrows the pointers."""
import ctypes as C
import sys

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
        self.h.hipFree.argtypes = [C.c_void_p]
        self.live = []

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = C.c_void_p()
        assert self.h.hipMalloc(C.byref(p), max(a.nbytes, 16)) == 0
        assert self.h.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), a.nbytes, 1) == 0     # host to device
        self.live.append(p)
        return p

    def download(self, p, n, dtype):
        out = np.empty(n, dtype)
        assert self.h.hipMemcpy(out.ctypes.data_as(C.c_void_p), p, out.nbytes, 2) == 0  # device to host
        return out

    def free_all(self):
        for p in self.live:
            self.h.hipFree(p)
        self.live = []


def test_device_resident_operands(engine_factory):
    rng = np.random.default_rng(50)
    M, N, K = 300, 260, 32
    mask = rng.random((M, N)) < 0.1
    r, c = np.nonzero(mask)
    v = rng.uniform(-1, 1, len(r)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r.astype(np.int32), c.astype(np.int32), v)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    ref = O.sddmm_csr(rowptr, col, val, A, B)
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    hip = Hip()
    e = engine_factory()            # creates the context (and selects the device) first
    try:
        dA, dB = hip.upload(A), hip.upload(B)
        d_rp, d_col, d_val = hip.upload(rowptr), hip.upload(col), hip.upload(val)
        L = e.L
        e._chk(L.sddmm_set_dense_device(e.h, M, N, K, dA, dB, capi.F32))
        e.nnz = len(col)
        for strategy in (capi.AUTO, capi.ROW_WAVE, capi.FLAT, capi.EXACT, capi.MFMA_TILE):
            # set again for every strategy: that clears P, so no kernel can pass on the values of the one before
            e._chk(L.sddmm_set_csr_device(e.h, M, N, len(col), d_rp, d_col, d_val))
            e.plan(strategy)
            e.run()
            got = e.values()
            assert O.check_values(got, ref, mag=mag)[0], capi.STRATEGY_NAMES[strategy]
            dP = C.c_void_p()
            e._chk(L.sddmm_get_values_device(e.h, C.byref(dP)))
            np.testing.assert_array_equal(hip.download(dP, len(col), f32), got)
        # borrowed values cannot be replaced through the context
        with pytest.raises(capi.SddmmError) as ei:
            e.update_values(val)
        assert ei.value.code == capi.ERR_STATE
        # a malformed device CSR is rejected by the device-side validation
        bad = col.copy()
        bad[5] = N
        d_bad = hip.upload(bad)
        assert L.sddmm_set_csr_device(e.h, M, N, len(col), d_rp, d_bad, d_val) == capi.ERR_PATTERN
        # misaligned dense pointers are refused
        assert L.sddmm_set_dense_device(e.h, M - 1, N, K, C.c_void_p(dA.value + 4), dB, capi.F32) == capi.ERR_INVALID
    finally:
        e.close()                   # the context goes first, the borrowed buffers after it
        hip.free_all()


def test_device_resident_coo(engine_factory):
    """Borrowed COO arrays: row-sorted input gets a row pointer (every strategy), shuffled
    input keeps its entry order on FLAT / EXACT; bad indices are found on the device."""
    rng = np.random.default_rng(54)
    M, N, K = 400, 350, 32
    mask = rng.random((M, N)) < 0.08
    r, c = np.nonzero(mask)
    r, c = r.astype(np.int32), c.astype(np.int32)
    v = rng.uniform(-1, 1, len(r)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    rowptr, col, val = O.csr_from_triplets(M, r, c, v)
    ref = O.sddmm_csr(rowptr, col, val, A, B)
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    hip = Hip()
    e = engine_factory()
    try:
        L = e.L
        e.set_dense(A, B)
        d_r, d_c, d_v = hip.upload(r), hip.upload(c), hip.upload(v)
        e.nnz = len(r)
        for strategy in (capi.AUTO, capi.ROW_WAVE, capi.FLAT, capi.MFMA_TILE, capi.EXACT):
            e._chk(L.sddmm_set_coo_device(e.h, M, N, len(r), d_r, d_c, d_v))     # clears P
            e.plan(strategy)
            e.run()
            assert O.check_values(e.values(), ref, mag=mag)[0], capi.STRATEGY_NAMES[strategy]
        with pytest.raises(capi.SddmmError):
            e.update_values(v)                       # borrowed values
        perm = rng.permutation(len(r))
        d_r2, d_c2, d_v2 = hip.upload(r[perm]), hip.upload(c[perm]), hip.upload(v[perm])
        for strategy in (capi.AUTO, capi.FLAT, capi.EXACT):
            e._chk(L.sddmm_set_coo_device(e.h, M, N, len(r), d_r2, d_c2, d_v2))
            e.plan(strategy)
            e.run()
            got = e.values()
            assert e.stats().strategy_used in (capi.FLAT, capi.EXACT)
            assert O.check_values(got, ref[perm], mag=mag[perm])[0]
        with pytest.raises(capi.SddmmError) as ei:
            e.plan(capi.ROW_WAVE)                    # needs row-sorted entries
        assert ei.value.code == capi.ERR_UNSUPPORTED
        bad = r.copy()
        bad[3] = M
        d_bad = hip.upload(bad)
        assert L.sddmm_set_coo_device(e.h, M, N, len(r), d_bad, d_c, d_v) == capi.ERR_PATTERN
        assert L.sddmm_set_coo_device(e.h, M, N, len(r), None, d_c, d_v) == capi.ERR_NULL
    finally:
        e.close()
        hip.free_all()


def test_operand_beyond_4gib_uses_64bit_offsets(engine_factory):
    """B of 4 GiB + a little: rows near the end sit beyond a 32-bit byte offset."""
    K = 32
    N = (1 << 25) + 64                       # N*K*4 bytes = 4 GiB + 8 KiB
    M = 64
    print("allocating %.2f GiB for B" % (N * K * 4 / 2 ** 30), flush=True)
    sys.stdout.flush()
    rng = np.random.default_rng(51)
    B = np.zeros((N, K), f32)
    hot = np.unique(np.concatenate([np.arange(0, 40), np.arange(N - 90, N), rng.integers(0, N, 300),
                                    (1 << 25) + np.arange(-20, 20), (1 << 24) + np.arange(-5, 5)]))
    B[hot] = rng.uniform(-1, 1, (len(hot), K)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    rows_cols = [np.sort(rng.choice(hot, size=int(rng.integers(1, 120)), replace=False)) for _ in range(M)]
    lens = np.array([len(x) for x in rows_cols])
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate(rows_cols).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    ref = O.sddmm_csr(rowptr, col, val, A, B)
    _, mag = O.sddmm_csr_f64(rowptr, col, val, A, B)
    assert np.count_nonzero(ref) > 0.9 * len(ref)
    e = engine_factory()
    e.set_dense(A, B)
    for strategy in (capi.AUTO, capi.FLAT, capi.ROW_WAVE, capi.SHORT_ROWS, capi.LDS_TILED, capi.MFMA_TILE, capi.EXACT):
        e.set_csr(M, N, rowptr, col, val)            # clears P
        e.plan(strategy)
        e.run()
        got = e.values()
        ok, worst, i = O.check_values(got, ref, mag=mag)
        assert ok, (capi.STRATEGY_NAMES[strategy], i, got[i], ref[i])
    e.close()


class _DeviceArray:
    """A device address as something torch.as_tensor can wrap without a copy."""

    def __init__(self, ptr, n, typestr="<f4"):
        self.__cuda_array_interface__ = {"shape": (n,), "typestr": typestr, "data": (ptr, False), "version": 2}


def test_lent_stream_orders_producers_launch_and_consumers(engine_factory):
    """The context enqueues on a stream the caller lends (torch's here): operands
    rewritten on that stream right before sddmm_launch, and P copied on that stream
    right after it, need no host synchronisation in between."""
    import torch

    rng = np.random.default_rng(52)
    M, N, K = 3000, 2500, 64
    lens = rng.integers(0, 120, M)
    rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    col = np.concatenate([np.sort(rng.choice(N, size=int(l), replace=False)) for l in lens]).astype(np.int32)
    val = rng.uniform(-1, 1, len(col)).astype(f32)
    A = rng.uniform(-1, 1, (M, K)).astype(f32)
    B = rng.uniform(-1, 1, (N, K)).astype(f32)
    dev = torch.device("cuda:0")
    tA, tB = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
    t_rp, t_col, t_val = torch.from_numpy(rowptr).to(dev), torch.from_numpy(col).to(dev), torch.from_numpy(val).to(dev)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream(device=dev)
    e = engine_factory()
    own = e.get_stream()
    assert own != 0
    e.set_stream(stream.cuda_stream)
    assert e.get_stream() == stream.cuda_stream
    L = e.L
    e._chk(L.sddmm_set_dense_device(e.h, M, N, K, C.c_void_p(tA.data_ptr()), C.c_void_p(tB.data_ptr()), capi.F32))
    e._chk(L.sddmm_set_csr_device(e.h, M, N, len(col), C.c_void_p(t_rp.data_ptr()), C.c_void_p(t_col.data_ptr()),
                                  C.c_void_p(t_val.data_ptr())))
    e.nnz = len(col)
    e.plan(capi.AUTO)
    dP = C.c_void_p()
    e._chk(L.sddmm_get_values_device(e.h, C.byref(dP)))
    tP = torch.as_tensor(_DeviceArray(dP.value, len(col)), device=dev)
    outs = []
    with torch.cuda.stream(stream):
        for step in range(3):
            # producers: a chain of updates of the borrowed operands on the lent stream
            for _ in range(20):
                tA.mul_(1.01)
                tB.add_(0.001)
            e.launch()                        # no host synchronisation on either side
            outs.append((tA.clone(), tB.clone(), tP.clone()))
    stream.synchronize()
    for a, b, p in outs:
        a, b, p = a.cpu().numpy(), b.cpu().numpy(), p.cpu().numpy()
        ref = O.sddmm_csr(rowptr, col, val, a, b)
        _, mag = O.sddmm_csr_f64(rowptr, col, val, a, b)
        ok, worst, i = O.check_values(p, ref, mag=mag)
        assert ok, (i, p[i], ref[i], worst)
    assert not np.array_equal(outs[0][2].cpu().numpy(), outs[2][2].cpu().numpy())
    # the null stream, then back to the context's own stream
    for lend, handle in ((True, 0), (False, 0)):
        e.set_stream(handle, lent=lend)
        assert e.get_stream() == (0 if lend else own)
        e.run()
        np.testing.assert_array_equal(e.values(), outs[2][2].cpu().numpy())
    e.close()


def test_launch_is_capturable_into_a_hip_graph(engine_factory):
    """sddmm_launch on a lent stream only enqueues kernels (no allocation, copy, fill
    or wait), so a planned launch can be recorded into a HIP graph.  Every replay is
    checked against an eager run of the same operands, with eager work and host
    synchronisations between the replays."""
    import torch

    rng = np.random.default_rng(53)
    dev = torch.device("cuda:0")
    for name, K in (("mixed_density", 32), ("fem_banded", 32), ("small_uniform", 32)):
        w = W.make(name, "small", K=K)
        tA, tB = torch.from_numpy(w.A).to(dev), torch.from_numpy(w.B).to(dev)
        t_rp, t_col, t_val = (torch.from_numpy(x).to(dev) for x in (w.rowptr, w.col, w.sval))
        e = engine_factory()
        L = e.L
        stream = torch.cuda.Stream(device=dev)
        e.set_stream(stream.cuda_stream)
        e._chk(L.sddmm_set_dense_device(e.h, w.M, w.N, K, C.c_void_p(tA.data_ptr()), C.c_void_p(tB.data_ptr()), capi.F32))
        e._chk(L.sddmm_set_csr_device(e.h, w.M, w.N, len(w.col), C.c_void_p(t_rp.data_ptr()),
                                      C.c_void_p(t_col.data_ptr()), C.c_void_p(t_val.data_ptr())))
        e.nnz = len(w.col)
        e.plan(capi.AUTO)
        e.run()                                            # warm: nothing is left to set up at capture time
        dP = C.c_void_p()
        e._chk(L.sddmm_get_values_device(e.h, C.byref(dP)))
        tP = torch.as_tensor(_DeviceArray(dP.value, len(w.col)), device=dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            e.launch()
        print(name, "captured, kernels per launch:", e.stats().kernels_launched, flush=True)
        for rep in range(4):
            # eager work between the replays: new operand values, P cleared
            tA.copy_(torch.from_numpy(rng.uniform(-1, 1, w.A.shape).astype(f32)))
            tP.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            replayed = tP.cpu().numpy().copy()
            tP.zero_()
            e.run()
            np.testing.assert_array_equal(replayed, e.values(), err_msg="%s replay %d" % (name, rep))
            a = tA.cpu().numpy()
            ref = O.sddmm_csr(w.rowptr, w.col, w.sval, a, w.B)
            _, mag = O.sddmm_csr_f64(w.rowptr, w.col, w.sval, a, w.B)
            assert O.check_values(replayed, ref, mag=mag)[0], (name, rep)
        del graph
        e.close()
