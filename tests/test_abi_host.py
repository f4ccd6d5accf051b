"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol,
and its host-only entry points and argument checks behave -- no GPU compute."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from dphpc_amd import capi
from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    L = capi.load_library()
    header = open(os.path.join(ROOT, "include", "sddmm_amd.h")).read()
    declared = set(re.findall(r"\b(sddmm_[a-z_]+)\s*\(", header))
    assert declared == set(capi.EXPORTS), declared ^ set(capi.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    assert b"gfx950" in L.sddmm_version()


def test_strerror_covers_all_codes():
    L = capi.load_library()
    seen = set()
    for code in range(0, -9, -1):
        s = L.sddmm_strerror(code)
        assert s and s != b"unknown error"
        seen.add(s)
    assert len(seen) == 9
    assert L.sddmm_strerror(-99) == b"unknown error"


def test_null_and_argument_errors_without_gpu():
    L = capi.load_library()
    assert L.sddmm_create(None, 0) == capi.ERR_NULL
    assert L.sddmm_run(None) == capi.ERR_NULL
    assert L.sddmm_plan(None, 0) == capi.ERR_NULL
    assert L.sddmm_get_values(None, None) == capi.ERR_NULL
    assert L.sddmm_last_stats(None, None) == capi.ERR_NULL
    assert L.sddmm_last_error(None) == b""
    L.sddmm_destroy(None)                              # must be a no-op
    rp = np.array([0, 1], np.int32)
    out = np.zeros(4, np.int32)
    assert L.sddmm_partition_rows(1, None, 1, 1, capi._ptr(out)) == capi.ERR_NULL
    assert L.sddmm_partition_rows(0, capi._ptr(rp), 1, 1, capi._ptr(out)) == capi.ERR_INVALID
    assert L.sddmm_partition_rows(1, capi._ptr(rp), 0, 1, capi._ptr(out)) == capi.ERR_INVALID
    assert L.sddmm_partition_rows(3, capi._ptr(rp), 1, 2, capi._ptr(out)) == capi.ERR_INVALID


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_create_fails_loudly_without_a_device():
    with pytest.raises(capi.SddmmError) as ei:
        capi.Engine()
    assert ei.value.code == capi.ERR_NO_DEVICE


# exact vectors of the reference's dispatcher tests (tests/matrix_test.cc:354-425, 460-477)
def test_partition_rows_kats():
    assert capi.partition_rows([0, 2, 4], 4).tolist() == [0, 1, 2, 2, 2]
    assert capi.partition_rows([0, 2, 4], 2).tolist() == [0, 1, 2]
    assert capi.partition_rows([0, 1, 2, 3, 4], 2).tolist() == [0, 2, 4]
    assert capi.partition_rows([0, 0, 1, 1, 1], 2).tolist() == [0, 4, 4]
    assert capi.partition_rows(np.arange(65), 4, 16).tolist() == [0, 16, 32, 48, 64]
    n = 150000
    np.testing.assert_array_equal(capi.partition_rows(np.arange(n + 1), n // 2), 2 * np.arange(n // 2 + 1))


def test_partition_rows_matches_oracle_on_random_patterns():
    rng = np.random.default_rng(11)
    for trial in range(40):
        M = int(rng.integers(1, 30)) * 16
        lens = rng.integers(0, 50, M)
        if trial % 4 == 0:
            lens[rng.integers(0, M)] = 5000           # one dominant row
        if trial % 5 == 0:
            lens[rng.random(M) < 0.7] = 0             # many empty rows
        if lens.sum() == 0:
            lens[0] = 1
        rowptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        for parts, stride in [(1, 1), (2, 1), (5, 1), (M, 1), (3 * M, 1), (3, 16), (64, 16)]:
            np.testing.assert_array_equal(capi.partition_rows(rowptr, parts, stride),
                                          O.dispatch(rowptr, parts, stride))
            got = capi.partition_rows(rowptr, parts, stride)
            assert got[0] == 0 and got[-1] == M and np.all(np.diff(got) >= 0)


def test_bf16_round_trip_helpers():
    x = np.array([1.0, -1.0, 0.5, 1.00390625, 1.01171875, 3.14159], np.float32)
    b = capi.to_bf16(x)
    y = capi.from_bf16(b)
    assert y[0] == 1.0 and y[1] == -1.0 and y[2] == 0.5
    assert y[3] == 1.0                                 # 1 + 2^-8: tie, rounds to even (1.0)
    assert y[4] == np.float32(1.015625)                # 1 + 3*2^-8: tie, rounds to even (1 + 2^-6)
    assert abs(y[5] - 3.14159) < 2 ** -7 * 3.14159
