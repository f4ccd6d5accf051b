"""MI355X-native SDDMM engine: P = S o (A B^T) over the stored entries of S.

The product is the HIP library `dphpc_amd/lib/libsddmm_amd.so` (C ABI in
include/sddmm_amd.h) and the C++ competitor adapter under dphpc_amd/host/.  The
Python in this package is a thin ctypes binding for tests and benchmarks plus the
seeded synthetic workloads; it contains no compute path of its own.
"""
from .capi import (  # noqa: F401
    Engine, SddmmError, Stats, library_path, load_library,
    AUTO, FLAT, ROW_WAVE, SHORT_ROWS, LDS_TILED, MFMA_TILE, EXACT, F32, BF16,
    STRATEGY_NAMES, partition_rows,
)
