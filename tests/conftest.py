import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _gpu_present():
    # /dev/kfd is the ROCm compute device node; nothing GPU-side is initialised here
    return os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK)


@pytest.fixture(scope="session")
def engine_factory():
    """Creates engines through the C ABI; fails loudly when the HIP library or the
    GPU is missing (there is no CPU stand-in for the product path)."""
    from dphpc_amd import capi

    assert os.path.exists(capi.library_path()), "HIP library not built: run __graft_entry__.build()"
    made = []

    def make(device=0):
        e = capi.Engine(device)
        made.append(e)
        return e

    yield make
    for e in made:
        e.close()
