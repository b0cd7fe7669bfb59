import ctypes
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real AMD GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def lib():
    """The ctypes view of the built C-ABI libraries; fails (not skips) when they are not built."""
    from infinicore_amd import libinfiniop

    return libinfiniop


@pytest.fixture(scope="session")
def oracle():
    from oracle import paged_oracle

    paged_oracle.load()
    return paged_oracle


@pytest.fixture()
def host_amd_handle(lib):
    """An AMD handle that needs no GPU: the ABI-visible handle is exactly {int device; int device_id},
    which is all descriptor creation (pure host code) reads. Lets validation run on a CPU-only host."""
    handle = lib.Handle(lib.InfiniDevice.AMD, 0)
    return ctypes.pointer(handle)


@pytest.fixture(scope="session")
def gpu_handle(lib):
    """A real handle on GPU 0, created the way callers do: infinirtSetDevice + infiniopCreateHandle."""
    lib.set_device(lib.InfiniDevice.AMD, 0)
    handle = lib.create_handle()
    yield handle
    lib.destroy_handle(handle)
