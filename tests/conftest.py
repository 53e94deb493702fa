import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def _gpu_present() -> bool:
    return os.path.exists("/dev/kfd")


@pytest.fixture(scope="session")
def pair_factory():
    """GPU tests: yields a constructor of harness.Pair; fails loudly when the
    HIP library is missing or no device is visible."""
    import ctypes as C

    from cortex_amd import capi

    n = C.c_int(0)
    capi.call("ct_device_count", C.byref(n))
    assert n.value >= 1, "no HIP device visible"
    capi.call("ct_set_device", 0)
    capi.call("ct_set_debug_sync", 1)
    import harness

    return harness.Pair
