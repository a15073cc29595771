import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """Session-wide library handle on device 0; fails loudly without the HIP library."""
    from alsparse_amd import capi, hiprt
    if hiprt.device_count() < 1:
        pytest.fail("GPU test collected on a machine without a GPU")
    hiprt.set_device(0)
    h = capi.Handle()
    yield h
    hiprt.synchronize()
    h.close()
