import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu")
    config.addinivalue_line("markers", "slow: long CPU sweep, enabled with SKL_EXHAUSTIVE=1")


@pytest.fixture(scope="session")
def gpu():
    """The GPU library, initialised on device 0. GPU tests fail (not skip) when
    the library or the device is missing: there is no CPU fallback to hide behind."""
    import skl_amd
    lib = skl_amd.load()
    rc = lib.skl_hip_init(0)
    assert rc == 0, f"skl_hip_init(0) failed: {lib.skl_hip_last_error_string().decode()}"
    yield lib
    lib.skl_hip_synchronize()
