import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ops-nn_amd"))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def opsnn():
    import opsnn as m
    m.lib()
    return m


@pytest.fixture(scope="session")
def gpu(opsnn):
    if not opsnn.gpu_available():
        pytest.fail("this test is marked gpu but no HIP device is visible")
    opsnn.check(opsnn.lib().aclInit(None), "aclInit")
    opsnn.check(opsnn.lib().aclrtSetDevice(0), "aclrtSetDevice")
    # every workspace the two-phase helpers allocate starts as NaN patterns: reading a part that the call has not written shows
    import opsnn.binding
    opsnn.binding.FILL_NEW_WORKSPACE = 0xFF
    return opsnn


@pytest.fixture(autouse=True)
def _stale_lds(request):
    """Before every GPU test the LDS of all compute units is filled with NaN patterns: a kernel that multiplies LDS it never
    wrote by zero weights would pass on clean LDS and fail only after certain other kernels."""
    if "gpu" in request.fixturenames:
        m = request.getfixturevalue("gpu")
        m.check(m.lib().opsnnDebugFillLds(None), "opsnnDebugFillLds")
    yield
