import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ocean-tensor-package_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hip():
    """The ctypes binding of the device library with a warmed-up device 0 and one stream."""
    import ocean_hip as oh
    if oh.device_count() < 1:
        pytest.fail("no HIP device visible: GPU tests must run on the GPU box")
    oh.check(oh.lib.och_device_set(0))
    oh.check(oh.lib.och_device_warmup(0))
    return oh


@pytest.fixture(scope="session")
def stream(hip):
    s = hip.Stream()
    yield s
    s.synchronize()
