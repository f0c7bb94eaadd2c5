import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with `-m gpu` on the GPU box)")


@pytest.fixture(scope="session")
def hip_device():
    """The one GPU of the box; GPU tests fail (they do not skip) when the library cannot see it."""
    from kyanite_amd import HipDevice

    assert HipDevice.count() >= 1, "no HIP device visible: GPU tests need the MI355X"
    return HipDevice(0)
