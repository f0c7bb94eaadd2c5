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


def pytest_sessionfinish(session, exitstatus):
    """Write the measured parity errors of every GPU comparison of the session next to the other run outputs, so
    that a regression of a case shows as a number and not only as a pass that became a failure."""
    try:
        from runner import PARITY_RECORDS
    except Exception:
        return
    if not PARITY_RECORDS:
        return
    import json

    out_dir = os.path.join(ROOT, "gpurun_out")
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "parity_report.json"), "w") as f:
        json.dump(PARITY_RECORDS, f, indent=0)
