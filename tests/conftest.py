import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def exe():
    """The HIP executor.  GPU tests fail (not skip) when the native library or the
    device is missing: a silent fallback would void every parity claim."""
    from mlcompiler_amd import HipExecutor

    e = HipExecutor.Instance()
    assert e.isAvailable(), "gfx950 device / native library unavailable: " + e.lastError()
    return e
