"""pytest configuration: the `gpu` marker and shared fixtures.

`-m "not gpu"` runs on a machine without a GPU: oracle pinning, host logic, and
the load / symbol checks of the native library.  `-m gpu` are the parity tests
proper; they need one gfx950 device and the in-tree built library, and fail
(not skip) when either is missing.
"""
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs one MI355X (gfx950) device")


@pytest.fixture(scope="session")
def ctx():
    """One C-ABI context on device 0 for the whole session."""
    from autograd_amd import capi

    c = capi.Context(0)
    yield c
    c.synchronize()
    c.close()
