import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o

    o.lib()
    return o


@pytest.fixture(scope="session")
def rnb():
    """The shipped package bound to librnb_hip.so; GPU tests skip cleanly when no device opens,
    mirroring the reference's device tests (crates/rnb-backend/cuda/src/runtime/tests.rs:22831-22834)."""
    import runnburn_amd as pkg

    if not pkg.device_available():
        pytest.skip(f"no HIP device: {pkg.last_error()}")
    return pkg
