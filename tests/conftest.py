import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "general-nvgpu-testing_amd"), os.path.join(ROOT, "oracle"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) GPU")


@pytest.fixture(scope="session")
def oracle():
    import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def beamc():
    """The ctypes binding of libbeam_hip.so (no GPU call is made by importing it)."""
    from beam import _C
    return _C


@pytest.fixture(scope="session")
def gpu(beamc):
    """Fails (not skips) when the device or the HIP library is unusable: GPU tests must never
    pass on a fallback."""
    info = beamc.device_info()
    assert "gfx950" in info["name"], info
    return info
