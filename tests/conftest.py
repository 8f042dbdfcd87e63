import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "dragon-alpha-v1.2_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def dh():
    """The product binding (loads libdragon_hip.so; import fails loudly if it is missing)."""
    import dragon_hip
    return dragon_hip


@pytest.fixture(scope="session")
def gpu(dh):
    """A GPU is mandatory for tests marked gpu: no silent skip, no CPU fallback."""
    n = dh.Cuda.getDeviceCount()
    assert n >= 1, "no HIP device visible: gpu-marked tests must run on the GPU box"
    dh.Cuda.setDevice(0)
    return dh
