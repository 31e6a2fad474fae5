import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def hip_backend():
    """The HIP kernel library on a real device. GPU tests fail (not skip) when it cannot be used."""
    from skainet_amd import kernels
    from skainet_amd import _lib
    assert os.path.exists(_lib.HIP_LIB_PATH), "libskainet_hip.so is not built (python -m skainet_amd.build)"
    assert kernels.is_available(), "HIP backend unavailable: " + _lib.last_error()
    return kernels


@pytest.fixture(scope="session")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "no GPU visible to torch"
    return torch
