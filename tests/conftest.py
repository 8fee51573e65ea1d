import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device; run with -m gpu on the GPU box")


@pytest.fixture(scope="session")
def kvx():
    """The loaded C-ABI library. GPU tests must never run on a fallback: a missing library or
    device is an error, not a skip."""
    from keys_values_amd import _lib

    lib = _lib.load()
    return lib


@pytest.fixture(scope="session")
def gpu(kvx):
    import torch

    assert torch.cuda.is_available(), "GPU tests need a ROCm device"
    assert kvx.kvx_device_count() > 0, "libkvx sees no gfx950 device"
    return torch.device("cuda", 0)
