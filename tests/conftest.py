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


# How the logits become weights: inside the split kernel once the row's other splits have arrived
# (the default), through the scratch buffer and the weights kernel (resident form switched off), and
# the bounded wait running out in every workgroup (limit 0) or in most of them (limit 1).
# (resident, spin_limit, poll_sleep) for kvx_decode_tuning; -1 = the default
DECODE_ROUTES = {"resident": (-1, -1, -1), "scratch": (0, -1, -1), "no-wait": (-1, 0, -1), "one-poll": (-1, 1, -1)}


@pytest.fixture(params=list(DECODE_ROUTES))
def decode_route(request, kvx):
    kvx.kvx_decode_tuning(*DECODE_ROUTES[request.param])
    yield request.param
    kvx.kvx_decode_tuning(-1, -1, -1)
