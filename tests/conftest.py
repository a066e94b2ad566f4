import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_mod():
    import oracle

    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def host_handle():
    """A device-less handle: descriptors, workspace queries and planning, no execution."""
    from hiptensor_amd import api

    h = api.check(api.hiptensorCreateHostOnly(), "hiptensorCreateHostOnly")
    yield h
    api.hiptensorDestroy(h)


@pytest.fixture(scope="session")
def gpu_handle():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a device"
    from hiptensor_amd import api

    torch.cuda.init()
    torch.zeros(1, device="cuda")
    h = api.check(api.hiptensorCreate(), "hiptensorCreate")
    yield h
    api.hiptensorDestroy(h)
