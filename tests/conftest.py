import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle_lib():
    import oracle
    oracle.lib()
    return oracle


@pytest.fixture
def tracea_gpu():
    """Initialised library on cuda:0; fails loudly if the HIP library is absent.
    (tracea_init is idempotent; calling it per test survives a tracea_shutdown elsewhere.)"""
    import torch
    from tracea_amd import capi, ops
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    capi.init()
    return ops
