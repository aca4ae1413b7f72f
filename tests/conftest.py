import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: long CPU-only check, not part of the default run")


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    return torch.device("cuda:0")


@pytest.fixture(scope="session")
def tc(dev):
    """The host-side wrapper module with the C-ABI library loaded (no fallback)."""
    from wmma_extension_amd import _lib, tcec
    _lib.lib()
    return tcec
