import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import blkq4_oracle
    blkq4_oracle.lib()  # builds the C oracle on first use if it is not there
    return blkq4_oracle


@pytest.fixture(scope="session")
def capi():
    from gemmlib_amd import capi as _capi
    _capi.load()  # raises if the library is not built: there is no fallback
    return _capi


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    return torch.device("cuda:0")
