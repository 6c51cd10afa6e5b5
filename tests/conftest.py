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


@pytest.fixture(scope="session")
def al():
    """The C-ABI library through its ctypes binding; GPU tests only."""
    import torch
    import aluminum_amd
    aluminum_amd.load()
    if not torch.cuda.is_available():
        pytest.fail("GPU test started without a GPU")
    rc = aluminum_amd.load().alamd_init()
    assert rc == 0, aluminum_amd.load().alamd_last_error()
    return aluminum_amd
