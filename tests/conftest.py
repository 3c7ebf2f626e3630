import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ccn():
    """The loaded C-ABI binding, initialised on device 0.  GPU tests only."""
    import torch
    from coconet_amd import capi
    assert torch.cuda.is_available(), "GPU test started without a GPU"
    capi.load()          # raises if the HIP library was not built: no fallback path exists
    capi.init(0)
    return capi
