import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def hip():
    """The ctypes binding; GPU tests go through the C ABI only."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from ditango_amd import _hip
    _hip.load_library()
    return _hip
