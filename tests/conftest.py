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
    """The loaded C-ABI library; GPU tests fail (not skip) if it is missing."""
    import torch
    assert torch.cuda.is_available(), "gpu-marked test started without a GPU"
    from s2cnn_amd import _hip
    return _hip.lib()
