import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def hiplib():
    """The built C-ABI library, device checked.  GPU tests fail (not skip) if it is missing."""
    import torch
    from bamboo_amd import hip
    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    hip.init()
    return hip
