import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) GPU")


@pytest.fixture(scope="session")
def gpu():
    """Initialise the engine on device 0; GPU tests fail loudly if it cannot."""
    import torch

    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    from nabla_amd import _lib

    _lib.init()
    return torch.device("cuda:0")
