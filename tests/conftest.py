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


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    """The counts the parity tests keep -- elements that needed the tolerance clause of the
    parameter comparison, oracle steps that had to follow the device's norm -- belong in the
    log of every run, captured output or not."""
    try:
        from tests import helpers as H
    except Exception:
        return
    if not H.REPORT_LINES and not H.NORM_FOLLOWED["steps"]:
        return
    tr = terminalreporter
    tr.section("parity: tolerance clause and norm differences")
    for line in H.REPORT_LINES:
        tr.write_line(line)
    tr.write_line(f"[norm-follow] {H.NORM_FOLLOWED['events']} of {H.NORM_FOLLOWED['steps']} clipped-capable oracle "
                  "steps had to be repeated with the device's norm")
