import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _inference_mode_by_default():
    """The path under test is forward-only, like the reference's (utils.py:6-8 runs it under
    torch.no_grad()): tests run with gradients disabled, so that KSLinear(algo='kernel') takes the
    chain launcher.  The backward tests switch gradients on themselves (torch.enable_grad())."""
    import torch

    prev = torch.is_grad_enabled()
    torch.set_grad_enabled(False)
    yield
    torch.set_grad_enabled(prev)


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library, loaded once."""
    from ksmm_amd import _lib

    return _lib.load()
