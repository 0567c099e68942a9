import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """The harness bound to cuda:0; fails (not skips) when the HIP library is missing."""
    import torch
    assert torch.cuda.is_available(), "a test marked gpu ran without a GPU"
    from tests import harness
    harness.check_library_loaded()
    return harness
