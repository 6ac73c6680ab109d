import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def km():
    """One kernel manager on cuda:0 for the whole session (GPU tests only)."""
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import einsummable_amd as ea

    torch.cuda.init()
    manager = ea.KernelManager(0)
    yield manager
    torch.cuda.synchronize()
    manager.close()
