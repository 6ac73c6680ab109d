import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _torch_owns_the_device_first(request):
    """torch supplies device memory and streams to the GPU tests, and it has to set the device up
    before the library makes its first HIP call: a test that builds a kernel manager of its own
    must work when it is the first one of the process."""
    if request.node.get_closest_marker("gpu") is not None:
        import torch

        torch.cuda.init()


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
