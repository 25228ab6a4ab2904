import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    return torch.device("cuda:0")


@pytest.fixture(scope="session", autouse=True)
def _require_library_on_gpu():
    """On a GPU box the HIP library must be the thing that runs: fail loudly if it is missing."""
    import torch

    if torch.cuda.is_available():
        from tilegym_amd import _lib

        _lib.load()
    yield
