import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """Load what is built; compile the HIP library (hipcc cross-compiles without a GPU) only if none is there."""
    from etha_amd.build import ensure_built

    ensure_built()


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from etha_amd import _native

    _native.lib()  # fails loudly when the HIP library is not built
    return torch.device("cuda:0")
