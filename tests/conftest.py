import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def po():
    """The CPU oracle binding (built on demand with make)."""
    from oracle import pyoracle
    pyoracle.load()
    return pyoracle


@pytest.fixture(scope="session")
def gpu_ready():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no HIP device")
    from diffgemma_amd import capi
    capi.load()  # raises if the HIP library was not built: never fall back
    return True
