import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def golden():
    """name -> npz file of tests/golden (numpy.load without pickle)."""
    import numpy as np

    class _Golden(dict):
        def __missing__(self, name):
            self[name] = np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
            return self[name]

    return _Golden()


@pytest.fixture(scope="session")
def ops():
    """The product's operator layer on cuda:0, initialised once.  Fails (not skips) if the GPU path is unusable."""
    import torch
    import pimaicompiler_amd as P

    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    P.initialize(0)
    yield P
    torch.cuda.synchronize()
