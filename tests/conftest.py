import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def oracle():
    import oracle as o
    return o


@pytest.fixture(scope="session")
def torch_gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible (there is no CPU fallback)")
    return torch


@pytest.fixture(scope="session")
def handle(torch_gpu):
    import cudaintro_amd
    h = cudaintro_amd.Handle()
    yield h
    torch_gpu.cuda.synchronize()
    h.close()


@pytest.fixture
def rng():
    return np.random.Generator(np.random.PCG64(12345))
