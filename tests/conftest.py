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


@pytest.fixture(scope="session")
def parity_stats():
    """Observed error figures of the configuration tests (errors in units of the bound each
    test gates on, bit-exactness verdicts).  Written as JSON next to the other outputs of a GPU
    run when the session ends, so that a run leaves the measured numbers behind and not only
    pass/fail."""
    import json
    stats = {}
    yield stats
    if not stats:
        return
    out_dir = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "parity_stats.json"), "w") as f:
            json.dump(stats, f, indent=1, sort_keys=True)
    except OSError:
        pass
