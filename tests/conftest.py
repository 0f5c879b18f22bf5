import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def O():
    """The CPU oracle (test infrastructure)."""
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def cg():
    import cumpsgemm_amd
    cumpsgemm_amd.lib()
    return cumpsgemm_amd


@pytest.fixture(scope="session")
def torch_gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    return torch


@pytest.fixture(scope="session")
def handle(cg, torch_gpu):
    h = cg.Handle()
    h.set_stream(torch_gpu.cuda.current_stream())
    yield h
    torch_gpu.cuda.synchronize()
    h.close()


class Dev:
    """Upload / download helpers around torch device memory."""

    def __init__(self, torch):
        self.torch = torch
        self.dev = torch.device("cuda:0")

    def up(self, arr):
        flat = np.ascontiguousarray(arr).reshape(-1)
        if flat.dtype == np.complex64:
            flat = flat.view(np.float32)
        return self.torch.from_numpy(flat.copy()).to(self.dev)

    def down(self, t, dtype=np.float32):
        self.torch.cuda.synchronize()
        a = t.cpu().numpy()
        return a.view(np.complex64) if dtype == np.complex64 else a


@pytest.fixture(scope="session")
def dev(torch_gpu):
    return Dev(torch_gpu)
