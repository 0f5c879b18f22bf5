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


class _TuningEnv:
    """monkeypatch whose environment changes reach the library: the GEMM path reads
    its CUMPSGEMM_* tuning variables once per process, so after every change the
    library is told to read them again."""

    def __init__(self, mp):
        self._mp = mp

    def _reload(self):
        import cumpsgemm_amd
        cumpsgemm_amd.lib().cuMpSGEMM_reload_tuning_env()

    def setenv(self, name, value, prepend=None):
        self._mp.setenv(name, value, prepend)
        self._reload()

    def delenv(self, name, raising=True):
        self._mp.delenv(name, raising)
        self._reload()

    def undo(self):
        self._mp.undo()
        self._reload()

    def __getattr__(self, name):
        return getattr(self._mp, name)


@pytest.fixture
def monkeypatch(monkeypatch):
    mp = _TuningEnv(monkeypatch)
    yield mp
    mp.undo()


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
