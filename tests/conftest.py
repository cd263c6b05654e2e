import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _ensure_built():
    import __graft_entry__ as g
    g.ensure_built()


_ensure_built()


@pytest.fixture(scope="session")
def gpu_thread():
    """One library-owned thread (HIP stream) shared by the GPU tests."""
    import torch
    import hcomm_amd as h
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    torch.cuda.init()
    code, handles = h.HcommThreadAlloc(h.CommEngine.CPU_TS, 1, 2)
    assert code == 0
    yield handles[0]
    h.HcommGfxThreadSynchronize(handles[0])
    h.HcommThreadFree(handles)
