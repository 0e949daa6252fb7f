import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box only)")


@pytest.fixture(scope="session")
def ref():
    """The CPU oracle (ctypes binding), built on demand with gcc."""
    from oracle import ref as _ref
    _ref.build()
    _ref.lib()
    return _ref


def announce(*parts):
    """Name the case on the real stderr (unbuffered, not captured) before a GPU step, so a run that
    dies inside the GPU call still shows which case it was."""
    sys.__stderr__.write("[case] " + " ".join(str(p) for p in parts) + "\n")
    sys.__stderr__.flush()


@pytest.fixture(scope="session")
def capi():
    """The HIP library through its C ABI.  Raises (never skips) if it is not built."""
    from onellm_amd import capi as _capi
    _capi.lib()
    return _capi


@pytest.fixture(scope="session")
def dev():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")
