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
