import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library, loaded from the in-tree build (built by __graft_entry__.build())."""
    from intra_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from intra_amd.build import build
        build()
    return _lib.load()
