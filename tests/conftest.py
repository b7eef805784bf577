import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def fta_lib():
    """The built C-ABI library. Built here on first use if absent (hipcc cross-compiles)."""
    from flash_tree_attn_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from flash_tree_attn_amd.build import build
        build(verbose=False)
    return _lib.load()
