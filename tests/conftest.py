import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


@pytest.hookimpl(tryfirst=True)
def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # pytest.ini asks for worker processes (-n 4). They are for the CPU suite only: unless the selection excludes the
    # GPU tests outright (-m "not gpu"), run everything in this one process. (pytest-xdist starts its workers from its
    # own pytest_configure, which runs after this one, and only if these two options say so.)
    if "not gpu" not in (getattr(config.option, "markexpr", "") or "") and hasattr(config.option, "tx"):
        config.option.dist = "no"
        config.option.tx = []
        config.option.numprocesses = 0


@pytest.fixture(scope="session")
def fta_lib():
    """The built C-ABI library. Built here on first use if absent (hipcc cross-compiles)."""
    import fcntl
    from flash_tree_attn_amd import _lib
    with open(_lib.LIB_PATH + ".lock", "w") as lock:      # worker processes of one run must not build into the same file at once
        fcntl.flock(lock, fcntl.LOCK_EX)
        if not os.path.exists(_lib.LIB_PATH):
            from flash_tree_attn_amd.build import build
            build(verbose=False)
    return _lib.load()
