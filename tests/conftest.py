import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """A fresh checkout has no built library (built files are not in the history): compile it once, here on the host,
    before the tests that load it.  Where the library is already there (every GPU run: it travels with the tree)
    nothing happens."""
    from patrickstar_amd import _lib, build

    if os.path.exists(_lib.LIB_PATH):
        return
    try:
        build.hipcc_path()
    except RuntimeError:
        return  # no compiler: the tests that need the library say so themselves
    build.build()


def _gpu_present():
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
