import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load what is built; only when a library is missing altogether (a fresh
    checkout) is it compiled here - hipcc cross-compiles for gfx950 without a GPU."""
    from hipress_amd import build as hb
    from hipress_amd.compll import build as cb

    if not os.path.exists(hb.LIB):
        hb.build()
    if not os.path.exists(cb.LIB):
        cb.build()


def _have_gpu():
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
