import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "ml-cross-entropy_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_sessionstart(session):
    """The tests load the library that is built in the tree; a tree without one gets it built first."""
    import __graft_entry__

    __graft_entry__.ensure_built()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real AMD GPU (run with -m gpu on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
