import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real AMD GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    """FGNN_PARITY_LOG=<file>: how much of the derived tolerance every sum-scaled comparison used (tests/util.py)."""
    path = os.environ.get("FGNN_PARITY_LOG")
    if not path:
        return
    import json
    from tests import util
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as fh:
        json.dump(util.PARITY_LOG, fh, indent=1)
