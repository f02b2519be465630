import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # the test models are small: left to itself a schedule would run their stages on one stream (the host cost
    # of two exceeds their kernels), and the two-stream path — events between stages, the running merge —
    # would go untested.  A test of the automatic choice clears this.
    os.environ.setdefault("PIPPY_AMD_CONCURRENT_STAGES", "1")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
