import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


# The suite runs the host with whole-forward graph replay switched on (the library's default is the eager layer loop):
# the replay is the path with more machinery - recording, signatures, invalidation - and the tests that compare it with
# the eager loop set the switch themselves either way.
os.environ.setdefault("TNN_ROCM_GRAPH", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    # GPU tests print which case is running before touching the device (a faulting box returns
    # only the tail of stdout), so make sure every gpu test is also skipped cleanly without a GPU.
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
