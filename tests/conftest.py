import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
TESTS = os.path.dirname(os.path.abspath(__file__))
if TESTS not in sys.path:
    sys.path.insert(0, TESTS)               # reference_space

# Tests never start a tuning run implicitly: a cache miss falls back to the default configuration.
os.environ.setdefault("AAT_TUNE_ON_MISS", "0")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        # on a GPU box every library the suite loads was built ahead of time: a missing one is an error,
        # never a multi-minute hipcc run inside a test
        os.environ.setdefault("AAT_NO_JIT", "1")
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
