import os
import sys

import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a GPU (run on the MI355X box)")
    config.addinivalue_line("markers", "slow: takes a minute or more (deselect with -m 'gpu and not slow')")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
