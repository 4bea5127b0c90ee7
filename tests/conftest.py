import os
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter):
    """How much of its tolerance the engine used at most, per precision (tests/helpers.py:assert_close)."""
    try:
        from helpers import worst_share
    except ImportError:
        return
    for dtype, (share, what) in sorted(worst_share.items()):
        terminalreporter.write_line(f"largest share of the {dtype} tolerance used: {share:.3f} ({what})")
