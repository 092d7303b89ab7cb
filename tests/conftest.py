import os
import sys

import pytest

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_sessionfinish(session, exitstatus):
    """With ARLE_TEST_STATS=<file>: the worst maximum and rms errors that the comparisons with the plain
    implementation saw, one line a comparison (what the tolerances are set against)."""
    path = os.environ.get("ARLE_TEST_STATS")
    if not path:
        return
    try:
        import replay
    except ImportError:
        return
    with open(path, "w") as fh:
        for what, (worst, rms, spread) in sorted(replay.last_stats.items()):
            fh.write(f"{worst:.3e} {rms:.3e} {spread:5.2f} {what}\n")
