"""pytest configuration: markers and import path."""

import os
import sys

import pytest

# The operator tests check results, not speed: use each kernel family's first (heuristically
# best) configuration instead of running the on-device sweep for every shape.  The sweep itself
# is covered by tests/test_tuner_gpu.py.
os.environ.setdefault("SPIO_TUNE", "0")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: large sampled sweeps")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, when no GPU is visible."""
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)
