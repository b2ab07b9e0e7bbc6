import os
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

# Hyper-parameters every benchmark configuration uses (decay, threshold, surrogate scale, window).
ALPHA, THRESH, BETA, INTERVAL = 0.25, 0.5, 1.0, 0.5


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, when no GPU is visible and `-m gpu` was not requested."""
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:  # pragma: no cover
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no ROCm GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def hyper():
    return dict(alpha=ALPHA, thresh=THRESH, beta=BETA, interval=INTERVAL)
