import os
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


@pytest.fixture(scope="session")
def golden():
    return np.load(os.path.join(REPO, "tests", "golden", "tk3d_small.npz"))


@pytest.fixture(scope="session")
def cuda():
    """Skip unless a GPU is visible; returns the device string."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return "cuda:0"
