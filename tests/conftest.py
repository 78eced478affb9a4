import os
import sys

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO not in sys.path:
    sys.path.insert(0, REPO)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz")
    return np.load(path, allow_pickle=False)


def golden_cases():
    path = os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz")
    with np.load(path, allow_pickle=False) as z:
        return [str(c) for c in z["cases"]]
