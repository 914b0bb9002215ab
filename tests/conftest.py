import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def centerpoint_input():
    d = np.load(os.path.join(GOLDEN, "centerpoint_input.npz"))
    return d["features"], d["indices_zyx"]


@pytest.fixture(scope="session")
def bevfusion_input():
    d = np.load(os.path.join(GOLDEN, "bevfusion_input.npz"))
    return d["features"], d["indices_xyz"]


@pytest.fixture(scope="session")
def nuscenes_frame():
    return np.load(os.path.join(GOLDEN, "nuscenes_frame.npz"))["points"]
