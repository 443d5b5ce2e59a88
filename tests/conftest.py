import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(GOLDEN_DIR, "reference_vectors.json")) as f:
        return json.load(f)


def load_scv(name):
    """The reference's comma separated test resources (src/test/resources/*.scv)."""
    return np.loadtxt(os.path.join(GOLDEN_DIR, name), delimiter=",", dtype=np.float32)


@pytest.fixture(scope="session")
def linear_function():
    d = load_scv("linear_function_1.scv")
    return d[:, :1].copy(), d[:, 1:2].copy()


@pytest.fixture(scope="session")
def logistic_data():
    d = load_scv("logistic_regression_1.scv")
    # test/Datasets.scala:42-56 scales both features by 1/100
    return (d[:, :2] / np.float32(100)).astype(np.float32), d[:, 2:3].copy()
