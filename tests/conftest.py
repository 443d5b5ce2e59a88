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


def load_sunspots():
    """`monthlySunspots(12)` of the reference's tests (test/Datasets.scala:72-97) from its own resource file: counts scaled
    to [0, 1] by the series' minimum and maximum, grouped by floor((year*12 + month) / 12) (so a group runs from
    December to November), a group of 12 is one sample and the first value of the next group its label.
    Returns (X [n, 12, 1], Y [n, 1]) in time order."""
    months, values = [], []
    with open(os.path.join(GOLDEN_DIR, "monthly-sunspots.csv")) as f:
        next(f)
        for line in f:
            line = line.strip()
            if not line:
                continue
            date, v = line.split(",")
            y, m = date.strip('"').split("-")
            months.append(int(y) * 12 + int(m))
            values.append(float(v))
    v = np.asarray(values, np.float32)
    lo, hi = v.min(), v.max()
    scaled = ((v - lo) / (hi - lo)).astype(np.float32)
    groups = {}
    for mth, s in zip(months, scaled):
        groups.setdefault(mth // 12, []).append(s)
    xs, ys = [], []
    for step in sorted(groups):
        if len(groups[step]) == 12 and step + 1 in groups:
            xs.append(groups[step])
            ys.append([groups[step + 1][0]])
    return np.asarray(xs, np.float32).reshape(-1, 12, 1), np.asarray(ys, np.float32)


@pytest.fixture(scope="session")
def sunspots():
    return load_sunspots()
