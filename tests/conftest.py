import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_w3j():
    return dict(np.load(os.path.join(GOLDEN, "w3j.npz")))


@pytest.fixture(scope="session")
def golden_sh():
    return dict(np.load(os.path.join(GOLDEN, "sh.npz")))


@pytest.fixture(scope="session")
def golden_tp():
    with open(os.path.join(GOLDEN, "tp_cases.json")) as f:
        meta = json.load(f)
    arrays = dict(np.load(os.path.join(GOLDEN, "tp_cases.npz")))
    return meta, arrays
