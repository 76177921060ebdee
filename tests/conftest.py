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


def pytest_sessionstart(session):
    # a checkout that has never been built: compile the library once (kernels are then specialised on first use)
    from e3nn_amd.csrc.build import ensure_built

    ensure_built()


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


def pytest_terminal_summary(terminalreporter):
    """Raw error figures of every comparison against the oracle made in this session (max abs, max relative),
    beside the pass / fail of the tolerance checks; also written as parity_errors.json into the directory named by
    E3X_PARITY_ERRORS_DIR, when that is set and exists."""
    from tests.helpers import ERROR_LOG

    if not ERROR_LOG:
        return
    tr = terminalreporter
    tr.section("raw errors against the oracle")
    tr.write_line(f"{'comparison':60s} {'n':>9s} {'max|err|':>10s} {'max|ref|':>10s} {'max rel':>10s} {'err/tol':>8s}")
    for r in ERROR_LOG:
        tr.write_line(f"{r['what'][:60]:60s} {r['n']:9d} {r['max_abs_err']:10.3e} {r['max_abs_ref']:10.3e} "
                      f"{r['max_rel_err']:10.3e} {r['worst_err_over_tol']:8.3f}")  # fmt: skip
    out_dir = os.environ.get("E3X_PARITY_ERRORS_DIR")
    if out_dir and os.path.isdir(out_dir):
        with open(os.path.join(out_dir, "parity_errors.json"), "w") as f:
            json.dump(ERROR_LOG, f, indent=1)
