import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def error_figures(got, want, rel_floor=0.1):
    """Plain error figures of a result against its reference: the largest absolute error, and the
    largest relative error over the elements whose reference is at least `rel_floor` in size."""
    import torch
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    big = want.abs() >= rel_floor
    rel = float((err[big] / want.abs()[big]).max()) if bool(big.any()) else 0.0
    return {"max_abs": float(err.max()), "max_rel": rel, "max_ref": float(want.abs().max())}


def report(name, **figures):
    """Appends one line of measured figures to the file named by HSA_TEST_REPORT (if set): the
    source of the error figures quoted beside the tolerances."""
    path = os.environ.get("HSA_TEST_REPORT")
    if path:
        import json
        with open(path, "a") as f:
            f.write(json.dumps({"test": name, **figures}) + "\n")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def bf():
    import oracle
    return oracle.BruteForce()
