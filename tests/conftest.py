import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu")


def rel_close(got, want, tol, floor=1e-3):
    """Elementwise |got - want| <= tol * max(|want|, floor * rms(want)): a relative error
    with a floor at `floor` of the output's RMS, so that a near-zero element (a sum that
    cancels) is held to the same absolute error as a small one."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    rms = np.sqrt(np.mean(want * want)) if want.size else 0.0
    bound = tol * np.maximum(np.abs(want), floor * rms)
    err = np.abs(got - want)
    worst = float(np.max(err / np.maximum(bound, 1e-300))) if want.size else 0.0
    return worst <= 1.0, worst * tol


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
