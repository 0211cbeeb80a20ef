import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def rel_err(y: np.ndarray, truth: np.ndarray) -> float:
    """max |y - t| / max(|t|, 1e-3 * rms(t)): relative error with a floor, so
    outputs that cancel to ~0 are judged against the scale of the vector."""
    y = np.asarray(y, np.float64).reshape(-1)
    t = np.asarray(truth, np.float64).reshape(-1)
    floor = 1e-3 * float(np.sqrt(np.mean(t * t))) + 1e-300
    return float(np.max(np.abs(y - t) / np.maximum(np.abs(t), floor)))


@pytest.fixture(scope="session")
def oracle():
    from oracle import cpu_oracle

    cpu_oracle.build()
    return cpu_oracle
