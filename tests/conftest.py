"""pytest configuration: repo root on sys.path, the ``gpu`` marker, shared helpers."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def max_rel(x, ref):
    """max|x - ref| / max|ref| -- the parity metric of the benchmark contract."""
    import numpy as np

    x = np.asarray(x, np.float64)
    ref = np.asarray(ref, np.float64)
    denom = max(float(np.abs(ref).max()), 1e-30)
    return float(np.abs(x - ref).max()) / denom


@pytest.fixture
def rel():
    return max_rel
