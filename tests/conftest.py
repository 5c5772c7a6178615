import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


def rel_err(y, y_ref):
    """Element-wise error of a GPU result against the fp64 oracle, relative to
    max(|y*|, 2^-10 * max|y*|): outputs of a zero-mean dot product cross zero,
    so a pure element-wise relative error is unbounded there; the floor is one
    fp16 ulp of the largest output."""
    y = np.asarray(y, np.float64)
    y_ref = np.asarray(y_ref, np.float64)
    floor = np.max(np.abs(y_ref)) * 2.0 ** -10 if y_ref.size else 0.0
    den = np.maximum(np.abs(y_ref), max(floor, 1e-30))
    return np.abs(y - y_ref) / den
