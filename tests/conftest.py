import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def rel_l2(a, b):
    """relative L2 error of a against the reference b"""
    import numpy as np
    a = np.asarray(a, dtype=np.complex128).ravel()
    b = np.asarray(b, dtype=np.complex128).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def max_rel(a, b):
    """max element error relative to the largest reference magnitude (the reference's outputs
    have zeros by construction, so a per-element ratio is undefined there)"""
    import numpy as np
    a = np.asarray(a, dtype=np.complex128).ravel()
    b = np.asarray(b, dtype=np.complex128).ravel()
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-300))


@pytest.fixture(scope="session")
def tol():
    # parity bar of this path: relative L2 <= 1e-5, max element relative error <= 1e-4 in complex fp32
    return {"l2": 1e-5, "max": 1e-4}
