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


def max_rel_elementwise(a, b, floor_frac=1e-2):
    """largest |a - b| / |b| over the elements whose reference magnitude is at least floor_frac of the largest
    reference magnitude (below that floor the ratio measures the rounding of a cancellation, not the kernel)"""
    import numpy as np
    a = np.asarray(a, dtype=np.complex128).ravel()
    b = np.asarray(b, dtype=np.complex128).ravel()
    mag = np.abs(b)
    keep = mag >= floor_frac * max(mag.max(), 1e-300)
    return float(np.max(np.abs(a - b)[keep] / mag[keep])) if keep.any() else 0.0


@pytest.fixture
def algo_1d():
    """sets the process-wide choice of the fused 1D kernel for one test and restores the choice by size afterwards.
    Selector 7 (a cluster of blocks per signal set) only runs on streams with an exchange buffer: unless attach=False,
    one is attached to torch's current stream for the rest of the test."""
    import turbofno_amd as tf
    held = []

    def choose(algo, attach=True):
        if algo == 7 and attach and not held:
            held.append(tf.ExchangeBuffer())
        return tf.set_1d_algo(algo)

    yield choose
    tf.set_1d_algo(0)
    for b in held:
        b.close()


@pytest.fixture(scope="session")
def tol():
    # parity bar of this path: relative L2 <= 1e-5, max element relative error <= 1e-4 in complex fp32
    # "max": largest element error relative to the largest reference magnitude; "elem": largest per-element ratio
    # over the elements above 1e-2 of the largest reference magnitude (max_rel_elementwise)
    return {"l2": 1e-5, "max": 1e-4, "elem": 1e-4}
