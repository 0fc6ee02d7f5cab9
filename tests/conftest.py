import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def rel_err(actual, expected):
    """Norm-wise relative error max|a - e| / max|e| -- the quantity the 1e-4 (fp32) and 2e-2 (bf16)
    parity bounds of the benchmark are stated in."""
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    denom = np.abs(expected).max()
    if denom == 0.0:
        return float(np.abs(actual).max())
    return float(np.abs(actual - expected).max() / denom)


def elem_err(actual, expected):
    """Element-wise error max_i |a_i - e_i| / (|e_i| + rms(e)): unlike the norm-wise rel_err it sees a
    wrong small entry next to large ones; the rms term keeps entries that cancel to (almost) zero
    from demanding more than the accumulation can give."""
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    rms = float(np.sqrt(np.mean(expected * expected))) if expected.size else 0.0
    if rms == 0.0:
        return float(np.abs(actual).max()) if actual.size else 0.0
    return float((np.abs(actual - expected) / (np.abs(expected) + rms)).max())


def close(actual, expected, tol):
    """Both bounds: norm-wise (the benchmark's stated tolerance) and element-wise."""
    return rel_err(actual, expected) <= tol and elem_err(actual, expected) <= tol


@pytest.fixture(scope="session")
def mi():
    """The ctypes binding of libmi_mlp.so; fails (not skips) when the library is not built."""
    import tbb_test_amd
    tbb_test_amd.lib()
    return tbb_test_amd


FP32_TOL = 1e-4  # rel-err bound for fp32 Y / dX / dW / updated W
BF16_TOL = 2e-2  # rel-err bound for the bf16 path against the fp32 CPU oracle
