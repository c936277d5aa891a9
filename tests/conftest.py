import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def rel_fro(a, b):
    """Relative Frobenius error ||a-b|| / ||b|| in fp64; -inf entries must
    coincide and are left out of the norm."""
    import numpy as np
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    inf_a, inf_b = np.isneginf(a), np.isneginf(b)
    assert np.array_equal(inf_a, inf_b), "-inf pattern differs"
    a, b = a[~inf_a], b[~inf_b]
    denom = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / (denom if denom > 0 else 1.0))


@pytest.fixture(scope="session")
def oracle():
    from oracle import cpu_oracle
    cpu_oracle.lib()
    return cpu_oracle
