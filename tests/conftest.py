import os
import sys

import numpy as np
import pytest
import scipy.sparse

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU and the built HIP library")


def _gpu_present():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def reference_test_matrix(fmt="csr", seed=0, shape=(127, 255), density=0.1):
    """The matrix family of the reference's own tests (tests/test_module_spmm.py:63:
    scipy.sparse.random(127, 255, density=0.1), deliberately non-square with odd sizes), seeded."""
    rng = np.random.default_rng(seed)
    m = scipy.sparse.random(shape[0], shape[1], density=density, format=fmt, random_state=rng, dtype=np.float32)
    return m


@pytest.fixture(scope="session")
def adj_127x255():
    return reference_test_matrix("csr", seed=0)
