import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.oracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)


def read_mtx_csr(name):
    """CSR (pos, crd, val, shape) of a MatrixMarket file under tests/golden, symmetric files expanded."""
    from scipy.io import mmread
    from scipy.sparse import csr_matrix
    A = csr_matrix(mmread(os.path.join(GOLDEN, name)))
    A.sort_indices()
    return A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(np.float64), A.shape


@pytest.fixture(scope="session")
def gpu():
    """torch + the initialised kernel library; fails (never skips) if the HIP library is absent."""
    import torch
    assert torch.cuda.is_available(), "a GPU test was collected without a GPU: run with -m 'not gpu'"
    from lapis_amd import hip
    hip.init()
    return hip
