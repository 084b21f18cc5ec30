import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "sparse-ops_amd")
for p in (PKG, os.path.join(PKG, "python"), os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own kernels, compiled from its sources (oracle/_ref)."""
    from oracle import Ref
    if not Ref.available():
        pytest.skip("oracle/_ref not built or host lacks avx512f")
    return Ref()


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(ROOT, "tests", "golden", "ref_vectors.npz")
    return np.load(path, allow_pickle=False)


@pytest.fixture(scope="session")
def ctx():
    """One C-ABI context on the GPU for the whole session; a missing library or
    device is an error, not a skip: GPU tests must run the HIP path."""
    import hipabi
    c = hipabi.Context()
    yield c
    c.close()


@pytest.fixture(scope="session")
def backend():
    import sparseops_backend
    return sparseops_backend


def as_oracle(E):
    from oracle import EllpackArrays
    return EllpackArrays(E.m, E.n, E.r, E.Wd, E.idx, E.nnz)


def sparse_matrix(rng, m, n, sparsity, signed=True):
    """The reference unit tests' generator (tests/unit/test_matmul.py:5-9:
    rand, zero where < sparsity), seeded; `signed` draws N(0,1) values instead."""
    if signed:
        W = rng.standard_normal((m, n)).astype(np.float32)
        W[rng.random((m, n)) < sparsity] = 0.0
    else:
        W = rng.random((m, n)).astype(np.float32)
        W[W < sparsity] = 0.0
    return W


def rel_err(y, ref64):
    """max|y - ref| / max|ref|: the metric used for fp32 outputs (bound 1e-5)."""
    ref64 = np.asarray(ref64, dtype=np.float64)
    if ref64.size == 0:
        return 0.0
    return float(np.abs(np.asarray(y, dtype=np.float64) - ref64).max() / max(np.abs(ref64).max(), 1e-30))
