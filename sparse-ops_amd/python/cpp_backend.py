"""Thin wrappers with the reference's names (python/cpp_backend.py:4-37): encode / matvec / matmul."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import sparseops_backend  # noqa: E402


def encode(sparse_matrix: np.ndarray) -> "sparseops_backend.Ellpack":
    """(M, K) dense float32 matrix -> ELLPACK handle."""
    return sparseops_backend.convert_to_ellpack(sparse_matrix)


def matvec(E, x, bias=None) -> np.ndarray:
    """y = E @ x + bias; x is (n,), returns (m,)."""
    return sparseops_backend.ellpack_matvec(E, x, bias)


def matmul(E, X, bias=None) -> np.ndarray:
    """Y = E @ X + bias[:, None]; X is (n, C), returns (m, C)."""
    return sparseops_backend.ellpack_matmul(E, X, bias)
