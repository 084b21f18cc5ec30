"""The reference's convenience names for the compiled module (python/cpp_backend.py:4-37).

encode(W)          (m, n) float32 matrix  ->  sparseops_backend.Ellpack
matvec(E, x, b)    x (n,)    ->  (m,)    = E @ x + b
matmul(E, X, b)    X (n, C)  ->  (m, C)  = E @ X + b[:, None]

`b` may be None (no bias), which the reference's binding does not accept.  The products run on the
GPU; without one they raise RuntimeError."""
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import sparseops_backend as _backend  # noqa: E402

encode = _backend.convert_to_ellpack


def matvec(E, x, bias=None):
    return _backend.ellpack_matvec(E, x, bias)


def matmul(E, X, bias=None):
    return _backend.ellpack_matmul(E, X, bias)
