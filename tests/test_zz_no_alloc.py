"""so_ellpack_encode_noalloc -- the device encoder for callers that cannot allocate -- against
so_ellpack_encode (same kernels, library-allocated scratch and outputs) and the host encoder,
bit for bit, through the C ABI: two calls in a row on one context, the second on a smaller
matrix (the static scratch array keeps the first call's partial results), then the limits."""

import numpy as np
import pytest

from conftest import sparse_matrix

import datagen
import hipabi

pytestmark = pytest.mark.gpu


def _check(ctx, W, r_cap, dWd, dIdx, dNnz):
    m, n = W.shape
    E = datagen.encode_dense(W)                    # host encoder (bit-exact with the reference's)
    dW = ctx.array(W)
    dE = ctx.encode_dense(dW, m, n)                # the allocating entry point
    Wd0, idx0, nnz0 = dE.download()
    r, total = ctx.encode_dense_noalloc(dW, m, n, r_cap, dWd, dIdx, dNnz)
    assert r == dE.r == E.r and total == int(E.nnz.sum())
    nnz = dNnz.download()[:m]
    Wd = dWd.download().reshape(-1)[: m * r].reshape(m, r)
    idx = dIdx.download().reshape(-1)[: m * r].reshape(m, r)
    assert np.array_equal(nnz, nnz0) and np.array_equal(nnz, E.nnz)
    assert np.array_equal(idx, idx0) and np.array_equal(idx, E.idx.reshape(m, r))
    assert np.array_equal(Wd.view(np.uint32), Wd0.view(np.uint32))
    assert np.array_equal(Wd.view(np.uint32), E.Wd.reshape(m, r).view(np.uint32))
    dW.free()
    dE.free()


def test_encode_noalloc_two_calls_then_limits(ctx):
    rng = np.random.default_rng(77)
    M, R_CAP = 700, 200
    dWd, dIdx = ctx.empty((M, R_CAP)), ctx.empty((M, R_CAP), np.uint32)
    dNnz = ctx.empty((M,), np.uint32)
    # poison the outputs: every slot the encoder owns must be written, padding included
    dWd.upload(np.full((M, R_CAP), np.float32(7.5)))
    dIdx.upload(np.full((M, R_CAP), 0xDEADBEEF, np.uint32))

    W1 = sparse_matrix(rng, 700, 1000, .85)
    W1[2, 1] = np.nan
    W1[3, 0] = -0.0
    W1[4] = 0
    _check(ctx, W1, R_CAP, dWd, dIdx, dNnz)

    W2 = sparse_matrix(rng, 37, 130, .6)           # smaller: fewer workgroups than the first call left partials for
    _check(ctx, W2, R_CAP, dWd, dIdx, dNnz)

    W3 = np.zeros((5, 9), np.float32)              # r = 0
    _check(ctx, W3, R_CAP, dWd, dIdx, dNnz)
    _check(ctx, W1, R_CAP, dWd, dIdx, dNnz)        # and the large one again

    # without counts the call does not wait; the result is the same
    dW = ctx.array(W2)
    assert ctx.encode_dense_noalloc(dW, 37, 130, R_CAP, dWd, dIdx, dNnz, want_counts=False) is None
    E2 = datagen.encode_dense(W2)
    assert np.array_equal(dWd.download().reshape(-1)[: 37 * E2.r].view(np.uint32), E2.Wd.reshape(-1).view(np.uint32))

    # a row longer than the caller's capacity: nothing packed, clear error, dNnz valid
    before = dWd.download().copy()
    with pytest.raises(hipabi.SoError, match="longest row"):
        ctx.encode_dense_noalloc(dW, 37, 130, 3, dWd, dIdx, dNnz)
    assert np.array_equal(dWd.download().view(np.uint32), before.view(np.uint32))
    assert np.array_equal(dNnz.download()[:37], E2.nnz)
    # more rows than the static scratch array has partial results for
    with pytest.raises(hipabi.SoError, match="static scratch"):
        ctx.encode_dense_noalloc(dW, (1 << 20) + 1, 1, 1, dWd, dIdx, dNnz)
    # empty matrices
    assert ctx.encode_dense_noalloc(None, 0, 0, 0, None, None, None) == (0, 0)
    assert ctx.encode_dense_noalloc(None, 5, 0, 0, None, None, dNnz) == (0, 0)
    assert np.array_equal(dNnz.download()[:5], np.zeros(5, np.uint32))
    for a in (dW, dWd, dIdx, dNnz):
        a.free()
