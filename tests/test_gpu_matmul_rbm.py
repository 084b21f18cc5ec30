"""so_matmul on the row-block-merged layout (SO_LAYOUT_RBM) against the oracle and the fp64 product.

The kernel adds a row's products column by column in the order of its streams, not in the row's
slot order, so the bound is the one the reference's own tests use for accumulation-order
differences: max|y - ref| <= 1e-5 * max|ref| (tests/unit/test_matmul.py:48 asserts
allclose(atol=1e-5) on data of magnitude 1), against the in-order oracle and against fp64.
Results must be the same bits on every launch."""

import numpy as np
import pytest

from conftest import as_oracle, rel_err, sparse_matrix
from test_oracle_kernels import MATMUL_CASES

import datagen
import hipabi

pytestmark = pytest.mark.gpu
TOL = 1e-5
RBM = hipabi.LAYOUT_ROW | hipabi.LAYOUT_RBM


def rbm_matmul(ctx, E, X, bias, act="none", split=None, repeat=1):
    env = {"SPARSEOPS_MATMUL_RBM": "1"}
    if split:
        env["SPARSEOPS_MATMUL_RBM_SPLIT"] = str(split)
    with ctx.tuning(**env):
        dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, RBM)
        dX, dY = ctx.array(X), ctx.empty((E.m, X.shape[1]))
        dB = ctx.array(bias) if bias is not None else None
        outs = []
        for _ in range(repeat):
            dY.upload(np.full((E.m, X.shape[1]), np.nan, np.float32))
            ctx.matmul(dE, dX, X.shape[1], dB, dY, act)
            outs.append(dY.download())
        for a in (dX, dY, dB):
            if a is not None:
                a.free()
        dE.free()
    for Y in outs[1:]:
        assert np.array_equal(Y, outs[0])
    return outs[0]


def check(Y, Yo, W, X, b):
    assert Y.shape == Yo.shape
    if Y.size == 0:
        return
    assert rel_err(Y, Yo) <= TOL
    ref64 = W.astype(np.float64) @ X.astype(np.float64) + (0 if b is None else b[:, None].astype(np.float64))
    assert rel_err(Y, ref64) <= TOL


@pytest.mark.parametrize("m,n,C,sp", [c for c in MATMUL_CASES if c[0] > 0] +
                         [(64, 96, 16, .5), (64, 96, 64, .5), (130, 70, 129, .6), (128, 4096, 64, .9), (129, 1000, 65, .5),
                          (300, 700, 256, .95), (1000, 3000, 100, .9), (2000, 2000, 10, .3), (257, 513, 320, .0)])
def test_rbm_matches_oracle(ctx, oracle, m, n, C, sp):
    rng = np.random.default_rng(m * 31 + n * 7 + C)
    W = sparse_matrix(rng, m, n, sp)
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    Y = rbm_matmul(ctx, E, X, b, repeat=2)
    check(Y, oracle.matmul(as_oracle(E), X, b), W, X, b)


@pytest.mark.parametrize("split", [1, 2, 4])
@pytest.mark.parametrize("act", ["none", "relu", "sigmoid", "tanh"])
def test_rbm_splits_and_epilogues(ctx, oracle, split, act):
    rng = np.random.default_rng(split)
    m, n, C = 300, 2100, 130
    W = sparse_matrix(rng, m, n, .9)
    W[5] = 0
    W[7] = rng.standard_normal(n)                    # a dense row: its columns take several parts
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    for bias in (b, None):
        Y = rbm_matmul(ctx, E, X, bias, act, split=split)
        Yo = oracle.matmul(as_oracle(E), X, bias, act)
        if act in ("none", "relu"):
            assert rel_err(Y, Yo) <= TOL
        else:
            # the bound holds for the sums; sigmoid (slope <= 1/4) and tanh (slope <= 1) carry their error over,
            # plus the 1e-6 by which the device's expf / tanhf differ from the host's
            pre = np.abs(oracle.matmul(as_oracle(E), X, bias, "none")).max()
            assert np.abs(Y.astype(np.float64) - Yo).max() <= TOL * pre * (0.25 if act == "sigmoid" else 1.0) + 1e-6


def test_rbm_dense_block_and_empty_matrix(ctx, oracle):
    """A fully dense 200 x 300 matrix (every column of a block has 128 or 72 pairs: 8 or 5 parts each) and an
    all-zero matrix (r = 0: no iteration at all, Y = bias)."""
    rng = np.random.default_rng(3)
    W = rng.standard_normal((200, 300)).astype(np.float32)
    X = rng.standard_normal((300, 70)).astype(np.float32)
    b = rng.standard_normal(200).astype(np.float32)
    E = datagen.encode_dense(W)
    check(rbm_matmul(ctx, E, X, b), oracle.matmul(as_oracle(E), X, b), W, X, b)
    Z = np.zeros((200, 300), np.float32)
    E = datagen.encode_dense(Z)
    assert E.r == 0
    assert np.array_equal(rbm_matmul(ctx, E, X, b), np.repeat(b[:, None], 70, axis=1))


def test_rbm_unordered_rows_and_special_values(ctx, oracle):
    """Rows whose stored columns do not ascend are fine for this layout (no order is relied on); an
    infinity in X reaches exactly the rows that use that X row, and padding never turns it into a NaN."""
    rng = np.random.default_rng(11)
    m, n, C = 140, 500, 64
    W = sparse_matrix(rng, m, n, .8)
    E = datagen.encode_dense(W)
    for i in range(m):                                   # reverse every row's stored order
        c = int(E.nnz[i])
        E.Wd[i, :c] = E.Wd[i, :c][::-1].copy()
        E.idx[i, :c] = E.idx[i, :c][::-1].copy()
    X = rng.standard_normal((n, C)).astype(np.float32)
    Y = rbm_matmul(ctx, E, X, None)
    assert rel_err(Y, W.astype(np.float64) @ X) <= TOL
    X[0, :] = np.inf                                     # row 0 of X is also what padding columns point at
    X[17, 3] = np.inf
    E = datagen.encode_dense(W)
    Y = rbm_matmul(ctx, E, X, None)
    Yo = oracle.matmul(as_oracle(E), X, None)
    assert np.array_equal(np.isfinite(Y), np.isfinite(Yo))
    assert np.array_equal(np.isnan(Y), np.isnan(Yo))
    fin = np.isfinite(Yo)
    assert np.array_equal(Y[~fin & ~np.isnan(Yo)], Yo[~fin & ~np.isnan(Yo)])
    assert np.abs(Y[fin] - Yo[fin]).max() <= TOL * np.abs(Yo[fin]).max()


def test_rbm_config1_config3_and_mlp_layers(ctx, oracle):
    E, X, b, W = datagen.config1()
    Y = rbm_matmul(ctx, E, X, b)
    assert rel_err(Y, oracle.matmul(as_oracle(E), X, b)) <= TOL
    assert rel_err(Y, W.astype(np.float64) @ X + b[:, None]) <= TOL
    E, X, b = datagen.config3()
    Y = rbm_matmul(ctx, E, X, b, repeat=3)
    assert rel_err(Y, oracle.matmul(as_oracle(E), X, b)) <= TOL
    # size-independent properties at full size: a column alone and a permutation of the columns give the same bits
    for c in (0, 77, 255):
        assert np.array_equal(rbm_matmul(ctx, E, np.ascontiguousarray(X[:, c:c + 1]), b)[:, 0], Y[:, c])
    perm = np.random.default_rng(0).permutation(256)
    assert np.array_equal(rbm_matmul(ctx, E, np.ascontiguousarray(X[:, perm]), b), Y[:, perm])
    # linearity: E (2 X) = 2 (E X) exactly (powers of two scale without rounding)
    assert np.array_equal(rbm_matmul(ctx, E, 2 * X, None), 2 * rbm_matmul(ctx, E, X, None))


def test_rbm_default_dispatch_and_workspace_growth(ctx, oracle):
    """Without the override so_matmul takes the kernel only when the launch covers the chip; launches of
    growing size on one context (the workspace grows) keep earlier results valid."""
    rng = np.random.default_rng(5)
    W = sparse_matrix(rng, 2048, 1536, .9)
    E = datagen.encode_dense(W)
    b = rng.standard_normal(2048).astype(np.float32)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, RBM)
    for C in (8, 64, 512, 1024, 64):
        X = rng.standard_normal((1536, C)).astype(np.float32)
        dX, dY, dB = ctx.array(X), ctx.empty((2048, C)), ctx.array(b)
        ctx.matmul(dE, dX, C, dB, dY, "relu")
        Y = dY.download()
        assert rel_err(Y, oracle.matmul(as_oracle(E), X, b, "relu")) <= TOL
        for a in (dX, dY, dB):
            a.free()
    dE.free()


def test_rbm_in_a_launch_graph(ctx, oracle):
    """so_matmul_reserve sizes the workspace ahead of time, so that a launch of the kernel whose workgroups
    exchange partial tiles (ksplit 2) can be recorded; the graph replays with the eager launch's bits, several
    times, with eager launches of the same handle and synchronisation in between.  Recording without the
    reservation is refused (the workspace cannot grow inside a recording), and the refusal leaves the context usable."""
    rng = np.random.default_rng(17)
    W = sparse_matrix(rng, 512, 1600, .9)
    E = datagen.encode_dense(W)
    b = rng.standard_normal(512).astype(np.float32)
    C = 128
    with ctx.tuning(SPARSEOPS_MATMUL_RBM="1", SPARSEOPS_MATMUL_RBM_SPLIT="2"):
        fresh = hipabi.Context(0)                      # a context whose workspace is still empty
        try:
            fE = fresh.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, RBM)
            fX, fY = fresh.empty((1600, C)), fresh.empty((512, C))
            fresh.graph_begin()
            with pytest.raises(hipabi.SoError, match="so_matmul_reserve"):
                fresh.matmul(fE, fX, C, None, fY, "none")
            g0 = fresh.graph_end()
            fresh.graph_free(g0)
            fresh.matmul(fE, fX, C, None, fY, "none")   # eager launches still work
            fresh.sync()
        finally:
            fresh.close()
        dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, RBM)
        dX, dY, dB = ctx.empty((1600, C)), ctx.empty((512, C)), ctx.array(b)
        ctx.matmul_reserve(dE, C)
        ctx.graph_begin()
        ctx.matmul(dE, dX, C, dB, dY, "relu")
        g = ctx.graph_end()
        for it in range(4):
            X = rng.standard_normal((1600, C)).astype(np.float32)
            dX.upload(X)
            ctx.matmul(dE, dX, C, dB, dY, "relu")
            eager = dY.download()
            ctx.fill_zero(dY)
            ctx.sync()
            ctx.graph_launch(g)
            Y = dY.download()
            assert np.array_equal(Y, eager), it
            assert rel_err(Y, oracle.matmul(as_oracle(E), X, b, "relu")) <= TOL
        ctx.graph_free(g)
        for a in (dX, dY, dB):
            a.free()
        dE.free()


@pytest.mark.parametrize("seed", range(16))
def test_rbm_random_sweep(ctx, oracle, seed):
    """Seeded random shapes, densities, K splits and sparsity patterns (uniform, a few dense columns, a few dense
    rows, whole empty row blocks) against the oracle and the fp64 product."""
    rng = np.random.default_rng(1000 + seed)
    m = int(rng.integers(1, 700))
    n = int(rng.integers(1, 2500))
    C = int(rng.choice([1, 3, 17, 63, 64, 65, 128, 200, 256, 333]))
    density = float(rng.choice([0.01, 0.05, 0.1, 0.3, 0.7]))
    W = (rng.standard_normal((m, n)) * (rng.random((m, n)) < density)).astype(np.float32)
    pattern = seed % 4
    if pattern == 1:                                   # columns that every row uses: parts of 16 pairs, many per column
        cols = rng.choice(n, size=min(n, 3), replace=False)
        W[:, cols] = rng.standard_normal((m, len(cols))).astype(np.float32)
    elif pattern == 2:                                 # dense rows: r = n
        rows = rng.choice(m, size=min(m, 2), replace=False)
        W[rows, :] = rng.standard_normal((len(rows), n)).astype(np.float32)
    elif pattern == 3 and m > 128:                     # a whole 128-row block without nonzeros
        W[:128, :] = 0
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32) if seed % 3 else None
    E = datagen.encode_dense(W)
    split = [None, 1, 2, 4][int(rng.integers(0, 4))]
    act = ["none", "relu"][seed % 2]
    Y = rbm_matmul(ctx, E, X, b, act=act, split=split, repeat=2)
    Yo = oracle.matmul(as_oracle(E), X, b, act)
    assert Y.shape == Yo.shape
    ref64 = W.astype(np.float64) @ X.astype(np.float64) + (0 if b is None else b[:, None].astype(np.float64))
    if act == "relu":
        ref64 = np.maximum(ref64, 0)
    scale = max(np.abs(ref64).max(), 1e-30)
    assert np.abs(Y - Yo).max() <= TOL * scale and np.abs(Y - ref64).max() <= TOL * scale
