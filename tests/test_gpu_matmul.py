"""so_matmul (C ABI) and sparseops_backend.ellpack_matmul on the GPU against the
oracle.  NONE/RELU epilogues must be bit-identical to the oracle (same rounding
sequence: bias, then one FMA per stored nonzero in ascending slot order);
SIGMOID/TANH use the device's expf/tanhf and must agree to 1e-6 relative."""

import numpy as np
import pytest

from conftest import as_oracle, rel_err, sparse_matrix
from test_oracle_kernels import MATMUL_CASES

import datagen
import hipabi

pytestmark = pytest.mark.gpu
ACT_TOL = 1e-6


def gpu_matmul(ctx, E, X, bias, act="none", layouts=hipabi.LAYOUT_ROW):
    # small test shapes would be routed to the row kernel: force the LDS-staged one
    # whenever its layout is requested (library tuning override)
    with ctx.tuning(SPARSEOPS_MATMUL_TILED="1" if layouts & hipabi.LAYOUT_TILED else "0"):
        return _gpu_matmul(ctx, E, X, bias, act, layouts)


def _gpu_matmul(ctx, E, X, bias, act, layouts):
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, layouts)
    dX, dY = ctx.array(X), ctx.empty((E.m, X.shape[1]))
    dB = ctx.array(bias) if bias is not None else None
    ctx.matmul(dE, dX, X.shape[1], dB, dY, act)
    Y = dY.download()
    for a in (dX, dY, dB):
        if a is not None:
            a.free()
    dE.free()
    return Y


@pytest.mark.parametrize("m,n,C,sp", MATMUL_CASES + [(64, 96, 16, .5), (64, 96, 64, .5), (64, 96, 128, .5),
                                                     (64, 96, 192, .5), (64, 96, 256, .5), (64, 96, 320, .5),
                                                     (64, 96, 512, .8), (64, 96, 1024, .8), (7, 9, 65, .3),
                                                     (130, 70, 129, .6), (2000, 2000, 10, .3), (3000, 3000, 10, .4)])
def test_matmul_bit_exact(ctx, oracle, m, n, C, sp):
    rng = np.random.default_rng(m * 31 + n * 7 + C)
    W = sparse_matrix(rng, m, n, sp)
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    Y = gpu_matmul(ctx, E, X, b)
    assert Y.shape == (m, C)
    assert np.array_equal(Y, oracle.matmul(as_oracle(E), X, b))
    if m and C:
        assert rel_err(Y, W.astype(np.float64) @ X + b[:, None].astype(np.float64)) <= 1e-5
        # the reference's own assertion (tests/unit/test_matmul.py:48)
        assert np.allclose(Y, W @ X + b[:, None], atol=1e-5 * max(1.0, np.abs(Y).max()))


@pytest.mark.parametrize("C", [1, 10, 64, 100, 128, 256, 300])
@pytest.mark.parametrize("act", ["none", "relu", "sigmoid", "tanh"])
def test_matmul_epilogues(ctx, oracle, C, act):
    rng = np.random.default_rng(C)
    W = sparse_matrix(rng, 150, 200, .85)
    X = rng.standard_normal((200, C)).astype(np.float32)
    b = rng.standard_normal(150).astype(np.float32)
    E = datagen.encode_dense(W)
    for bias in (b, None):
        Y, Yo = gpu_matmul(ctx, E, X, bias, act), oracle.matmul(as_oracle(E), X, bias, act)
        if act in ("none", "relu"):
            assert np.array_equal(Y, Yo)
        else:
            assert rel_err(Y, Yo) <= ACT_TOL


def test_matmul_reference_vectors(ctx, golden):
    E = datagen.encode_dense(golden["enc_W"])
    b = golden["mm_bias"]
    for C in (1, 10, 16, 64, 100, 128, 256):
        X = golden["mm_X_%d" % C]
        assert np.array_equal(gpu_matmul(ctx, E, X, b), golden["mm_Y_%d" % C])
        assert np.array_equal(gpu_matmul(ctx, E, X, b, "relu"), golden["mm_Yrelu_%d" % C])
    assert np.array_equal(gpu_matmul(ctx, E, golden["mm_X_64"], None), golden["mm_Ynobias_64"])


def test_matmul_config1_and_config3(ctx, oracle):
    E, X, b, W = datagen.config1()
    assert abs(E.r - 133) < 20 and abs(E.total_nnz - 104858) < 2000
    Y = gpu_matmul(ctx, E, X, b)
    assert np.array_equal(Y, oracle.matmul(as_oracle(E), X, b))
    assert rel_err(Y, W.astype(np.float64) @ X + b[:, None]) <= 1e-5
    E, X, b = datagen.config3()
    assert E.r == 410 and E.total_nnz == 4096 * 410 and (E.nnz == 410).all()
    Y = gpu_matmul(ctx, E, X, b)
    assert np.array_equal(Y, oracle.matmul(as_oracle(E), X, b))
    # size-independent properties at full size: every column is computed
    # independently of the tiling, so one column alone gives the same bits ...
    for c in (0, 77, 255):
        assert np.array_equal(gpu_matmul(ctx, E, np.ascontiguousarray(X[:, c:c + 1]), b)[:, 0], Y[:, c])
    # ... and a permutation of X's columns permutes Y's columns
    perm = np.random.default_rng(0).permutation(256)
    assert np.array_equal(gpu_matmul(ctx, E, np.ascontiguousarray(X[:, perm]), b), Y[:, perm])


TILED = hipabi.LAYOUT_ROW | hipabi.LAYOUT_TILED


@pytest.mark.parametrize("m,n,C,sp", [(16, 32, 16, .3), (64, 128, 64, .5), (130, 300, 68, .7), (256, 512, 256, .9),
                                      (1, 1000, 32, .1), (1000, 1, 20, .1), (7, 9, 132, .3), (500, 700, 512, .95),
                                      (65, 257, 64, 0.), (300, 1000, 20, .5), (67, 1025, 200, .2), (1030, 520, 96, .98)])
@pytest.mark.parametrize("act", ["none", "relu", "tanh"])
def test_matmul_lds_tiled_layout(ctx, oracle, m, n, C, sp, act):
    """The K-tiled device layout (X staged through LDS, four rows per wave) gives the
    same bits as the row kernel: partial tiles in every dimension, empty rows, a
    dense row (more steps in a tile than the kernel keeps in registers)."""
    rng = np.random.default_rng(m * 31 + n * 7 + C)
    W = sparse_matrix(rng, m, n, sp)
    if m > 5:
        W[3] = 0
        W[m - 2] = rng.standard_normal(n)
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    for bias in (b, None):
        Y, Yo = gpu_matmul(ctx, E, X, bias, act, TILED), oracle.matmul(as_oracle(E), X, bias, act)
        if act == "tanh":
            assert rel_err(Y, Yo) <= ACT_TOL
        else:
            assert np.array_equal(Y, Yo)


@pytest.mark.parametrize("m,n,C", [(300, 2100, 512), (260, 2100, 640), (520, 4200, 256), (130, 1100, 1024)])
def test_matmul_lds_tiled_x_larger_than_an_l2(ctx, oracle, m, n, C):
    """X above 4 MiB: the kernel deals column slabs (not whole row groups) to the XCDs,
    with a slab count that divides 8 (C = 256, 512), does not (640), or exceeds it (1024)."""
    assert n * C * 4 > 4 << 20
    rng = np.random.default_rng(m + n + C)
    W = sparse_matrix(rng, m, n, .9)
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    assert np.array_equal(gpu_matmul(ctx, E, X, b, "relu", TILED), oracle.matmul(as_oracle(E), X, b, "relu"))


def test_matmul_lds_tiled_reference_vectors_and_config3(ctx, oracle, golden):
    E = datagen.encode_dense(golden["enc_W"])
    b = golden["mm_bias"]
    for C in (16, 64, 100, 128, 256):
        X = golden["mm_X_%d" % C]
        assert np.array_equal(gpu_matmul(ctx, E, X, b, "none", TILED), golden["mm_Y_%d" % C])
        assert np.array_equal(gpu_matmul(ctx, E, X, b, "relu", TILED), golden["mm_Yrelu_%d" % C])
    E, X, b = datagen.config3()
    Y = gpu_matmul(ctx, E, X, b, "none", TILED)
    assert np.array_equal(Y, oracle.matmul(as_oracle(E), X, b))
    assert np.array_equal(Y, gpu_matmul(ctx, E, X, b))                  # row kernel, same bits
    Xi = X.copy()
    Xi[0, :] = np.inf                                                   # padded steps must not touch X
    rows_without_col0 = E.idx[:, 0] != 0
    Yi = gpu_matmul(ctx, E, Xi, b, "none", TILED)
    assert np.isfinite(Yi[rows_without_col0]).all() and np.array_equal(Yi[rows_without_col0], Y[rows_without_col0])


@pytest.mark.parametrize("m,n,C,sp", [(1024, 2048, 256, .9), (200, 1300, 64, .7), (64, 5000, 128, .95)])
def test_matmul_lds_tiled_many_launches(ctx, oracle, m, n, C, sp):
    """Several K-tiles per workgroup: the waves synchronise through progress counters in LDS
    instead of a barrier per tile.  Every one of many back-to-back launches gives the oracle's
    bits (a race between a tile's stores and its reads would show up as a launch that differs)."""
    rng = np.random.default_rng(m + n + C)
    W = sparse_matrix(rng, m, n, sp)
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    Yo = oracle.matmul(as_oracle(E), X, b)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, TILED)
    dX, dB = ctx.array(X), ctx.array(b)
    outs = [ctx.empty((m, C)) for _ in range(4)]
    with ctx.tuning(SPARSEOPS_MATMUL_TILED="1"):
        for rep in range(25):
            for dY in outs:                                  # four launches in flight behind one another
                ctx.matmul(dE, dX, C, dB, dY, "none")
            for dY in outs:
                assert np.array_equal(dY.download(), Yo), "launch %d differs" % rep
    ctx.sync()                                               # fails if a wave gave up waiting on the progress counters
    dE.free()
    for a in [dX, dB] + outs:
        a.free()


def test_matmul_lds_tiled_keeps_negative_zero(ctx, oracle):
    """Rows that share a wave with longer rows run padding steps; those must leave a
    -0.0 accumulator (bias -0.0, no contribution yet) as it is, sign bit included."""
    rng = np.random.default_rng(5)
    W = sparse_matrix(rng, 64, 512, .8)
    W[::3] = 0                                   # empty rows next to populated ones
    W[1, :] = 0
    W[1, 7] = 2.0                                # one nonzero, late K-tiles are padding only
    X = rng.standard_normal((512, 64)).astype(np.float32)
    X[7, :] = -0.0                               # 2 * -0 = -0 on top of bias -0
    b = np.full(64, -0.0, np.float32)
    E = datagen.encode_dense(W)
    Yo = oracle.matmul(as_oracle(E), X, b)
    assert np.signbit(Yo[0]).all() and np.signbit(Yo[1]).all()
    for layouts in (TILED, hipabi.LAYOUT_ROW):
        Y = gpu_matmul(ctx, E, X, b, "none", layouts)
        assert np.array_equal(Y, Yo) and np.array_equal(np.signbit(Y), np.signbit(Yo))


@pytest.mark.parametrize("m,n,C,sp", [(1, 1000, 32, .1), (3, 5000, 100, .8), (10, 4096, 256, .9), (2, 3000, 64, 0.),
                                      (7, 700, 132, .3), (4, 200, 64, .1), (5, 6000, 20, .5), (1, 130, 1, 0.),
                                      (1, 513, 64, 0.), (2, 1025, 70, 0.)])
@pytest.mark.parametrize("act", ["none", "relu", "tanh"])
def test_matmul_few_rows_shared_gather(ctx, oracle, m, n, C, sp, act):
    """At most one (row, 64-column tile) per CU and rows of 128 nonzeros or more: the 16 waves of a
    workgroup gather one row's X segments into LDS and its first wave accumulates them in slot
    order.  Rows longer than one 512-slot chunk, rows that end inside a wave's share, an empty
    row, a partial column tile, an infinite X entry next to slots that must not be read."""
    rng = np.random.default_rng(m * 131 + n + C)
    W = sparse_matrix(rng, m, n, sp)
    if m > 2:
        W[1] = 0
    X = rng.standard_normal((n, C)).astype(np.float32)
    X[0, 0] = np.inf
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    assert E.nnz.max() >= 128
    results = []
    for share in ("1", "0"):           # "0": the same launch on the row kernel
        with ctx.tuning(SPARSEOPS_MATMUL_SHARE=share):
            for bias in (b, None):
                Y, Yo = _gpu_matmul(ctx, E, X, bias, act, hipabi.LAYOUT_ROW), oracle.matmul(as_oracle(E), X, bias, act)
                if act == "tanh":
                    assert rel_err(Y[np.isfinite(Yo)], Yo[np.isfinite(Yo)]) <= ACT_TOL
                else:
                    assert np.array_equal(Y, Yo, equal_nan=True)
                results.append(Y)
    assert np.array_equal(results[0], results[2], equal_nan=True) and np.array_equal(results[1], results[3], equal_nan=True)


def test_matmul_degenerate_shapes(ctx, oracle):
    # zero-sized launches are early-outs, not HIP errors
    for (m, n, C) in [(0, 0, 0), (0, 5, 3), (5, 0, 3), (5, 4, 0)]:
        W = np.ones((m, n), np.float32)
        E = datagen.encode_dense(W)
        b = np.arange(m, dtype=np.float32)
        Y = gpu_matmul(ctx, E, np.ones((n, C), np.float32), b)
        assert Y.shape == (m, C)
        if Y.size:
            assert np.array_equal(Y, np.repeat(b[:, None], C, axis=1))     # r = 0: bias only
    E = datagen.encode_dense(np.zeros((32, 32), np.float32))              # all-zero matrix, r = 0
    assert E.r == 0
    assert np.array_equal(gpu_matmul(ctx, E, np.ones((32, 7), np.float32), None), np.zeros((32, 7), np.float32))


def test_matmul_padding_is_not_read(ctx):
    """0 * inf = NaN: a kernel that streamed padded slots (Wd = 0, idx = 0) would
    poison rows shorter than r when X[0, :] is infinite."""
    W = np.zeros((4, 6), np.float32)
    W[0, 1:5] = 1
    W[1, 2] = 2
    X = np.ones((6, 70), np.float32)
    X[0, :] = np.inf
    Y = gpu_matmul(ctx, datagen.encode_dense(W), X, None)
    assert np.isfinite(Y).all() and np.array_equal(Y[:, 0], [4, 2, 0, 0])


def test_upload_validation_and_layout_round_trip(ctx):
    rng = np.random.default_rng(4)
    E = datagen.encode_dense(sparse_matrix(rng, 50, 70, .8))
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, hipabi.LAYOUT_ROW | hipabi.LAYOUT_SLOT | hipabi.LAYOUT_BINS)
    Wd, idx, nnz = dE.download(hipabi.LAYOUT_ROW)
    assert np.array_equal(Wd, E.Wd) and np.array_equal(idx, E.idx) and np.array_equal(nnz, E.nnz)
    WdT, idxT, _ = dE.download(hipabi.LAYOUT_SLOT)                       # slot-major: WdT[k*m+i] == Wd[i*r+k]
    assert np.array_equal(WdT, E.Wd.T) and np.array_equal(idxT, E.idx.T)
    dE.free()
    bad = E.idx.copy()
    bad[3, 0] = 70
    with pytest.raises(hipabi.SoError) as e:
        ctx.upload_ellpack(E.Wd, bad, E.nnz, E.m, E.n, E.r)
    assert e.value.status == hipabi.SO_ERR_BOUNDS
    badn = E.nnz.copy()
    badn[0] = E.r + 1
    with pytest.raises(hipabi.SoError) as e:
        ctx.upload_ellpack(E.Wd, E.idx, badn, E.m, E.n, E.r)
    assert e.value.status == hipabi.SO_ERR_BOUNDS
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    with pytest.raises(hipabi.SoError):
        dE.download(hipabi.LAYOUT_SLOT)                                   # not uploaded
    dE.free()


# ---- the drop-in module: the reference's own unit cases (tests/unit/test_matmul.py:12-48), seeded

@pytest.mark.parametrize("m,n,C,sp", MATMUL_CASES)
def test_backend_matmul(backend, oracle, m, n, C, sp):
    rng = np.random.default_rng(m + n + C)
    W = sparse_matrix(rng, m, n, sp, signed=False)
    E = backend.convert_to_ellpack(W)
    X = rng.random((n, C)).astype(np.float32)
    b = rng.random(m).astype(np.float32)
    y = backend.ellpack_matmul(E, X, b)
    assert y.shape == (m, C)
    assert np.allclose(y, W @ X + np.expand_dims(b, axis=1), atol=1e-5)
    assert np.array_equal(y, oracle.matmul(oracle.encode(W), X, b))
    if m and C:
        assert np.array_equal(backend.ellpack_matmul(E, X, None), oracle.matmul(oracle.encode(W), X, None))
        # non-contiguous / float64 inputs are force-cast like the reference does (src/bindings.cpp:112-113)
        assert np.array_equal(backend.ellpack_matmul(E, np.asfortranarray(X).astype(np.float64), b), y)


@pytest.mark.parametrize("m,n,sp", [(1, 1, 0.), (7, 130, .6), (300, 257, .9), (64, 1000, .99), (5, 9, 1.)])
def test_device_decode_round_trip(ctx, oracle, golden, m, n, sp):
    """so_ellpack_decode == decode_from_ellpack: exact round trip of the encoder (the reference's
    own encoder test, tests/unit/test_ellpack_encoder.py), -0.0 dropped, NaN kept."""
    rng = np.random.default_rng(m * 13 + n)
    W = sparse_matrix(rng, m, n, sp)
    if m > 4:
        W[2, 1] = np.nan
        W[3, 0] = -0.0
    E = datagen.encode_dense(W)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    D = dE.decode()
    dE.free()
    want = oracle.decode(as_oracle(E))
    assert D.shape == (m, n) and np.array_equal(D, want, equal_nan=True)
    assert np.array_equal(np.signbit(D), np.signbit(want))          # the dropped -0.0 comes back as +0.0
    assert np.array_equal(D, np.where(W == 0, 0, W), equal_nan=True)
    # the committed reference vectors decode to the reference's own dense matrix
    Eg = datagen.encode_dense(golden["enc_W"])
    dEg = ctx.upload_ellpack(Eg.Wd, Eg.idx, Eg.nnz, Eg.m, Eg.n, Eg.r)
    assert np.array_equal(dEg.decode(), golden["enc_W"] + 0.0)
    dEg.free()


@pytest.mark.parametrize("m,n,sp", [(1, 1, 0.), (7, 130, .6), (300, 257, .9), (64, 1000, .99), (5, 9, 1.), (33, 64, .5),
                                    (1024, 1024, .9)])
def test_device_encoder_matches_host_encoder(ctx, oracle, m, n, sp):
    """so_ellpack_encode == convert_to_ellpack bit for bit (nnz, r, idx, Wd, zero padding; -0.0
    dropped, NaN kept), and the encoded matrix multiplies like the host-encoded one."""
    rng = np.random.default_rng(m * 17 + n)
    W = sparse_matrix(rng, m, n, sp)
    if m > 4:
        W[2, 1] = np.nan
        W[3, 0] = -0.0
        W[4] = 0
    E = datagen.encode_dense(W)
    dW = ctx.array(W)
    dE = ctx.encode_dense(dW, m, n)
    assert dE.r == E.r
    Wd, idx, nnz = dE.download()
    assert np.array_equal(nnz, E.nnz) and np.array_equal(idx, E.idx.reshape(m, E.r))
    assert np.array_equal(Wd.view(np.uint32), E.Wd.reshape(m, E.r).view(np.uint32))        # bits, NaN included
    assert np.array_equal(dE.decode(), oracle.decode(as_oracle(E)), equal_nan=True)
    if m > 4:
        W[2, 1] = 1.5                                     # no NaN for the product check
        dW2 = ctx.array(W)
        dE2 = ctx.encode_dense(dW2, m, n)
        X = rng.standard_normal((n, 8)).astype(np.float32)
        dX, dY = ctx.array(X), ctx.empty((m, 8))
        ctx.matmul(dE2, dX, 8, None, dY, "none")
        assert np.array_equal(dY.download(), oracle.matmul(as_oracle(datagen.encode_dense(W)), X, None))
        for a in (dW2, dX, dY):
            a.free()
        dE2.free()
    dW.free()
    dE.free()


def test_device_encoder_degenerate(ctx):
    for (m, n) in [(0, 0), (0, 5), (5, 0)]:
        dE = ctx.encode_dense(None, m, n)
        assert dE.r == 0
        dE.free()
    dZ = ctx.array(np.zeros((6, 70), np.float32))
    dE = ctx.encode_dense(dZ, 6, 70)
    assert dE.r == 0 and np.array_equal(dE.decode(), np.zeros((6, 70), np.float32))
    dZ.free()
    dE.free()
    # the column limit: 16 fully dense rows of 2^28 columns would wrap a workgroup's 32-bit nonzero count,
    # so 2^28 columns are refused (argument check only: nothing is launched and the pointer is never read)
    with pytest.raises(hipabi.SoError) as err:
        h = hipabi.ct.c_void_p()
        ctx._ck(ctx.lib.so_ellpack_encode(ctx.h, hipabi.ct.c_void_p(16), 1, 1 << 28, hipabi.ct.byref(h)))
    assert err.value.status == hipabi.SO_ERR_INVALID and "columns" in str(err.value)


def _shuffle_slots(E, rng):
    """The same matrix with every row's stored slots in a random order (as a caller filling the
    struct by hand might leave them); the reference's kernels take slots in whatever order they come."""
    Wd, idx = E.Wd.copy(), E.idx.copy()
    for i in range(E.m):
        p = rng.permutation(int(E.nnz[i]))
        Wd[i, :len(p)], idx[i, :len(p)] = E.Wd[i, p], E.idx[i, p]
    return datagen.EllpackHost(E.m, E.n, E.r, Wd, idx, E.nnz)


def test_matmul_rows_not_in_ascending_column_order(ctx, oracle):
    """The K-tiled layout walks a row's columns in ascending order; for a matrix whose slots are in
    another order it is not built (the handle reports ROW only) and so_matmul still multiplies in
    slot order, like the reference: bit-identical to the oracle on the shuffled arrays."""
    rng = np.random.default_rng(77)
    E = _shuffle_slots(datagen.encode_dense(sparse_matrix(rng, 200, 700, .8)), rng)
    X = rng.standard_normal((700, 64)).astype(np.float32)
    b = rng.standard_normal(200).astype(np.float32)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, TILED | hipabi.LAYOUT_BINS)
    layouts = hipabi.ct.c_int()
    ctx._ck(ctx.lib.so_ellpack_dims(dE.h, None, None, None, None, hipabi.ct.byref(layouts)))
    assert layouts.value == hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS
    dE.free()
    assert np.array_equal(gpu_matmul(ctx, E, X, b, "relu", TILED), oracle.matmul(as_oracle(E), X, b, "relu"))
    # a duplicated column is "not ascending" too
    E2 = datagen.encode_dense(sparse_matrix(rng, 64, 300, .5))
    E2.idx[5, 1] = E2.idx[5, 0]
    assert np.array_equal(gpu_matmul(ctx, E2, X[:300], b[:64], "none", TILED), oracle.matmul(as_oracle(E2), X[:300], b[:64]))


def test_bounded_wait_give_up_is_reported(ctx, oracle):
    """The LDS-staged kernels' waits on progress counters are bounded.  With the poll budget set to zero
    (SPARSEOPS_WAIT_SPINS=0) every wait gives up at once: the kernel still runs to its end, the waves count
    themselves in the context's status word, and the next call that waits for the stream fails with
    SO_ERR_HIP; the word is cleared by that, and a normal launch afterwards gives the oracle's bits."""
    rng = np.random.default_rng(99)
    W = sparse_matrix(rng, 256, 1024, .9)
    X = rng.standard_normal((1024, 64)).astype(np.float32)
    b = rng.standard_normal(256).astype(np.float32)
    E = datagen.encode_dense(W)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, TILED)
    dX, dY, dB = ctx.array(X), ctx.empty((256, 64)), ctx.array(b)
    ctx.sync()
    with ctx.tuning(SPARSEOPS_MATMUL_TILED="1", SPARSEOPS_WAIT_SPINS="0"):
        ctx.matmul(dE, dX, 64, dB, dY)
        with pytest.raises(hipabi.SoError) as err:
            ctx.sync()
        assert err.value.status == hipabi.SO_ERR_HIP and "gave up" in str(err.value)
        ctx.sync()                                        # reported once, then cleared
    with ctx.tuning(SPARSEOPS_MATMUL_TILED="1"):
        ctx.matmul(dE, dX, 64, dB, dY)
        Y = dY.download()                                 # so_d2h looks at the word too: no error now
    assert np.array_equal(Y, oracle.matmul(as_oracle(E), X, b))
    # the same through a read-back: so_d2h reports what so_sync would
    with ctx.tuning(SPARSEOPS_MATMUL_TILED="1", SPARSEOPS_WAIT_SPINS="0"):
        ctx.matmul(dE, dX, 64, dB, dY)
        with pytest.raises(hipabi.SoError):
            dY.download()
    ctx.sync()
    for a in (dX, dY, dB):
        a.free()
    dE.free()
