"""so_conv2d (implicit im2col), so_maxpool, so_gap, so_add, so_act, so_transpose on
the GPU against the oracle: bit-exact for everything whose arithmetic is fixed
(conv with NONE/RELU, max, the ordered GAP sum, add, relu, transpose), 1e-6
relative for the sigmoid/tanh library calls."""

import numpy as np
import pytest

from conftest import as_oracle, rel_err, sparse_matrix

import datagen
import hipabi

pytestmark = pytest.mark.gpu


def gpu_conv(ctx, E, g, X, B, bias, act="none", window=None, residual=None):
    """window=True forces the LDS-windowed kernel (and requires that the plan offers it),
    False forbids it, None leaves the library's own choice."""
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, g)
    if window:
        assert ctx.conv_plan_window(plan) is not None and B % 4 == 0
    with ctx.tuning(SPARSEOPS_CONV_WINDOW=None if window is None else ("1" if window else "0")):
        return _gpu_conv(ctx, dE, plan, g, X, B, bias, act, residual)


def _gpu_conv(ctx, dE, plan, g, X, B, bias, act, residual=None):
    dX, dY = ctx.array(X), ctx.empty((g.Cout, g.H_out, g.W_out, B))
    dB = ctx.array(bias) if bias is not None else None
    dR = ctx.array(residual) if residual is not None else None
    ctx.conv2d(plan, dX, B, dB, dY, act, residual=dR)
    Y = dY.download()
    ctx.conv_plan_free(plan)
    dE.free()
    for a in (dX, dY, dB, dR):
        if a is not None:
            a.free()
    return Y


CASES = [(5, 7, 9, 11, 3, (3, 3), (1, 1), (1, 1), (1, 1)), (5, 7, 9, 11, 3, (3, 3), (2, 2), (1, 1), (1, 1)),
         (8, 16, 14, 14, 32, (1, 1), (2, 2), (0, 0), (1, 1)), (3, 4, 10, 10, 5, (3, 2), (1, 2), (2, 0), (2, 1)),
         (16, 32, 28, 28, 32, (3, 3), (1, 1), (1, 1), (1, 1)), (3, 64, 32, 32, 8, (7, 7), (2, 2), (3, 3), (1, 1)),
         (4, 3, 6, 6, 1, (3, 3), (1, 1), (0, 0), (1, 1)), (2, 9, 5, 5, 64, (5, 5), (1, 1), (2, 2), (1, 1)),
         (64, 64, 8, 8, 16, (3, 3), (1, 1), (1, 1), (1, 1))]


@pytest.mark.parametrize("Cin,Cout,H,Wi,B,k,s,p,d", CASES)
def test_conv_bit_exact(ctx, oracle, Cin, Cout, H, Wi, B, k, s, p, d):
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(Cin * 100 + H + B)
    Wc = sparse_matrix(rng, Cout, Cin * k[0] * k[1], .7)
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d), ocg(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
    for act in ("none", "relu"):
        for bias in (b, None):
            assert np.array_equal(gpu_conv(ctx, E, g, X, B, bias, act), oracle.conv2d_pf(as_oracle(E), og, X, B, bias, act))
    for act in ("sigmoid", "tanh"):
        assert rel_err(gpu_conv(ctx, E, g, X, B, b, act), oracle.conv2d_pf(as_oracle(E), og, X, B, b, act)) <= 1e-6


# (Cin, Cout, H, W, B, kernel, stride, pad, dilation, sparsity): shapes the windowed kernel takes
WINDOW_CASES = [
    (16, 32, 28, 28, 32, (3, 3), (1, 1), (1, 1), (1, 1), .7),     # whole tiles, 3 chunks (16 = 7 + 7 + 2)
    (9, 21, 13, 11, 32, (3, 3), (1, 1), (1, 1), (1, 1), .5),      # ragged tiles, channels and channel block
    (16, 24, 30, 30, 16, (3, 3), (2, 2), (1, 1), (1, 1), .6),     # stride 2, batch tile 16
    (3, 64, 32, 32, 32, (7, 7), (2, 2), (3, 3), (1, 1), .7),      # stem: one channel per chunk
    (8, 8, 12, 12, 64, (3, 3), (1, 1), (2, 2), (2, 2), .5),       # dilation 2, two batch tiles
    (4, 5, 10, 17, 48, (3, 2), (1, 2), (2, 0), (2, 1), .3),       # odd kernel, strides and pads; batch 48 = 3 tiles of 16
    (2, 9, 9, 9, 32, (5, 5), (1, 1), (2, 2), (1, 1), .5),         # 5x5
    (64, 64, 8, 8, 16, (3, 3), (1, 1), (1, 1), (1, 1), .8),       # 10 chunks, image smaller than... one tile row
    (20, 6, 6, 6, 32, (1, 1), (1, 1), (0, 0), (1, 1), .3),        # 1x1 with enough nonzeros per chunk
    (16, 32, 28, 28, 8, (3, 3), (1, 1), (1, 1), (1, 1), .7),      # batch tile 8
    (9, 21, 13, 11, 24, (3, 3), (2, 2), (1, 1), (1, 1), .5),      # batch 24 = 3 tiles of 8
    (16, 24, 30, 30, 4, (3, 3), (1, 1), (1, 1), (1, 1), .6),      # batch tile 4 (half the lanes of a wave idle)
    (3, 64, 32, 32, 12, (7, 7), (2, 2), (3, 3), (1, 1), .7),      # batch 12 = 3 tiles of 4
    (64, 48, 28, 28, 32, (1, 1), (2, 2), (0, 0), (1, 1), .5),     # 1x1 stride 2 (a ResNet projection): the window holds every second pixel only
    (32, 40, 15, 13, 8, (1, 1), (2, 3), (0, 0), (1, 1), .3),      # 1x1, strides 2 and 3, ragged tiles
    (16, 24, 20, 20, 16, (1, 3), (2, 2), (0, 1), (1, 1), .5),     # one tap along h only: subsampled rows, full columns
    (16, 24, 21, 20, 4, (3, 1), (2, 2), (1, 0), (1, 1), .5),      # and the other way round, batch tile 4
]


@pytest.mark.parametrize("Cin,Cout,H,Wi,B,k,s,p,d,sp", WINDOW_CASES)
def test_conv_lds_window_kernel(ctx, oracle, Cin, Cout, H, Wi, B, k, s, p, d, sp):
    """The LDS-windowed kernel gives the gather kernel's and the oracle's bits."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(Cin * 1000 + Cout * 10 + B)
    Wc = sparse_matrix(rng, Cout, Cin * k[0] * k[1], sp)
    Wc[Cout // 2] = 0                                      # an output channel without nonzeros
    if Cout > 3:
        Wc[1] = rng.standard_normal(Wc.shape[1])           # a dense one: every chunk full
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d), ocg(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
    for act in ("none", "relu"):
        for bias in (b, None):
            Yo = oracle.conv2d_pf(as_oracle(E), og, X, B, bias, act)
            assert np.array_equal(gpu_conv(ctx, E, g, X, B, bias, act, window=True), Yo)
    assert np.array_equal(gpu_conv(ctx, E, g, X, B, b, "none", window=False), oracle.conv2d_pf(as_oracle(E), og, X, B, b))
    assert rel_err(gpu_conv(ctx, E, g, X, B, b, "tanh", window=True), oracle.conv2d_pf(as_oracle(E), og, X, B, b, "tanh")) <= 1e-6


@pytest.mark.parametrize("Cin,Cout,H,B,sp", [(64, 64, 28, 32, .8), (256, 96, 7, 16, .8), (96, 40, 14, 48, .7)])
def test_conv_lds_window_kernel_many_launches(ctx, oracle, Cin, Cout, H, B, sp):
    """Several chunks per workgroup on the 16-entry batch tile: the waves synchronise through
    progress counters in LDS instead of barriers.  Every one of many back-to-back launches gives
    the oracle's bits (a race between a window's stores and its reads would show up as a launch
    that differs)."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(Cin + Cout + H)
    Wc = sparse_matrix(rng, Cout, Cin * 9, sp)
    X = rng.standard_normal((Cin, H, H, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, H, (1, 1), (1, 1), (1, 1)), ocg(Cin, Cout, 3, 3, H, H, (1, 1), (1, 1), (1, 1))
    Yo = oracle.conv2d_pf(as_oracle(E), og, X, B, b, "relu")
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, g)
    ctx.conv_plan_tune(plan, B)
    win = ctx.conv_plan_window(plan)
    assert win is not None and win["chunks"] >= 2
    dX, dB = ctx.array(X), ctx.array(b)
    outs = [ctx.empty((Cout, g.H_out, g.W_out, B)) for _ in range(4)]
    with ctx.tuning(SPARSEOPS_CONV_WINDOW="1"):
        for rep in range(25):
            for dY in outs:                                  # four launches in flight behind one another
                ctx.conv2d(plan, dX, B, dB, dY, "relu")
            for dY in outs:
                assert np.array_equal(dY.download(), Yo), "launch %d differs" % rep
    ctx.sync()                                               # fails if a wave gave up waiting on the progress counters
    ctx.conv_plan_free(plan)
    dE.free()
    for a in [dX, dB] + outs:
        a.free()


@pytest.mark.parametrize("B,window", [(3, False), (4, False), (32, False), (32, True), (16, True), (8, True), (4, True)])
def test_conv_with_fused_residual_add(ctx, oracle, B, window):
    """so_conv2d_add == conv, then the reference's Add, then the activation: same bits as
    the three layers one after the other, in both convolution kernels."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(B)
    Cin, Cout, H, Wi, k = 12, 10, 9, 13, (3, 3)
    Wc = sparse_matrix(rng, Cout, Cin * 9, .6)
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    R = rng.standard_normal((Cout, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1)), ocg(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1))
    conv = oracle.conv2d_pf(as_oracle(E), og, X, B, b)
    for act in ("none", "relu"):
        want = oracle.act(oracle.add(conv, R), act)
        assert np.array_equal(gpu_conv(ctx, E, g, X, B, b, act, window=window, residual=R), want)
    want = oracle.act(oracle.add(conv, R), "tanh")
    assert rel_err(gpu_conv(ctx, E, g, X, B, b, "tanh", window=window, residual=R), want) <= 1e-6


def test_conv_plan_tune_changes_layout_not_results(ctx, oracle):
    """so_conv_plan_tune re-sizes the windowed layout for a batch; outputs keep their bits."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(77)
    Cin, Cout, H, Wi = 32, 64, 56, 56
    Wc = sparse_matrix(rng, Cout, Cin * 9, .8)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1)), ocg(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1))
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, g)
    seen = set()
    for B in (16, 32, 128, 16):
        ctx.conv_plan_tune(plan, B)
        seen.add(ctx.conv_plan_window(plan)["channels_per_wave"])
        Bx = 16                                           # results for a batch of 16 under every tuning
        X = rng.standard_normal((Cin, H, Wi, Bx)).astype(np.float32)
        dX, dY = ctx.array(X), ctx.empty((Cout, H, Wi, Bx))
        ctx.conv2d(plan, dX, Bx, None, dY, "relu")
        assert np.array_equal(dY.download(), oracle.conv2d_pf(as_oracle(E), og, X, Bx, None, "relu"))
        dX.free()
        dY.free()
    assert len(seen) > 1                                  # fewer channels per wave for the small batch
    ctx.conv_plan_free(plan)
    dE.free()


@pytest.mark.parametrize("Cin,Cout,H,Wi,s", [(128, 96, 7, 7, 1), (64, 80, 14, 14, 1), (40, 48, 28, 28, 1), (48, 64, 15, 13, 2)])
@pytest.mark.parametrize("B", [4, 8, 16])
def test_conv_plan_tuned_for_small_batches(ctx, oracle, Cin, Cout, H, Wi, s, B):
    """A plan tuned for a batch tile of 4 or 8 takes pixel tiles of a whole wave (64 or 32 pixels)
    and, on small images, fewer computing waves per workgroup; entries are held in lanes.  Deep
    layers on small images, several channel chunks, an empty and a dense output channel."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(Cin + Cout * 7 + H * 31 + B)
    Wc = sparse_matrix(rng, Cout, Cin * 9, .8)
    Wc[5] = 0
    Wc[Cout - 1] = rng.standard_normal(Cin * 9)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, Wi, (s, s), (1, 1)), ocg(Cin, Cout, 3, 3, H, Wi, (s, s), (1, 1))
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, g)
    ctx.conv_plan_tune(plan, B)
    win = ctx.conv_plan_window(plan)
    assert win is not None
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    R = rng.standard_normal((Cout, g.H_out, g.W_out, B)).astype(np.float32)
    Yo = oracle.conv2d_pf(as_oracle(E), og, X, B, b, "none")
    with ctx.tuning(SPARSEOPS_CONV_WINDOW="1"):
        assert np.array_equal(_conv_keep_plan(ctx, plan, g, X, B, b, "none"), Yo)
        assert np.array_equal(_conv_keep_plan(ctx, plan, g, X, B, None, "relu"), oracle.conv2d_pf(as_oracle(E), og, X, B, None, "relu"))
        assert np.array_equal(_conv_keep_plan(ctx, plan, g, X, B, b, "relu", R), oracle.act(oracle.add(Yo, R), "relu"))
        with ctx.tuning(SPARSEOPS_CONV_MIN_CG="16"):          # the same launch without shrinking the channel groups
            assert np.array_equal(_conv_keep_plan(ctx, plan, g, X, B, b, "none"), Yo)
    ctx.conv_plan_free(plan)
    dE.free()


def _conv_keep_plan(ctx, plan, g, X, B, bias, act, residual=None):
    dX, dY = ctx.array(X), ctx.empty((g.Cout, g.H_out, g.W_out, B))
    dB = ctx.array(bias) if bias is not None else None
    dR = ctx.array(residual) if residual is not None else None
    ctx.conv2d(plan, dX, B, dB, dY, act, residual=dR)
    Y = dY.download()
    for a in (dX, dY, dB, dR):
        if a is not None:
            a.free()
    return Y


def test_conv_reference_vectors(ctx, golden):
    for i, c in enumerate(golden["conv_cases"]):
        Cin, Cout, H, Wi, B = (int(v) for v in c[:5])
        k, s, p, d = [tuple(int(v) for v in c[j:j + 2]) for j in (5, 7, 9, 11)]
        g = hipabi.conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
        E = datagen.encode_dense(golden["conv%d_W" % i])
        X, b = golden["conv%d_X" % i], golden["conv%d_b" % i]
        assert np.array_equal(gpu_conv(ctx, E, g, X, B, b), golden["conv%d_Y" % i])
        assert np.array_equal(gpu_conv(ctx, E, g, X, B, b, "relu"), golden["conv%d_Yrelu" % i])


def test_conv_special_cases(ctx, oracle):
    rng = np.random.default_rng(12)
    Cin, Cout, H, Wi, B = 6, 5, 7, 9, 4
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    W = sparse_matrix(rng, Cout, Cin, .4)
    E = datagen.encode_dense(W)
    # 1x1 conv == so_matmul on [Cin x H*W*B], bit for bit
    Y = gpu_conv(ctx, E, hipabi.conv_geom(Cin, Cout, 1, 1, H, Wi), X, B, b)
    assert np.array_equal(Y.reshape(Cout, -1), oracle.matmul(as_oracle(E), X.reshape(Cin, -1), b))
    # delta kernel at the centre of a padded 3x3 is the identity
    W4 = np.zeros((Cin, Cin, 3, 3), np.float32)
    W4[np.arange(Cin), np.arange(Cin), 1, 1] = 1
    Y = gpu_conv(ctx, datagen.encode_dense(W4.reshape(Cin, -1)), hipabi.conv_geom(Cin, Cin, 3, 3, H, Wi, pad=(1, 1)), X, B, None)
    assert np.array_equal(Y, X)
    # padding taps are skipped, not multiplied: inf at the border must not leak NaN through zero weights
    Xi = X.copy()
    Xi[:, 0, 0, :] = np.inf
    Y = gpu_conv(ctx, datagen.encode_dense(W4.reshape(Cin, -1)), hipabi.conv_geom(Cin, Cin, 3, 3, H, Wi, pad=(1, 1)), Xi, B, None)
    assert np.array_equal(Y, Xi)


def test_conv_plan_validation(ctx):
    E = datagen.encode_dense(np.ones((4, 18), np.float32))
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    g = hipabi.conv_geom(2, 4, 3, 3, 8, 8)
    bad = hipabi.conv_geom(3, 4, 3, 3, 8, 8)             # K mismatch
    with pytest.raises(hipabi.SoError):
        ctx.conv_plan(dE, bad)
    wrong = hipabi.conv_geom(2, 4, 3, 3, 8, 8)
    wrong.H_out = 7                                       # not the loader's formula
    with pytest.raises(hipabi.SoError):
        ctx.conv_plan(dE, wrong)
    ctx.conv_plan_free(ctx.conv_plan(dE, g))
    dE.free()


@pytest.mark.parametrize("C,H,Wi,B,k,s,p", [(3, 8, 8, 2, (2, 2), (2, 2), (0, 0)), (4, 9, 7, 3, (3, 3), (2, 2), (1, 1)),
                                           (2, 5, 6, 1, (3, 2), (1, 1), (1, 0)), (64, 56, 56, 8, (3, 3), (2, 2), (1, 1)),
                                           (5, 11, 13, 4, (3, 3), (2, 2), (1, 1)), (3, 7, 7, 12, (2, 3), (1, 2), (0, 1))])
def test_maxpool(ctx, oracle, C, H, Wi, B, k, s, p):
    rng = np.random.default_rng(C + H)
    X = rng.standard_normal((C, H, Wi, B)).astype(np.float32)
    Yo = oracle.maxpool_pf(X, C, H, Wi, B, k, s, p)
    dY = ctx.empty(Yo.shape)
    ctx.maxpool(C, H, Wi, k, s, p, ctx.array(X), B, dY)
    assert np.array_equal(dY.download(), Yo)


def test_gap_add_act_transpose(ctx, oracle):
    rng = np.random.default_rng(3)
    C, H, Wi, B = 37, 7, 6, 33
    X = rng.standard_normal((C, H, Wi, B)).astype(np.float32)
    dX = ctx.array(X)
    Yo = oracle.gap_pf(X, C, H, Wi, B)
    dY = ctx.empty(Yo.shape)
    ctx.gap(C, H, Wi, dX, B, dY)
    assert np.array_equal(dY.download(), Yo)
    A = rng.standard_normal(X.shape).astype(np.float32)
    dA, dD = ctx.array(A), ctx.empty(X.shape)
    ctx.add(dX, dA, X.size, dD)
    assert np.array_equal(dD.download(), oracle.add(X, A))
    ctx.add(dX, dA, X.size, dA)                          # in place on an operand
    assert np.array_equal(dA.download(), X + A)
    V = (rng.standard_normal(100003) * 4).astype(np.float32)
    dV, dO = ctx.array(V), ctx.empty(V.shape)
    for act in ("none", "relu", "sigmoid", "tanh"):
        ctx.act(act, dV, V.size, dO)
        if act in ("none", "relu"):
            assert np.array_equal(dO.download(), oracle.act(V, act))
        else:
            assert rel_err(dO.download(), oracle.act(V, act)) <= 1e-6
    for (r, c) in [(70, 130), (1, 1), (64, 64), (32, 150528 // 64), (1000, 3)]:
        S = rng.standard_normal((r, c)).astype(np.float32)
        dT = ctx.empty((c, r))
        ctx.transpose(ctx.array(S), r, c, dT)
        assert np.array_equal(dT.download(), S.T)


def test_add_long_and_unaligned(ctx):
    """so_add over lengths that span many 16 KB chunks plus a tail, on operands that start off a 16-byte
    boundary, and in place: D = A + B bit for bit (src/layers/add.cpp:9-76)."""
    rng = np.random.default_rng(31)
    n = 1_000_003
    A, Bv = rng.standard_normal(n + 8).astype(np.float32), rng.standard_normal(n + 8).astype(np.float32)
    dA, dB, dD = ctx.array(A), ctx.array(Bv), ctx.empty((n + 8,))
    for off, length in ((0, n), (1, n - 5), (3, 4097), (0, 1), (2, 3)):
        ctx.fill_zero(dD)
        ctx.add(dA.offset(off), dB.offset(off), length, dD.offset(off))
        got = dD.download()
        assert np.array_equal(got[off:off + length], A[off:off + length] + Bv[off:off + length])
        assert not got[off + length:].any() and not got[:off].any()
    ctx.add(dA, dB, n, dB)
    assert np.array_equal(dB.download()[:n], A[:n] + Bv[:n])


@pytest.mark.parametrize("dims", [(7, 5, 3, 32), (56, 56, 64, 4), (1, 1, 1, 1), (3, 2, 5, 33), (2, 9, 1, 7)])
def test_reverse_axes3(ctx, dims):
    """so_reverse_axes3: [d0][d1][d2][inner] -> [d2][d1][d0][inner], i.e. a Fortran-order (B,C,H,W) array
    ([W][H][C][B] in memory, include/conv_kernels.hpp:8-24) to [C][H][W][B] and back."""
    rng = np.random.default_rng(9)
    S = rng.standard_normal(dims).astype(np.float32)
    dS, dT, dR = ctx.array(S), ctx.empty((dims[2], dims[1], dims[0], dims[3])), ctx.empty(dims)
    ctx.reverse_axes3(dS, dims[0], dims[1], dims[2], dims[3], dT)
    T = dT.download()
    assert np.array_equal(T, S.transpose(2, 1, 0, 3))
    ctx.reverse_axes3(dT, dims[2], dims[1], dims[0], dims[3], dR)
    assert np.array_equal(dR.download(), S)
    # the Fortran-order reading: element (b, c, h, w) of a (B, C, H, W) array with d = (W, H, C, B)
    F = np.asfortranarray(rng.standard_normal((dims[3], dims[2], dims[1], dims[0])).astype(np.float32))
    dF = ctx.array(np.frombuffer(F.tobytes(order="F"), dtype=np.float32))
    ctx.reverse_axes3(dF, dims[0], dims[1], dims[2], dims[3], dT)
    assert np.array_equal(dT.download(), np.ascontiguousarray(F.transpose(1, 2, 3, 0)))


def test_launch_graph_replays(ctx, oracle):
    """A recorded chain replays with the same bits as eager execution, several
    times, with eager work and synchronisation in between."""
    rng = np.random.default_rng(21)
    W1, W2 = sparse_matrix(rng, 96, 64, .8), sparse_matrix(rng, 40, 96, .8)
    E1, E2 = datagen.encode_dense(W1), datagen.encode_dense(W2)
    d1 = ctx.upload_ellpack(E1.Wd, E1.idx, E1.nnz, E1.m, E1.n, E1.r)
    d2 = ctx.upload_ellpack(E2.Wd, E2.idx, E2.nnz, E2.m, E2.n, E2.r)
    C = 48
    dX, dH, dY = ctx.empty((64, C)), ctx.empty((96, C)), ctx.empty((40, C))
    ctx.graph_begin()
    ctx.matmul(d1, dX, C, None, dH, "relu")
    ctx.matmul(d2, dH, C, None, dY, "none")
    g = ctx.graph_end()
    for it in range(4):
        X = rng.standard_normal((64, C)).astype(np.float32)
        dX.upload(X)
        ctx.fill_zero(dY)
        ctx.sync()
        ctx.graph_launch(g)
        Y = dY.download()
        Yo = oracle.matmul(as_oracle(E2), oracle.matmul(as_oracle(E1), X, None, "relu"), None)
        assert np.array_equal(Y, Yo), it
    ctx.graph_free(g)


def test_conv_rows_not_in_ascending_column_order(ctx, oracle):
    """The windowed layout takes a chunk of input channels to be a slot range of every row; for weights
    whose slots are in another order the plan carries no such layout, and the gather kernel computes the
    convolution in slot order: bit-identical to the oracle on the shuffled arrays."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(78)
    Cin, Cout, H, Wi, B = 16, 24, 12, 12, 16
    E = datagen.encode_dense(sparse_matrix(rng, Cout, Cin * 9, .6))
    Wd, idx = E.Wd.copy(), E.idx.copy()
    for i in range(E.m):
        p = rng.permutation(int(E.nnz[i]))
        Wd[i, :len(p)], idx[i, :len(p)] = E.Wd[i, p], E.idx[i, p]
    Es = datagen.EllpackHost(E.m, E.n, E.r, Wd, idx, E.nnz)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1)), ocg(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1))
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, g)
    assert ctx.conv_plan_window(plan) is not None          # the sorted matrix gets the windowed layout
    ctx.conv_plan_free(plan)
    dE.free()
    dE = ctx.upload_ellpack(Es.Wd, Es.idx, Es.nnz, Es.m, Es.n, Es.r)
    plan = ctx.conv_plan(dE, g)
    assert ctx.conv_plan_window(plan) is None
    ctx.conv_plan_tune(plan, 8)
    assert ctx.conv_plan_window(plan) is None
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    Y = _gpu_conv(ctx, dE, plan, g, X, B, b, "relu")
    assert np.array_equal(Y, oracle.conv2d_pf(as_oracle(Es), og, X, B, b, "relu"))
