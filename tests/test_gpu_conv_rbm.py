"""The row-block-merged (RBM) format on the GPU: so_rbm_upload + so_conv_plan_set_rbm make so_conv2d walk
the reference's blocked-CSC re-encoding (include/rbm_conv.hpp:8-27, src/layers/rbm_conv.cpp:7-73) the way
conv2d_rbm_fmajor_implicit does (src/layers/conv_kernels.cpp:66-147).  Checked bit for bit against the
oracle's restatement of that kernel, against the per-row oracle (same bits: a row's products keep their
order), against the per-row GPU kernels, and against the reference's own RBM kernel's outputs
(tests/golden/ref_vectors.npz was written from its variant 3)."""
import numpy as np
import pytest

from conftest import as_oracle, rel_err, sparse_matrix

import datagen
import hipabi

pytestmark = pytest.mark.gpu


def rbm_conv(ctx, oracle, E, g, X, B, bias, act="none", residual=None, Ct_max=8, expect_streams=True, info=None):
    R = oracle.rbm_build(as_oracle(E), Ct_max)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, g)
    rbm = ctx.upload_rbm(R.M, R.N, R.Ct_max, R.block_union, R.krel, R.colptr, R.pair_row, R.pair_w)
    assert ctx.rbm_dims(rbm) == dict(M=E.m, N=E.n, Ct_max=Ct_max, nblocks=R.nblocks, union=len(R.krel), pairs=len(R.pair_w))
    ctx.conv_plan_tune(plan, B)
    ctx.conv_plan_set_rbm(plan, rbm)
    st = ctx.conv_plan_rbm_info(plan)
    assert (st is not None) == expect_streams
    if st is not None:
        assert st["pairs"] == E.total_nnz and st["slots"] >= st["pairs"] and st["slots_per_record"] == 2
        if info is not None:
            info.update(st)
    dX, dY = ctx.array(X), ctx.array(np.full((g.Cout, g.H_out, g.W_out, B), np.nan, np.float32))
    dB = ctx.array(bias) if bias is not None else None
    dR = ctx.array(residual) if residual is not None else None
    with ctx.tuning(SPARSEOPS_CONV_RBM="1"):                     # whatever the launch size: these shapes are small
        ctx.conv2d(plan, dX, B, dB, dY, act, residual=dR)
        Y = dY.download()
    with ctx.tuning(SPARSEOPS_CONV_RBM="0"):                     # the same plan on the per-row kernels
        ctx.fill_zero(dY)
        ctx.conv2d(plan, dX, B, dB, dY, act, residual=dR)
        Yrow = dY.download()
    ctx.conv_plan_set_rbm(plan, None)                            # detach: back to the per-row kernels for good
    assert ctx.conv_plan_rbm_info(plan) is None
    ctx.conv_plan_free(plan)
    ctx.rbm_free(rbm)
    dE.free()
    for a in (dX, dY, dB, dR):
        if a is not None:
            a.free()
    return Y, Yrow, R


RBM_CASES = [
    # Cin, Cout, H, W, B, kernel, stride, pad, dilation, sparsity
    (16, 32, 28, 28, 32, (3, 3), (1, 1), (1, 1), (1, 1), .8),     # the shape of a ResNet basic-block layer
    (64, 64, 14, 14, 16, (3, 3), (1, 1), (1, 1), (1, 1), .8),     # several input-channel chunks
    (24, 40, 13, 11, 16, (3, 3), (2, 2), (1, 1), (1, 1), .7),     # stride 2, ragged tiles
    (3, 64, 32, 32, 16, (7, 7), (2, 2), (3, 3), (1, 1), .6),      # a ResNet stem
    (64, 48, 28, 28, 32, (1, 1), (2, 2), (0, 0), (1, 1), .5),     # 1x1 stride 2 (a ResNet projection)
    (20, 6, 6, 6, 32, (1, 1), (1, 1), (0, 0), (1, 1), .3),        # one block of 6 rows
    (16, 21, 12, 12, 8, (3, 3), (1, 1), (1, 1), (1, 1), .6),      # batch tile 8; last block has 5 rows
    (16, 24, 30, 30, 4, (3, 3), (1, 1), (1, 1), (1, 1), .6),      # batch tile 4
    (9, 17, 13, 11, 24, (3, 3), (1, 1), (1, 1), (2, 2), .5),      # batch 24 = 3 tiles of 8, dilation 2
    (16, 16, 9, 9, 16, (3, 3), (1, 1), (1, 1), (1, 1), 0.),       # dense weights: every tap has 8 pairs = 4 records
    (32, 16, 10, 10, 16, (3, 3), (1, 1), (1, 1), (1, 1), .97),    # nearly empty: most taps have one pair
]


@pytest.mark.parametrize("Cin,Cout,H,Wi,B,k,s,p,d,sp", RBM_CASES)
def test_conv_rbm_bit_exact(ctx, oracle, Cin, Cout, H, Wi, B, k, s, p, d, sp):
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(Cin * 1000 + Cout * 10 + B)
    Wc = sparse_matrix(rng, Cout, Cin * k[0] * k[1], sp)
    Wc[Cout // 2] = 0                                      # an output channel without nonzeros
    if Cout > 3 and sp > 0:
        Wc[1] = rng.standard_normal(Wc.shape[1])           # a dense one
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d), ocg(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
    for act in ("none", "relu"):
        for bias in (b, None):
            Y, Yrow, R = rbm_conv(ctx, oracle, E, g, X, B, bias, act)
            want = oracle.conv2d_rbm_pf(R, og, X, B, bias, act)
            assert np.array_equal(want, oracle.conv2d_pf(as_oracle(E), og, X, B, bias, act))
            assert np.array_equal(Y, want)
            assert np.array_equal(Yrow, want)
    Y, _, R = rbm_conv(ctx, oracle, E, g, X, B, b, "tanh")
    assert rel_err(Y, oracle.conv2d_rbm_pf(R, og, X, B, b, "tanh")) <= 1e-6


def test_conv_rbm_reference_vectors(ctx, oracle, golden):
    """Outputs of the reference's conv2d_rbm_fmajor_implicit, bit for bit."""
    for i, c in enumerate(golden["rbmconv_cases"]):
        Cin, Cout, H, Wi, B = (int(v) for v in c[:5])
        k, s, p, d = [tuple(int(v) for v in c[j:j + 2]) for j in (5, 7, 9, 11)]
        g = hipabi.conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
        E = datagen.encode_dense(golden["rbmconv%d_W" % i])
        X, b = golden["rbmconv%d_X" % i], golden["rbmconv%d_b" % i]
        for act, key in (("none", "rbmconv%d_Y"), ("relu", "rbmconv%d_Yrelu")):
            Y, Yrow, _ = rbm_conv(ctx, oracle, E, g, X, B, b, act)
            assert np.array_equal(Y, golden[key % i]) and np.array_equal(Yrow, golden[key % i])


def test_conv_rbm_with_fused_residual_add(ctx, oracle):
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(5)
    Cin, Cout, H, Wi, B = 12, 20, 9, 13, 16
    Wc = sparse_matrix(rng, Cout, Cin * 9, .6)
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    Rs = rng.standard_normal((Cout, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1)), ocg(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1))
    conv = oracle.conv2d_pf(as_oracle(E), og, X, B, b)
    for act in ("none", "relu"):
        Y, Yrow, _ = rbm_conv(ctx, oracle, E, g, X, B, b, act, residual=Rs)
        want = oracle.act(oracle.add(conv, Rs), act)
        assert np.array_equal(Y, want) and np.array_equal(Yrow, want)


def test_conv_rbm_smaller_blocks_and_special_values(ctx, oracle):
    """Blocks of 4 rows; an infinity in the input must reach only the outputs whose taps touch it (padding
    slots multiply -0 into a spare register, never into an output); -0.0 results keep their sign."""
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(9)
    Cin, Cout, H, Wi, B = 8, 12, 8, 8, 16
    Wc = sparse_matrix(rng, Cout, Cin * 9, .7)
    E = datagen.encode_dense(Wc)
    g, og = hipabi.conv_geom(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1)), ocg(Cin, Cout, 3, 3, H, Wi, (1, 1), (1, 1))
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    X[2, 3, 4, :] = np.inf
    X[5] = -0.0
    Y, Yrow, R = rbm_conv(ctx, oracle, E, g, X, B, None, Ct_max=4)
    want = oracle.conv2d_rbm_pf(R, og, X, B, None)
    assert R.Ct_max == 4 and np.array_equal(Y, want, equal_nan=True) and np.array_equal(Yrow, want, equal_nan=True)
    assert np.array_equal(np.signbit(Y), np.signbit(want))
    assert np.isfinite(Y).any() and not np.isfinite(Y).all()


def test_rbm_upload_validation(ctx, oracle):
    rng = np.random.default_rng(3)
    E = datagen.encode_dense(sparse_matrix(rng, 20, 36, .6))
    R = oracle.rbm_build(as_oracle(E), 8)
    args = dict(block_union=R.block_union, krel=R.krel, colptr=R.colptr, pair_row=R.pair_row, pair_w=R.pair_w)

    def upload(**change):
        a = {k: v.copy() for k, v in args.items()}
        for k, fn in change.items():
            fn(a[k])
        return ctx.upload_rbm(R.M, R.N, R.Ct_max, **a)

    ctx.rbm_free(upload())
    def set_(i, v):
        return lambda arr: arr.__setitem__(i, v)
    for change in (dict(krel=set_(0, 36)), dict(krel=set_(1, int(R.krel[0]))), dict(pair_row=set_(0, 8)),
                   dict(colptr=set_(1, 0)), dict(block_union=set_(1, int(R.block_union[2]) + 1))):
        with pytest.raises(hipabi.SoError) as e:
            upload(**change)
        assert e.value.status == hipabi.SO_ERR_BOUNDS
    with pytest.raises(hipabi.SoError) as e:                          # 20 rows in blocks of 8 are 3 blocks
        ctx.upload_rbm(R.M, R.N, 4, **args)
    assert e.value.status == hipabi.SO_ERR_INVALID
    # a format that does not describe the plan's weights, or has blocks larger than the kernel holds
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
    plan = ctx.conv_plan(dE, hipabi.conv_geom(4, 20, 3, 3, 8, 8, (1, 1), (1, 1)))
    E2 = datagen.encode_dense(sparse_matrix(rng, 24, 36, .6))
    R2 = oracle.rbm_build(as_oracle(E2), 8)
    other = ctx.upload_rbm(R2.M, R2.N, 8, R2.block_union, R2.krel, R2.colptr, R2.pair_row, R2.pair_w)
    R16 = oracle.rbm_build(as_oracle(E), 16)
    big = ctx.upload_rbm(R16.M, R16.N, 16, R16.block_union, R16.krel, R16.colptr, R16.pair_row, R16.pair_w)
    for bad in (other, big):
        with pytest.raises(hipabi.SoError) as e:
            ctx.conv_plan_set_rbm(plan, bad)
        assert e.value.status == hipabi.SO_ERR_INVALID
    ctx.conv_plan_free(plan)
    ctx.rbm_free(other)
    ctx.rbm_free(big)
    dE.free()
