"""Pins the oracle's kernels (oracle.c) against what fixes them independently:
fp64 closed forms, brute force on small inputs, library routines (torch conv2d /
max_pool2d on the CPU), special cases, the compiled reference (bit for bit) and the
committed reference vectors."""
import numpy as np
import pytest

from conftest import rel_err, sparse_matrix

MATMUL_CASES = [(16, 32, 1, .3), (16, 32, 10, .3), (16, 32, 100, .3), (64, 128, 10, .5), (128, 256, 20, .7),
                (256, 512, 10, .9), (1, 1, 1, 0.), (1, 1000, 1, .1), (1000, 1, 1, .1), (0, 0, 0, 0.),
                (32, 32, 1, 1.), (10, 10, 1, 0.), (10, 10, 10, .5), (10, 10, 10, .9), (20, 20, 10, .2),
                (100, 100, 10, .2), (1000, 1000, 10, .1), (500, 500, 10, .05), (300, 300, 64, .4), (200, 200, 256, .9)]


@pytest.mark.parametrize("m,n,C,sp", MATMUL_CASES)
def test_matmul_closed_form(oracle, m, n, C, sp):
    rng = np.random.default_rng(m * 31 + n * 7 + C)
    W = sparse_matrix(rng, m, n, sp)
    X = rng.standard_normal((n, C)).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = oracle.encode(W)
    Y = oracle.matmul(E, X, b)
    assert Y.shape == (m, C)
    Y64 = W.astype(np.float64) @ X.astype(np.float64) + b.astype(np.float64)[:, None]
    assert rel_err(Y, Y64) <= 1e-5
    assert np.array_equal(Y, oracle.matmul(E, X, b, scalar=True))       # tiling changes no bit
    Y0 = oracle.matmul(E, X, None)
    assert rel_err(Y0, W.astype(np.float64) @ X) <= 1e-5


def test_matmul_special_cases(oracle):
    rng = np.random.default_rng(5)
    X = rng.standard_normal((40, 33)).astype(np.float32)
    b = rng.standard_normal(40).astype(np.float32)
    # identity matrix: Y = fma(1, x, b) = x + b exactly
    assert np.array_equal(oracle.matmul(oracle.encode(np.eye(40, dtype=np.float32)), X, b), X + b[:, None])
    # a row permutation picks rows of X exactly
    perm = rng.permutation(40)
    P = np.zeros((40, 40), np.float32)
    P[np.arange(40), perm] = 1
    assert np.array_equal(oracle.matmul(oracle.encode(P), X, None), X[perm])
    # all-zero matrix: bias only
    assert np.array_equal(oracle.matmul(oracle.encode(np.zeros((40, 40), np.float32)), X, b),
                          np.repeat(b[:, None], 33, axis=1))
    # accumulation order is ascending column: catastrophic-cancellation probe
    W = np.array([[1e8, 1.0, -1e8]], np.float32)
    Xo = np.ones((3, 1), np.float32)
    assert oracle.matmul(oracle.encode(W), Xo, None)[0, 0] == 0.0       # (1e8 + 1) - 1e8 in fp32
    W = np.array([[1e8, -1e8, 1.0]], np.float32)
    assert oracle.matmul(oracle.encode(W), Xo, None)[0, 0] == 1.0


def test_matmul_activations(oracle):
    rng = np.random.default_rng(6)
    W = sparse_matrix(rng, 50, 60, .7)
    X = rng.standard_normal((60, 20)).astype(np.float32)
    b = rng.standard_normal(50).astype(np.float32)
    E = oracle.encode(W)
    Y = oracle.matmul(E, X, b).astype(np.float64)
    assert np.array_equal(oracle.matmul(E, X, b, "relu"), np.maximum(Y, 0).astype(np.float32))
    assert rel_err(oracle.matmul(E, X, b, "sigmoid"), 1 / (1 + np.exp(-Y))) <= 1e-6
    assert rel_err(oracle.matmul(E, X, b, "tanh"), np.tanh(Y)) <= 1e-6
    for act in ("relu", "sigmoid", "tanh"):                     # fused == matmul then the separate layer
        assert np.array_equal(oracle.matmul(E, X, b, act), oracle.act(oracle.matmul(E, X, b), act))


def test_matmul_bit_exact_vs_compiled_reference(oracle, ref):
    rng = np.random.default_rng(8)
    for (m, n, C, sp) in [(300, 257, 1, .9), (300, 257, 10, .9), (300, 257, 64, .9), (300, 257, 100, .9),
                          (128, 512, 256, .5), (1000, 1000, 48, .95)]:
        W = sparse_matrix(rng, m, n, sp)
        X = rng.standard_normal((n, C)).astype(np.float32)
        b = rng.standard_normal(m).astype(np.float32)
        E, h = oracle.encode(W), ref.encode(W)
        assert np.array_equal(oracle.matmul(E, X, b), ref.matmul(h, X, b))
        assert np.array_equal(oracle.matmul(E, X, None), ref.matmul(h, X, None))
        for mask in ([True, False] if C % 16 == 0 else [True]):
            assert np.array_equal(oracle.matmul(E, X, b, "relu"), ref.matmul_fused(h, X, b, mask, True))


def test_matmul_vs_reference_vectors(oracle, golden):
    E = oracle.encode(golden["enc_W"])
    b = golden["mm_bias"]
    for C in (1, 10, 16, 64, 100, 128, 256):
        X = golden["mm_X_%d" % C]
        assert np.array_equal(oracle.matmul(E, X, b), golden["mm_Y_%d" % C])
        assert np.array_equal(oracle.matmul(E, X, b, "relu"), golden["mm_Yrelu_%d" % C])
    assert np.array_equal(oracle.matmul(E, golden["mm_X_64"], None), golden["mm_Ynobias_64"])


MATVEC_CASES = [(16, 32, .3), (64, 128, .5), (128, 256, .7), (256, 512, .9), (1, 1, 0.), (1, 1000, .1),
                (1000, 1, .1), (0, 0, 0.), (32, 32, 1.), (10, 10, 0.), (10, 10, .5), (10, 10, .9), (20, 20, .2),
                (100, 100, .2), (1000, 1000, .1), (500, 500, .05), (2000, 2000, .3), (3000, 3000, .4)]


@pytest.mark.parametrize("m,n,sp", MATVEC_CASES)
def test_matvec_closed_form(oracle, m, n, sp):
    rng = np.random.default_rng(m * 13 + n)
    W = sparse_matrix(rng, m, n, sp)
    x = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    y = oracle.matvec(oracle.encode(W), x, b)
    assert y.shape == (m,)
    assert rel_err(y, W.astype(np.float64) @ x + b) <= 1e-5
    assert rel_err(oracle.matvec(oracle.encode(W), x, None), W.astype(np.float64) @ x) <= 1e-5


def test_matvec_bit_exact_vs_compiled_reference(oracle, ref, golden):
    rng = np.random.default_rng(9)
    for (m, n, sp) in [(300, 257, .9), (64, 1000, .3), (1000, 17, .5), (513, 513, .97)]:
        W = sparse_matrix(rng, m, n, sp)
        x = rng.standard_normal(n).astype(np.float32)
        b = rng.standard_normal(m).astype(np.float32)
        assert np.array_equal(oracle.matvec(oracle.encode(W), x, b), ref.matvec(ref.encode(W), x, b))
    E = oracle.encode(golden["enc_W"])
    assert np.array_equal(oracle.matvec(E, golden["mv_x"], golden["mm_bias"]), golden["mv_y"])
    assert np.array_equal(oracle.matvec(E, golden["mv_x"], None), golden["mv_ynobias"])


def test_activations(oracle, golden):
    v = golden["act_x"]
    v64 = v.astype(np.float64)
    assert np.array_equal(oracle.act(v, "relu"), np.maximum(v, 0))
    assert rel_err(oracle.act(v, "sigmoid"), 1 / (1 + np.exp(-v64))) <= 1e-6
    assert rel_err(oracle.act(v, "tanh"), np.tanh(v64)) <= 1e-6
    for a in ("relu", "sigmoid", "tanh"):                       # reference's in-place kernels, same libm
        assert np.array_equal(oracle.act(v, a), golden["act_" + a])
    assert oracle.act(np.array([-0.0, 0.0, -1.0], np.float32), "relu").tolist() == [0.0, 0.0, 0.0]


# ------------------------------------------------------------------ conv

def brute_conv(W4, X, bias, stride, pad, dil):
    """7-loop definition on [C][H][W][B] tensors, fp64."""
    Cout, Cin, kH, kW = W4.shape
    _, H, Wi, B = X.shape
    Ho = (H + 2 * pad[0] - (dil[0] * (kH - 1) + 1)) // stride[0] + 1
    Wo = (Wi + 2 * pad[1] - (dil[1] * (kW - 1) + 1)) // stride[1] + 1
    Y = np.zeros((Cout, Ho, Wo, B))
    for co in range(Cout):
        for ho in range(Ho):
            for wo in range(Wo):
                acc = np.full(B, float(bias[co]))
                for ci in range(Cin):
                    for kh in range(kH):
                        for kw in range(kW):
                            hi, wi = ho * stride[0] - pad[0] + kh * dil[0], wo * stride[1] - pad[1] + kw * dil[1]
                            if 0 <= hi < H and 0 <= wi < Wi:
                                acc += float(W4[co, ci, kh, kw]) * X[ci, hi, wi].astype(np.float64)
                Y[co, ho, wo] = acc
    return Y


CONV_CASES = [(3, 4, 6, 7, 2, (3, 3), (1, 1), (1, 1), (1, 1)), (3, 4, 6, 7, 2, (3, 3), (2, 2), (1, 1), (1, 1)),
              (4, 5, 6, 6, 3, (1, 1), (2, 2), (0, 0), (1, 1)), (2, 3, 8, 8, 2, (3, 2), (1, 2), (2, 0), (2, 1)),
              (2, 2, 5, 5, 1, (5, 5), (1, 1), (2, 2), (1, 1))]


@pytest.mark.parametrize("Cin,Cout,H,Wi,B,k,s,p,d", CONV_CASES)
def test_conv_brute_force_and_torch(oracle, Cin, Cout, H, Wi, B, k, s, p, d):
    import torch
    from oracle import conv_geom
    rng = np.random.default_rng(Cin * 100 + H)
    W4 = rng.standard_normal((Cout, Cin, k[0], k[1])).astype(np.float32)
    W4[rng.random(W4.shape) < 0.5] = 0
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    g = conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
    E = oracle.encode(W4.reshape(Cout, -1))
    Y = oracle.conv2d_pf(E, g, X, B, b)
    assert rel_err(Y, brute_conv(W4, X, b, s, p, d)) <= 1e-5
    Yt = torch.nn.functional.conv2d(torch.from_numpy(X.transpose(3, 0, 1, 2).copy()).double(),
                                    torch.from_numpy(W4).double(), torch.from_numpy(b).double(),
                                    stride=s, padding=p, dilation=d).numpy().transpose(1, 2, 3, 0)
    assert rel_err(Y, Yt) <= 1e-5
    assert np.array_equal(oracle.conv2d_pf(E, g, X, B, b, "relu"), np.maximum(Y, 0))


def test_conv_special_cases(oracle):
    from oracle import conv_geom
    rng = np.random.default_rng(12)
    Cin, Cout, H, Wi, B = 6, 5, 7, 9, 4
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    # 1x1 stride-1 conv is ellpack_matmul on the [Cin x (H*W*B)] matrix, bit for bit
    W = sparse_matrix(rng, Cout, Cin, .4)
    E = oracle.encode(W)
    Y = oracle.conv2d_pf(E, conv_geom(Cin, Cout, 1, 1, H, Wi), X, B, b)
    assert np.array_equal(Y.reshape(Cout, -1), oracle.matmul(E, X.reshape(Cin, -1), b))
    # a delta kernel (centre tap of a padded 3x3) is the identity; an off-centre tap is a shift
    for (kh, kw) in [(1, 1), (0, 2)]:
        W4 = np.zeros((Cin, Cin, 3, 3), np.float32)
        W4[np.arange(Cin), np.arange(Cin), kh, kw] = 1
        Y = oracle.conv2d_pf(oracle.encode(W4.reshape(Cin, -1)), conv_geom(Cin, Cin, 3, 3, H, Wi, pad=(1, 1)), X, B, None)
        S = np.zeros_like(X)
        dh, dw = kh - 1, kw - 1
        hs, ws = slice(max(0, -dh), H - max(0, dh)), slice(max(0, -dw), Wi - max(0, dw))
        hd, wd = slice(max(0, dh), H - max(0, -dh)), slice(max(0, dw), Wi - max(0, -dw))
        S[:, hs, ws] = X[:, hd, wd]
        assert np.array_equal(Y, S)


def test_conv_vs_compiled_reference_and_vectors(oracle, golden):
    from oracle import Ref, conv_geom
    for i, c in enumerate(golden["conv_cases"]):
        Cin, Cout, H, Wi, B = (int(v) for v in c[:5])
        k, s, p, d = tuple(c[5:7]), tuple(c[7:9]), tuple(c[9:11]), tuple(c[11:13])
        g = conv_geom(Cin, Cout, int(k[0]), int(k[1]), H, Wi, tuple(map(int, s)), tuple(map(int, p)), tuple(map(int, d)))
        Wc, X, b = golden["conv%d_W" % i], golden["conv%d_X" % i], golden["conv%d_b" % i]
        E = oracle.encode(Wc)
        assert np.array_equal(oracle.conv2d_pf(E, g, X, B, b), golden["conv%d_Y" % i])
        assert np.array_equal(oracle.conv2d_pf(E, g, X, B, b, "relu"), golden["conv%d_Yrelu" % i])
        if "conv%d_Ypf" % i in golden.files:        # the variant applyConv runs, where its stride code is right
            assert np.array_equal(oracle.conv2d_pf(E, g, X, B, b), golden["conv%d_Ypf" % i])
        if Ref.available():
            r = Ref()
            XF = np.ascontiguousarray(X.transpose(2, 1, 0, 3))
            Y = r.conv(Wc, g, XF.ravel(), B, b, False, 3).reshape(g.W_out, g.H_out, Cout, B).transpose(2, 1, 0, 3)
            assert np.array_equal(oracle.conv2d_pf(E, g, X, B, b), Y)


# ------------------------------------------------------- pool / gap / add

@pytest.mark.parametrize("C,H,Wi,B,k,s,p", [(3, 8, 8, 2, (2, 2), (2, 2), (0, 0)), (4, 9, 7, 3, (3, 3), (2, 2), (1, 1)),
                                           (2, 5, 6, 1, (3, 2), (1, 1), (1, 0)), (64, 12, 12, 4, (3, 3), (2, 2), (1, 1))])
def test_maxpool(oracle, C, H, Wi, B, k, s, p):
    import torch
    rng = np.random.default_rng(C + H)
    X = rng.standard_normal((C, H, Wi, B)).astype(np.float32)
    Y = oracle.maxpool_pf(X, C, H, Wi, B, k, s, p)
    Yt = torch.nn.functional.max_pool2d(torch.from_numpy(X.transpose(3, 0, 1, 2).copy()), k, s, p).numpy().transpose(1, 2, 3, 0)
    assert np.array_equal(Y, Yt)
    Ho, Wo = Y.shape[1:3]
    Yb = np.full(Y.shape, -np.inf, np.float32)
    for ho in range(Ho):
        for wo in range(Wo):
            for kh in range(k[0]):
                for kw in range(k[1]):
                    hi, wi = ho * s[0] - p[0] + kh, wo * s[1] - p[1] + kw
                    if 0 <= hi < H and 0 <= wi < Wi:
                        Yb[:, ho, wo] = np.maximum(Yb[:, ho, wo], X[:, hi, wi])
    assert np.array_equal(Y, Yb)


def test_gap_and_add(oracle):
    rng = np.random.default_rng(3)
    C, H, Wi, B = 5, 7, 6, 3
    X = rng.standard_normal((C, H, Wi, B)).astype(np.float32)
    Y = oracle.gap_pf(X, C, H, Wi, B)
    assert rel_err(Y, X.astype(np.float64).mean(axis=(1, 2))) <= 1e-6
    s = np.zeros((C, B), np.float32)                   # explicit (h, w)-ordered fp32 sum times reciprocal
    for h in range(H):
        for w in range(Wi):
            s = s + X[:, h, w]
    assert np.array_equal(Y, s * np.float32(1.0 / (H * Wi)))
    A = rng.standard_normal(1000).astype(np.float32)
    Bv = rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(oracle.add(A, Bv), A + Bv)
