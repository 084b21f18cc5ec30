"""Pins the oracle's restatement of the row-block-merged (RBM) format and kernel
(src/layers/rbm_conv.cpp:7-73, src/layers/conv_kernels.cpp:66-147): a hand-written known answer,
an independent numpy construction, the decode invariant, the reference's own build_rbm_from_ellpack
(live where oracle/_ref runs, and through tests/golden/ref_vectors.npz everywhere), and for the kernel
the per-row oracle, the reference's conv2d_rbm_fmajor_implicit outputs and the 1x1 == matmul identity."""
import numpy as np
import pytest

from conftest import sparse_matrix
from oracle import RbmArrays, conv_geom


def test_rbm_build_known_answer(oracle):
    """Worked by hand: rows 0,1 share column 3; blocks of two rows."""
    W = np.array([[1, 0, 0, 2], [0, 3, 0, 6], [0, 0, 4, 0], [0, 0, 0, 5]], dtype=np.float32)
    R = oracle.rbm_build(oracle.encode(W), 2)
    assert R.nblocks == 2
    assert R.block_union.tolist() == [0, 3, 5]
    assert R.krel.tolist() == [0, 1, 3, 2, 3]
    assert R.colptr.tolist() == [0, 1, 2, 4, 5, 6]
    assert R.pair_row.tolist() == [0, 1, 0, 1, 0, 1]
    assert R.pair_w.tolist() == [1, 3, 2, 6, 4, 5]
    # one block for the whole matrix: column 3 is shared by rows 0, 1 and 3
    R = oracle.rbm_build(oracle.encode(W), 8)
    assert R.block_union.tolist() == [0, 4] and R.krel.tolist() == [0, 1, 2, 3]
    assert R.colptr.tolist() == [0, 1, 2, 3, 6] and R.pair_row.tolist() == [0, 1, 2, 0, 1, 3]
    assert R.pair_w.tolist() == [1, 3, 4, 2, 6, 5]


def numpy_rbm(W, Ct_max):
    """Independent construction straight from the dense matrix: per block, the nonzeros in
    column-major order are exactly the (column, row)-sorted triples."""
    m, n = W.shape
    bu, krel, colptr, prow, pw = [0], [], [0], [], []
    for M0 in range(0, m, Ct_max):
        blk = W[M0:M0 + Ct_max]
        cols, rows = np.nonzero(blk.T)                    # ascending column, then ascending row
        for k in np.unique(cols):
            sel = cols == k
            krel.append(int(k))
            prow += rows[sel].tolist()
            pw += blk[rows[sel], k].tolist()
            colptr.append(len(prow))
        bu.append(len(krel))
    return RbmArrays(m, n, Ct_max, bu, krel, colptr, prow, np.array(pw, dtype=np.float32))


def decode_rbm(R):
    W = np.zeros((R.M, R.N), dtype=np.float32)
    for b in range(R.nblocks):
        for u in range(int(R.block_union[b]), int(R.block_union[b + 1])):
            for p in range(int(R.colptr[u]), int(R.colptr[u + 1])):
                W[b * R.Ct_max + int(R.pair_row[p]), int(R.krel[u])] = R.pair_w[p]
    return W


@pytest.mark.parametrize("m,n,sp,ct", [(37, 53, .8, 8), (37, 53, .8, 4), (16, 32, .5, 8), (9, 100, .9, 8), (64, 64, 0., 8),
                                       (20, 20, 1., 8), (1, 7, .3, 8), (50, 30, .7, 16), (33, 40, .6, 1)])
def test_rbm_build_against_numpy_and_decode(oracle, m, n, sp, ct):
    rng = np.random.default_rng(m * 100 + n + ct)
    W = sparse_matrix(rng, m, n, sp)
    if m > 4:
        W[2] = 0                                          # an empty row inside a block
    E = oracle.encode(W)
    R = oracle.rbm_build(E, ct)
    assert R.same_as(numpy_rbm(W, ct))
    assert np.array_equal(decode_rbm(R), W)
    assert len(R.pair_w) == E.total_nnz and R.nblocks == (m + ct - 1) // ct
    # an all-zero block contributes no union column (src/layers/rbm_conv.cpp:32-37)
    W[:] = 0
    R0 = oracle.rbm_build(oracle.encode(W), ct)
    assert len(R0.krel) == 0 and R0.colptr.tolist() == [0] and not R0.block_union.any()


def test_rbm_build_against_the_reference(oracle, golden):
    E = oracle.encode(golden["enc_W"])
    for ct in (8, 4):
        want = RbmArrays(E.m, E.n, ct, *(golden["rbm%d_%s" % (ct, k)] for k in ("block_union", "krel", "colptr", "pair_row", "pair_w")))
        assert oracle.rbm_build(E, ct).same_as(want)


@pytest.mark.parametrize("m,n,sp,ct", [(37, 53, .8, 8), (64, 576, .8, 8), (100, 90, .5, 16), (21, 45, .7, 3)])
def test_rbm_build_against_the_compiled_reference(oracle, ref, m, n, sp, ct):
    rng = np.random.default_rng(m + n)
    W = sparse_matrix(rng, m, n, sp)
    assert oracle.rbm_build(oracle.encode(W), ct).same_as(ref.rbm_build(ref.encode(W), ct))


CONV = [(5, 7, 9, 11, 3, (3, 3), (1, 1), (1, 1), (1, 1)), (5, 21, 9, 11, 4, (3, 3), (2, 2), (1, 1), (1, 1)),
        (3, 4, 10, 10, 5, (3, 2), (1, 2), (2, 0), (2, 1)), (6, 40, 7, 7, 8, (3, 3), (1, 1), (1, 1), (1, 1)),
        (8, 16, 6, 6, 2, (1, 1), (2, 2), (0, 0), (1, 1))]


@pytest.mark.parametrize("Cin,Cout,H,Wi,B,k,s,p,d", CONV)
@pytest.mark.parametrize("ct", [8, 3])
def test_rbm_conv_has_the_per_row_kernels_bits(oracle, Cin, Cout, H, Wi, B, k, s, p, d, ct):
    """Walking the union columns in ascending order gives every row its products in ascending column
    order, which is the per-row kernel's order: identical bits, activations included."""
    rng = np.random.default_rng(Cin + Cout + ct)
    Wc = sparse_matrix(rng, Cout, Cin * k[0] * k[1], .6)
    E = oracle.encode(Wc)
    R = oracle.rbm_build(E, ct)
    g = conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
    X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    for act in ("none", "relu", "tanh"):
        assert np.array_equal(oracle.conv2d_rbm_pf(R, g, X, B, b, act), oracle.conv2d_pf(E, g, X, B, b, act))
    assert np.array_equal(oracle.conv2d_rbm_pf(R, g, X, B, None), oracle.conv2d_pf(E, g, X, B, None))


def test_rbm_conv_against_the_reference(oracle, golden):
    """Outputs of the reference's conv2d_rbm_fmajor_implicit (variant 3 of oracle/ref_driver.cpp)."""
    for prefix, cases in (("conv", golden["conv_cases"]), ("rbmconv", golden["rbmconv_cases"])):
        for i, c in enumerate(cases):
            Cin, Cout, H, Wi, B = (int(v) for v in c[:5])
            k, s, p, d = [tuple(int(v) for v in c[j:j + 2]) for j in (5, 7, 9, 11)]
            g = conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
            R = oracle.rbm_build(oracle.encode(golden["%s%d_W" % (prefix, i)]), 8)
            X, b = golden["%s%d_X" % (prefix, i)], golden["%s%d_b" % (prefix, i)]
            assert np.array_equal(oracle.conv2d_rbm_pf(R, g, X, B, b), golden["%s%d_Y" % (prefix, i)])
            assert np.array_equal(oracle.conv2d_rbm_pf(R, g, X, B, b, "relu"), golden["%s%d_Yrelu" % (prefix, i)])


def test_rbm_conv_1x1_is_matmul(oracle):
    rng = np.random.default_rng(4)
    W = sparse_matrix(rng, 19, 23, .5)
    E = oracle.encode(W)
    X = rng.standard_normal((23, 1, 1, 12)).astype(np.float32)
    b = rng.standard_normal(19).astype(np.float32)
    Y = oracle.conv2d_rbm_pf(oracle.rbm_build(E, 8), conv_geom(23, 19, 1, 1, 1, 1), X, 12, b)
    assert np.array_equal(Y.reshape(19, 12), oracle.matmul(E, X.reshape(23, 12), b))


def flatten_plan(P):
    """sparseops_backend.RBMPlan (the host layer's build_rbm_from_ellpack) -> RbmArrays."""
    bu, colptr, base = [0], [0], 0
    for b in P.blocks:
        colptr += [base + int(c) for c in b.colptr[1:]]
        base += len(b.pair_w)
        bu.append(bu[-1] + len(b.krel))
    cat = lambda key, dt: np.concatenate([getattr(b, key) for b in P.blocks]).astype(dt) if P.blocks else np.zeros(0, dt)
    return RbmArrays(P.M, P.N, P.Ct_max, bu, cat("krel", np.uint32), colptr, cat("pair_row", np.uint16), cat("pair_w", np.float32))


@pytest.mark.parametrize("m,n,sp,ct", [(37, 53, .8, 8), (64, 576, .8, 8), (21, 45, .7, 3), (50, 30, 0., 16), (5, 9, 1., 8)])
def test_host_builder_matches_the_oracle(oracle, backend, m, n, sp, ct):
    """build_rbm_from_ellpack of the shipped host layer (a k-way merge over the rows' ascending columns,
    no sort) produces the arrays of the restated reference builder, blocks and bias slices included."""
    rng = np.random.default_rng(m * n + ct)
    W = sparse_matrix(rng, m, n, sp)
    bias = rng.standard_normal(m).astype(np.float32)
    P = backend.build_rbm_from_ellpack(backend.convert_to_ellpack(W), bias, ct)
    assert (P.M, P.N, P.Ct_max) == (m, n, ct) and len(P.blocks) == (m + ct - 1) // ct
    assert flatten_plan(P).same_as(oracle.rbm_build(oracle.encode(W), ct))
    for i, b in enumerate(P.blocks):
        assert b.M0 == i * ct and b.Ct == min(ct, m - i * ct) and len(b.colptr) == len(b.krel) + 1
        assert np.array_equal(b.bias, bias[b.M0:b.M0 + b.Ct])
    assert all(len(b.bias) == 0 for b in backend.build_rbm_from_ellpack(backend.convert_to_ellpack(W)).blocks)
