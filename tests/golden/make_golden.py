"""Writes tests/golden/ref_vectors.npz: inputs and the outputs the REFERENCE's own
compiled kernels (oracle/_ref, built from the reference sources by oracle/Makefile)
produce for them.  Run in the build container, where the reference tree exists:

    make -C oracle && python tests/golden/make_golden.py

The fixture is data only (seeded inputs + expected outputs); it lets the oracle and
the HIP kernels be checked against the reference on machines where the reference
cannot be built.  Loaded with numpy.load(allow_pickle=False).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", "..", "oracle"))
from oracle import Ref, conv_geom  # noqa: E402


def main():
    ref = Ref()
    rng = np.random.default_rng(20240607)
    out = {}

    # encoder + matmul + matvec on one rectangular matrix with an empty row, a
    # full row, a -0.0 and a NaN entry
    W = rng.standard_normal((37, 53)).astype(np.float32)
    W[rng.random(W.shape) < 0.8] = 0.0
    W[5, :] = 0.0
    W[9, :] = rng.standard_normal(53).astype(np.float32) + 3.0
    W[11, 7] = -0.0
    h = ref.encode(W)
    E = ref.arrays(h)
    out.update(enc_W=W, enc_Wd=E.Wd, enc_idx=E.idx, enc_nnz=E.nnz, enc_decoded=ref.decode(h))

    Wn = W.copy()
    Wn[3, 4] = np.nan
    En = ref.arrays(ref.encode(Wn))
    out.update(encnan_W=Wn, encnan_Wd=En.Wd, encnan_idx=En.idx, encnan_nnz=En.nnz)

    bias = (rng.standard_normal(37) * 0.1).astype(np.float32)
    for C in (1, 10, 16, 64, 100, 128, 256):
        X = rng.standard_normal((53, C)).astype(np.float32)
        out["mm_X_%d" % C] = X
        out["mm_Y_%d" % C] = ref.matmul(h, X, bias)
        out["mm_Yrelu_%d" % C] = ref.matmul_fused(h, X, bias, use_mask=(C % 16 != 0), fuse_relu=True)
    out["mm_bias"] = bias
    out["mm_Ynobias_64"] = ref.matmul(h, out["mm_X_64"], None)

    x = rng.standard_normal(53).astype(np.float32)
    out.update(mv_x=x, mv_y=ref.matvec(h, x, bias), mv_ynobias=ref.matvec(h, x, None))

    v = (rng.standard_normal(4096) * 4).astype(np.float32)
    out.update(act_x=v, act_relu=ref.act_inplace(v, "relu"), act_sigmoid=ref.act_inplace(v, "sigmoid"),
               act_tanh=ref.act_inplace(v, "tanh"))

    # conv: reference variant 3 (RBM implicit, correct for every geometry) on the
    # Fortran (B,C,H,W) layout, re-laid out here as [C][H][W][B]; variant 0
    # (patch-major tiled, what applyConv runs) where its stride handling is
    # right (stride_w == 1)
    cases = [(5, 7, 9, 11, 3, (3, 3), (1, 1), (1, 1), (1, 1)),
             (5, 7, 9, 11, 3, (3, 3), (2, 2), (1, 1), (1, 1)),
             (4, 6, 8, 8, 16, (1, 1), (2, 2), (0, 0), (1, 1)),
             (3, 4, 10, 10, 5, (3, 2), (1, 2), (2, 0), (2, 1)),
             (6, 40, 7, 7, 17, (3, 3), (1, 1), (1, 1), (1, 1))]
    out["conv_cases"] = np.array([[c[0], c[1], c[2], c[3], c[4], *c[5], *c[6], *c[7], *c[8]] for c in cases], dtype=np.int64)
    for i, (Cin, Cout, H, Wi, B, k, s, p, d) in enumerate(cases):
        g = conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
        Wc = rng.standard_normal((Cout, Cin * k[0] * k[1])).astype(np.float32)
        Wc[rng.random(Wc.shape) < 0.6] = 0.0
        X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
        cb = rng.standard_normal(Cout).astype(np.float32)
        XF = np.ascontiguousarray(X.transpose(2, 1, 0, 3))
        for relu in (False, True):
            Y = ref.conv(Wc, g, XF.ravel(), B, cb, relu, 3).reshape(g.W_out, g.H_out, Cout, B).transpose(2, 1, 0, 3)
            out["conv%d_Y%s" % (i, "relu" if relu else "")] = np.ascontiguousarray(Y)
        if s[1] == 1:
            out["conv%d_Ypf" % i] = ref.conv(Wc, g, X.ravel(), B, cb, False, 0).reshape(Cout, g.H_out, g.W_out, B)
        out["conv%d_W" % i], out["conv%d_X" % i], out["conv%d_b" % i] = Wc, X, cb

    # row-block-merged format: the reference's build_rbm_from_ellpack on the first matrix (blocks of
    # 8 rows and of 4), flattened as oracle.RbmArrays; and its RBM convolution (variant 3) on shapes
    # whose batch suits this build's RBM kernel (multiples of 16, enough nonzeros per channel)
    for ct in (8, 4):
        R = ref.rbm_build(h, ct)
        for key in ("block_union", "krel", "colptr", "pair_row", "pair_w"):
            out["rbm%d_%s" % (ct, key)] = getattr(R, key)
    rcases = [(16, 32, 12, 12, 16, (3, 3), (1, 1), (1, 1), (1, 1)),
              (8, 24, 10, 10, 32, (3, 3), (2, 2), (1, 1), (1, 1)),
              (32, 20, 6, 6, 16, (1, 1), (1, 1), (0, 0), (1, 1))]
    out["rbmconv_cases"] = np.array([[c[0], c[1], c[2], c[3], c[4], *c[5], *c[6], *c[7], *c[8]] for c in rcases], dtype=np.int64)
    for i, (Cin, Cout, H, Wi, B, k, s, p, d) in enumerate(rcases):
        g = conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
        Wc = rng.standard_normal((Cout, Cin * k[0] * k[1])).astype(np.float32)
        Wc[rng.random(Wc.shape) < 0.75] = 0.0
        X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
        cb = rng.standard_normal(Cout).astype(np.float32)
        XF = np.ascontiguousarray(X.transpose(2, 1, 0, 3))
        for relu in (False, True):
            Y = ref.conv(Wc, g, XF.ravel(), B, cb, relu, 3).reshape(g.W_out, g.H_out, Cout, B).transpose(2, 1, 0, 3)
            out["rbmconv%d_Y%s" % (i, "relu" if relu else "")] = np.ascontiguousarray(Y)
        out["rbmconv%d_W" % i], out["rbmconv%d_X" % i], out["rbmconv%d_b" % i] = Wc, X, cb

    path = os.path.join(HERE, "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
