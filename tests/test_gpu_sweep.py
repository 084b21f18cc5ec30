"""Seeded random sweep over shapes the hand-picked cases do not list: convolution geometry
(kernel, stride, dilation, padding, ragged tiles, any batch), matmul and matvec shapes, every
kernel variant the library can take for them, against the oracle (bit-exact for matmul and
convolution, 1e-5 relative for matvec)."""
import numpy as np
import pytest

from conftest import as_oracle

import datagen
import hipabi

pytestmark = pytest.mark.gpu


def _sparse(rng, m, n, sp):
    W = rng.standard_normal((m, n)).astype(np.float32)
    W[rng.random((m, n)) < sp] = 0
    return W


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_convolutions(ctx, oracle, seed):
    from oracle import conv_geom as ocg
    rng = np.random.default_rng(seed)
    for it in range(40):
        Cin, Cout = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        k = (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
        s = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        d = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        p = (int(rng.integers(0, 4)), int(rng.integers(0, 4)))
        H = int(rng.integers(d[0] * (k[0] - 1) + 1, 30))
        Wi = int(rng.integers(d[1] * (k[1] - 1) + 1, 30))
        B = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 20, 32, 48]))
        Wc = _sparse(rng, Cout, Cin * k[0] * k[1], float(rng.choice([0.0, 0.3, 0.6, 0.9, 0.98])))
        if Cout > 2:
            Wc[int(rng.integers(0, Cout))] = 0
        X = rng.standard_normal((Cin, H, Wi, B)).astype(np.float32)
        b = rng.standard_normal(Cout).astype(np.float32) if rng.random() < 0.7 else None
        act = str(rng.choice(["none", "relu"]))
        case = "seed %d case %d: Cin=%d Cout=%d k=%s s=%s d=%s p=%s H=%d W=%d B=%d act=%s" % (seed, it, Cin, Cout, k, s, d, p, H, Wi, B, act)
        E = datagen.encode_dense(Wc)
        g, og = hipabi.conv_geom(Cin, Cout, k[0], k[1], H, Wi, s, p, d), ocg(Cin, Cout, k[0], k[1], H, Wi, s, p, d)
        want = oracle.conv2d_pf(as_oracle(E), og, X, B, b, act)
        dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r)
        plan = ctx.conv_plan(dE, g)
        dX, dY = ctx.array(X), ctx.empty((Cout, g.H_out, g.W_out, B))
        dB = ctx.array(b) if b is not None else None
        for window in (None, "0", "1"):
            if window == "1" and (ctx.conv_plan_window(plan) is None or B % 4):
                continue
            with ctx.tuning(SPARSEOPS_CONV_WINDOW=window):
                dY.upload(np.full((Cout, g.H_out, g.W_out, B), np.nan, np.float32))
                ctx.conv2d(plan, dX, B, dB, dY, act)
                assert np.array_equal(dY.download(), want), "%s window=%s" % (case, window)
        ctx.conv_plan_free(plan)
        dE.free()
        for a in (dX, dY, dB):
            if a is not None:
                a.free()


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_products(ctx, oracle, seed):
    rng = np.random.default_rng(seed)
    every = hipabi.LAYOUT_ROW | hipabi.LAYOUT_SLOT | hipabi.LAYOUT_BINS | hipabi.LAYOUT_TILED
    for it in range(40):
        m, n = int(rng.integers(1, 400)), int(rng.integers(1, 700))
        C = int(rng.choice([1, 3, 4, 16, 20, 64, 68, 100, 128, 256, 260]))
        W = _sparse(rng, m, n, float(rng.choice([0.0, 0.5, 0.9, 0.99])))
        if m > 3:
            W[2] = 0
        E = datagen.encode_dense(W)
        X = rng.standard_normal((n, C)).astype(np.float32)
        b = rng.standard_normal(m).astype(np.float32) if rng.random() < 0.7 else None
        act = str(rng.choice(["none", "relu"]))
        case = "seed %d case %d: m=%d n=%d C=%d act=%s" % (seed, it, m, n, C, act)
        want = oracle.matmul(as_oracle(E), X, b, act)
        dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, every)
        dX, dY = ctx.array(X), ctx.empty((m, C))
        dB = ctx.array(b) if b is not None else None
        for tiled in ("0", "1"):
            with ctx.tuning(SPARSEOPS_MATMUL_TILED=tiled):
                dY.upload(np.full((m, C), np.nan, np.float32))
                ctx.matmul(dE, dX, C, dB, dY, act)
                assert np.array_equal(dY.download(), want), "%s tiled=%s" % (case, tiled)
        x = rng.standard_normal(n).astype(np.float32)
        dx, dy = ctx.array(x), ctx.empty((m,))
        y64 = W.astype(np.float64) @ x + (b if b is not None else 0)
        for layout in (hipabi.LAYOUT_ROW, hipabi.LAYOUT_SLOT, hipabi.LAYOUT_BINS, 0):
            for lanes in ((None, 8, 16, 32, 64) if layout == hipabi.LAYOUT_ROW else (None,)):
                with ctx.tuning(SPARSEOPS_MATVEC_LANES=lanes):
                    dy.upload(np.full(m, np.nan, np.float32))
                    ctx.matvec(dE, dx, dB, dy, layout)
                    err = np.abs(dy.download() - y64).max() / max(np.abs(y64).max(), 1e-30)
                assert err <= 1e-5, "%s matvec layout=%d lanes=%s err=%g" % (case, layout, lanes, err)
        dE.free()
        for a in (dX, dY, dB, dx, dy):
            if a is not None:
                a.free()


@pytest.mark.parametrize("seed", [31, 32])
def test_random_pool_add_transpose(ctx, oracle, seed):
    rng = np.random.default_rng(seed)
    for it in range(40):
        C, H, Wi = int(rng.integers(1, 20)), int(rng.integers(1, 25)), int(rng.integers(1, 25))
        B = int(rng.choice([1, 2, 3, 4, 6, 8, 16, 20, 32]))
        k = (int(rng.integers(1, min(H, 4) + 1)), int(rng.integers(1, min(Wi, 4) + 1)))
        s = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        pad = (int(rng.integers(0, k[0])), int(rng.integers(0, k[1])))       # a window always meets the image
        X = rng.standard_normal((C, H, Wi, B)).astype(np.float32)
        case = "seed %d case %d: C=%d H=%d W=%d B=%d k=%s s=%s pad=%s" % (seed, it, C, H, Wi, B, k, s, pad)
        want = oracle.maxpool_pf(X, C, H, Wi, B, k, s, pad)
        dX, dY = ctx.array(X), ctx.empty(want.shape)
        ctx.maxpool(C, H, Wi, k, s, pad, dX, B, dY)
        assert np.array_equal(dY.download(), want), case
        dG = ctx.empty((C, B))
        ctx.gap(C, H, Wi, dX, B, dG)
        assert np.array_equal(dG.download(), oracle.gap_pf(X, C, H, Wi, B)), case
        R = rng.standard_normal(X.shape).astype(np.float32)
        dR, dS = ctx.array(R), ctx.empty(X.shape)
        ctx.add(dX, dR, X.size, dS)
        assert np.array_equal(dS.download(), oracle.add(X, R)), case
        ctx.act("relu", dS, X.size, dS)
        assert np.array_equal(dS.download(), oracle.act(oracle.add(X, R), "relu")), case
        rows, cols = C * H, Wi * B
        dT = ctx.empty((cols, rows))
        ctx.transpose(dX, rows, cols, dT)
        assert np.array_equal(dT.download(), X.reshape(rows, cols).T), case
        # rows of `cols` floats into rows `stride` apart, the tail of every row zeroed, and back
        stride = cols + int(rng.integers(0, 5))
        dP = ctx.array(np.full((rows, stride), np.nan, np.float32))
        ctx.copy_rows(dX, cols, rows, cols, dP, stride, zero_fill=True)
        P = dP.download()
        assert np.array_equal(P[:, :cols], X.reshape(rows, cols)) and not P[:, cols:].any(), case
        dQ = ctx.array(np.full((rows, cols), np.nan, np.float32))
        ctx.copy_rows(dP, stride, rows, cols, dQ, cols)
        assert np.array_equal(dQ.download(), X.reshape(rows, cols)), case
        for a in (dX, dY, dG, dR, dS, dT, dP, dQ):
            a.free()


def _random_cnn(rng, B):
    """A random graph of the operators the loader supports with exact arithmetic: Conv (bias or not,
    random kernel/stride/padding) + optional Relu, MaxPool, residual blocks (Conv-Relu-Conv + skip,
    the skip either the block's input or a 1x1 projection, Add, optional Relu), then
    GlobalAveragePool or Flatten and a Gemm head."""
    import onnx_wire as ow
    nodes, inits = [], []
    C, H, W = int(rng.integers(1, 5)), int(rng.integers(9, 21)), int(rng.integers(9, 21))
    shape_in = (B, C, H, W)
    cur, uid = "input", [0]

    def name(prefix):
        uid[0] += 1
        return "%s%d" % (prefix, uid[0])

    def conv(src, cin, cout, k, s, p, relu):
        nonlocal H, W
        w = rng.standard_normal((cout, cin, k, k)).astype(np.float32) * np.float32(0.3)
        w[rng.random(w.shape) < 0.6] = 0
        wn, out = name("w"), name("conv")
        inits.append((wn, w))
        ins = [src, wn]
        if rng.random() < 0.6:
            bn = name("b")
            inits.append((bn, rng.standard_normal(cout).astype(np.float32)))
            ins.append(bn)
        nodes.append(ow.node("Conv", ins, [out], kernel_shape=[k, k], strides=[s, s], pads=[p, p, p, p], dilations=[1, 1], group=1))
        Ho, Wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
        if relu:
            r = name("relu")
            nodes.append(ow.node("Relu", [out], [r]))
            out = r
        return out, Ho, Wo

    for _ in range(int(rng.integers(1, 4))):
        kind = rng.choice(["conv", "block", "pool"])
        if kind == "conv":
            cout, k = int(rng.integers(2, 12)), int(rng.choice([1, 3, 5]))
            s, p = int(rng.integers(1, 3)), int(rng.integers(0, k // 2 + 1))
            if H + 2 * p < k or W + 2 * p < k:
                continue
            cur, H, W = conv(cur, C, cout, k, s, p, rng.random() < 0.7)
            C = cout
        elif kind == "block":
            cout, s = int(rng.integers(2, 12)), int(rng.integers(1, 3))
            a, Ha, Wa = conv(cur, C, cout, 3, s, 1, True)
            H0, W0 = H, W
            H, W = Ha, Wa
            b2, H, W = conv(a, cout, cout, 3, 1, 1, False)
            if s == 1 and cout == C and rng.random() < 0.5:
                skip = cur
            else:
                H, W = H0, W0
                skip, H, W = conv(cur, C, cout, 1, s, 0, False)
            out = name("add")
            nodes.append(ow.node("Add", [b2, skip] if rng.random() < 0.5 else [skip, b2], [out]))
            if rng.random() < 0.7:
                r = name("relu")
                nodes.append(ow.node("Relu", [out], [r]))
                out = r
            cur, C = out, cout
        elif H >= 3 and W >= 3:
            k, s = int(rng.integers(2, 4)), int(rng.integers(1, 3))
            p = int(rng.integers(0, k // 2 + 1))
            out = name("pool")
            nodes.append(ow.node("MaxPool", [cur], [out], kernel_shape=[k, k], strides=[s, s], pads=[p, p, p, p]))
            cur, H, W = out, (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    if rng.random() < 0.5:
        nodes.append(ow.node("GlobalAveragePool", [cur], ["gap"]))
        nodes.append(ow.node("Flatten", ["gap"], ["flat"], axis=1))
        feats = C
    else:
        nodes.append(ow.node("Flatten", [cur], ["flat"], axis=1))
        feats = C * H * W
    classes = int(rng.integers(1, 9))
    fw = rng.standard_normal((classes, feats)).astype(np.float32)
    fw[rng.random(fw.shape) < 0.5] = 0
    inits += [("fcw", fw), ("fcb", rng.standard_normal(classes).astype(np.float32))]
    nodes.append(ow.node("Gemm", ["flat", "fcw", "fcb"], ["output"], alpha=1.0, beta=1.0, transB=1))
    return ow.model(nodes, [("input", shape_in)], [("output", (B, classes))], inits), shape_in


@pytest.mark.parametrize("seed", [41, 42, 43, 44])
def test_random_cnn_graphs(backend, oracle, tmp_path, seed):
    """Whole models: loader (shape inference, fusions), planner, device chain and launch graph on
    random graphs, bit for bit against the oracle's layer-by-layer execution of the same file."""
    import onnx_wire as ow
    from graph_oracle import run_graph
    rng = np.random.default_rng(seed)
    for it in range(10):
        B = int(rng.choice([1, 2, 3, 4, 8, 16]))
        payload, shape_in = _random_cnn(rng, B)
        path = ow.save(str(tmp_path / ("g%d.onnx" % it)), payload)
        model = backend.SparseOnnxModel(path)
        X = rng.standard_normal(shape_in).astype(np.float32)
        want = run_graph(oracle, payload, X)
        got = model.run(X)
        assert got.shape == want.shape and np.array_equal(got, want), "seed %d graph %d: %s" % (seed, it, model.describe())
        assert np.array_equal(model.run(np.asfortranarray(X)), want)
        B2 = int(rng.choice([1, 4, 5]))
        X2 = rng.standard_normal((B2,) + tuple(shape_in[1:])).astype(np.float32)
        assert np.array_equal(model.run(X2), run_graph(oracle, payload, X2)), "seed %d graph %d at batch %d" % (seed, it, B2)
