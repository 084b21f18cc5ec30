"""SparseOnnxModel on the GPU: ONNX graphs written by python/onnx_wire.py, executed
by the device-resident layer chain, checked layer-composition-wise against the
oracle (bit-exact where every layer is, 1e-5 relative otherwise) and against
torch on the CPU (the reference's own comparisons use atol=1e-4,
tests/test_onnx.py:135, tests/full_test.py:88)."""
import os

import numpy as np
import pytest

from conftest import rel_err

import datagen
import onnx_wire as ow

pytestmark = pytest.mark.gpu
ACTS = {"Relu": "relu", "Sigmoid": "sigmoid", "Tanh": "tanh", None: "none"}


def oracle_mlp(oracle, Ws, acts, X_bm, biases=None):
    """X_bm is (B, features); the chain runs on [features x B]."""
    A = np.ascontiguousarray(X_bm.T)
    for l, W in enumerate(Ws):
        A = oracle.matmul(oracle.encode(W), A, None if biases is None else biases[l], ACTS[acts[l]])
    return np.ascontiguousarray(A.T)


@pytest.mark.parametrize("use_gemm", [False, True])
def test_mlp_small(backend, oracle, tmp_path, use_gemm):
    rng = np.random.default_rng(5)
    dims, B = (37, 64, 50, 11), 24
    Ws = [datagen.magnitude_prune(rng.standard_normal((o, i)).astype(np.float32), .8) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.standard_normal(o).astype(np.float32) for o in dims[1:]] if use_gemm else None
    acts = ["Relu", "Sigmoid", None]
    path = ow.save(str(tmp_path / "mlp.onnx"), ow.mlp_model(Ws, acts, B, bs, use_gemm))
    model = backend.SparseOnnxModel(path)
    assert model.output_shape() == [B, 11] and model.input_shape() == [B, 37]
    desc = model.describe()
    assert len(desc) == 3 and "act=relu" in desc[0] and "act=sigmoid" in desc[1] and "act=none" in desc[2]   # fused
    X = rng.random((B, 37)).astype(np.float32)
    Yo = oracle_mlp(oracle, Ws, acts, X, bs)
    Y = model.run(X)                                      # C-order (B, F): transposed on the device
    assert Y.shape == (B, 11) and rel_err(Y, Yo) <= 1e-6
    Yf = model.run(np.asfortranarray(X))                  # Fortran order is already [F x B]
    assert Yf.shape == (B, 11) and np.array_equal(Yf, Y)
    assert np.array_equal(model.run(X.astype(np.float64)), Y)
    # fp64 ground truth
    A = X.astype(np.float64)
    for l, W in enumerate(Ws):
        A = A @ W.T.astype(np.float64) + (0 if bs is None else bs[l])
        A = {"Relu": lambda v: np.maximum(v, 0), "Sigmoid": lambda v: 1 / (1 + np.exp(-v)), None: lambda v: v}[acts[l]](A)
    assert rel_err(Y, A) <= 1e-5 and np.allclose(Y, A, atol=1e-4)


def test_mlp_resize_and_repeat(backend, oracle, tmp_path):
    rng = np.random.default_rng(6)
    Ws = [datagen.magnitude_prune(rng.standard_normal((48, 30)).astype(np.float32), .7),
          datagen.magnitude_prune(rng.standard_normal((9, 48)).astype(np.float32), .5)]
    acts = ["Tanh", "Relu"]
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "m.onnx"), ow.mlp_model(Ws, acts, 16)))
    for B in (16, 16, 5, 64, 16, 1):
        if B == 64:
            model.resize_buffers(64)
            assert model.batch() == 64
        X = rng.standard_normal((B, 30)).astype(np.float32)
        Y = model.run(X)
        assert model.batch() == B and model.output_shape() == [B, 9]
        assert rel_err(Y, oracle_mlp(oracle, Ws, acts, X)) <= 1e-6
    with pytest.raises(RuntimeError, match="features per sample"):
        model.run(np.zeros((4, 31), np.float32))


def test_mlp_graph_and_eager_agree(backend, tmp_path):
    rng = np.random.default_rng(7)
    Ws = [datagen.magnitude_prune(rng.standard_normal((80, 60)).astype(np.float32), .8),
          datagen.magnitude_prune(rng.standard_normal((20, 80)).astype(np.float32), .8)]
    path = ow.save(str(tmp_path / "m.onnx"), ow.mlp_model(Ws, ["Relu", "Tanh"], 32))
    X = rng.standard_normal((32, 60)).astype(np.float32)
    Yd = backend.SparseOnnxModel(path).run(X)      # the library's own choice (short chain: no graph)
    results = {}
    for no_graph in ("0", "1"):                    # "0": always record a launch graph, "1": never
        os.environ["SPARSEOPS_NO_GRAPH"] = no_graph
        try:
            model = backend.SparseOnnxModel(path)
            results[no_graph] = [model.run(X) for _ in range(3)]      # replays too
        finally:
            del os.environ["SPARSEOPS_NO_GRAPH"]
    for Y in results["0"] + results["1"]:
        assert np.array_equal(Y, Yd)


def test_mlp_config4(backend, oracle, tmp_path):
    """784 -> 4096 -> 4096 -> 4096 -> 10, 90 % magnitude-pruned, ReLU/Sigmoid/Tanh, B = 256."""
    Ws = datagen.config4_weights()
    acts = ["Relu", "Sigmoid", "Tanh", None]
    X = datagen.config4_input()
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "c4.onnx"), ow.mlp_model(Ws, acts, 256)))
    desc = model.describe()
    assert len(desc) == 4 and all(d.startswith("MatMul") for d in desc)
    Y = model.run(X)
    Yo = oracle_mlp(oracle, Ws, acts, X)
    assert Y.shape == (256, 10)
    assert rel_err(Y, Yo) <= 1e-5 and np.allclose(Y, Yo, atol=1e-4)
    assert np.array_equal(model.run(X), Y)               # deterministic across replays


def cnn_model(rng, B, H=16):
    """The reference's full_test.py topology (tests/full_test.py:21-41):
    Conv3x3 -> ReLU -> MaxPool -> {Conv3x3 -> ReLU, Conv1x1} -> Add -> GAP -> Flatten -> FC -> ReLU,
    plus a stride-2 conv and an Identity to exercise aliasing."""
    t = {"W1": datagen.he_sparse_conv(rng, 8, 3, 3, .5), "b1": rng.standard_normal(8).astype(np.float32),
         "W2": datagen.he_sparse_conv(rng, 16, 8, 3, .7), "b2": rng.standard_normal(16).astype(np.float32),
         "W3": datagen.he_sparse_conv(rng, 16, 8, 1, .3),
         "Wf": datagen.magnitude_prune(rng.standard_normal((10, 16)).astype(np.float32), .5),
         "bf": rng.standard_normal(10).astype(np.float32)}
    nodes = [ow.node("Conv", ["x", "W1", "b1"], ["c1"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1]),
             ow.node("Relu", ["c1"], ["r1"]),
             ow.node("MaxPool", ["r1"], ["p1"], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1]),
             ow.node("Identity", ["p1"], ["p1i"]),
             ow.node("Conv", ["p1i", "W2", "b2"], ["c2"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[2, 2]),
             ow.node("Relu", ["c2"], ["r2"]),
             ow.node("Conv", ["p1", "W3"], ["c3"], kernel_shape=[1, 1], strides=[2, 2]),
             ow.node("Add", ["r2", "c3"], ["a1"]),
             ow.node("GlobalAveragePool", ["a1"], ["g1"]),
             ow.node("Flatten", ["g1"], ["f1"], axis=1),
             ow.node("Gemm", ["f1", "Wf", "bf"], ["fc"], alpha=1.0, beta=1.0, transB=1),
             ow.node("Relu", ["fc"], ["y"])]
    return ow.model(nodes, [("x", (B, 3, H, H))], [("y", (B, 10))], list(t.items())), t


def torch_cnn(t, X):
    import torch
    import torch.nn.functional as F
    T = {k: torch.from_numpy(v).double() for k, v in t.items()}
    x = torch.from_numpy(X).double()
    p1 = F.max_pool2d(F.relu(F.conv2d(x, T["W1"], T["b1"], padding=1)), 3, 2, 1)
    a1 = F.relu(F.conv2d(p1, T["W2"], T["b2"], stride=2, padding=1)) + F.conv2d(p1, T["W3"], None, stride=2)
    return F.relu(a1.mean(dim=(2, 3)) @ T["Wf"].T + T["bf"]).numpy()


def oracle_cnn(oracle, t, X):
    from oracle import conv_geom
    B, _, H, _ = X.shape
    A = np.ascontiguousarray(X.transpose(1, 2, 3, 0))                        # [C][H][W][B]
    E1, E2, E3 = (oracle.encode(t[k].reshape(t[k].shape[0], -1)) for k in ("W1", "W2", "W3"))
    c1 = oracle.conv2d_pf(E1, conv_geom(3, 8, 3, 3, H, H, pad=(1, 1)), A, B, t["b1"], "relu")
    p1 = oracle.maxpool_pf(c1, 8, H, H, B, (3, 3), (2, 2), (1, 1))
    Hp = p1.shape[1]
    r2 = oracle.conv2d_pf(E2, conv_geom(8, 16, 3, 3, Hp, Hp, (2, 2), (1, 1)), p1, B, t["b2"], "relu")
    c3 = oracle.conv2d_pf(E3, conv_geom(8, 16, 1, 1, Hp, Hp, (2, 2)), p1, B, None)
    a1 = oracle.add(r2, c3)
    g1 = oracle.gap_pf(a1, 16, a1.shape[1], a1.shape[2], B)
    return oracle.matmul(oracle.encode(t["Wf"]), g1, t["bf"], "relu").T


@pytest.mark.parametrize("B", [1, 4, 7, 9, 12, 20, 32])      # carried in rows of 4, 4, 8, 16, 16, 32, 32 entries
def test_cnn(backend, oracle, tmp_path, B):
    rng = np.random.default_rng(8 + B)
    payload, t = cnn_model(rng, B)
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "cnn.onnx"), payload))
    desc = model.describe()
    # the residual Add is fused into the second 3x3 convolution
    assert [d.split()[0] for d in desc] == ["Conv", "MaxPool", "Conv", "Conv", "GlobalAveragePool", "Gemm"]
    assert "act=relu" in desc[0] and "act=relu" in desc[2] and "act=none" in desc[3] and "+residual" in desc[3]
    assert "act=relu" in desc[5]
    X = rng.standard_normal((B, 3, 16, 16)).astype(np.float32)
    Y = model.run(X)                                                         # C-order NCHW in, (B, 10) out
    assert Y.shape == (B, 10)
    assert np.array_equal(Y, oracle_cnn(oracle, t, X))                       # every layer is bit-exact
    Yt = torch_cnn(t, X)
    assert rel_err(Y, Yt) <= 1e-5 and np.allclose(Y, Yt, atol=1e-4)
    assert np.array_equal(model.run(np.asfortranarray(X)), Y)                # any memory order, same answer


def test_conv_output_model(backend, oracle, tmp_path):
    """A graph that ends in a 4-D tensor returns (B, C, H, W) in C order."""
    from oracle import conv_geom
    rng = np.random.default_rng(9)
    W = datagen.he_sparse_conv(rng, 5, 2, 3, .5)
    payload = ow.model([ow.node("Conv", ["x", "W"], ["y"], kernel_shape=[3, 3], pads=[0, 0, 0, 0])],
                       [("x", (3, 2, 9, 7))], [("y", (3, 5, 7, 5))], [("W", W)])
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "c.onnx"), payload))
    assert model.output_shape() == [3, 5, 7, 5]
    X = rng.standard_normal((3, 2, 9, 7)).astype(np.float32)
    Y = model.run(X)
    Yo = oracle.conv2d_pf(oracle.encode(W.reshape(5, -1)), conv_geom(2, 5, 3, 3, 9, 7),
                          np.ascontiguousarray(X.transpose(1, 2, 3, 0)), 3, None)
    assert Y.shape == (3, 5, 7, 5) and np.array_equal(Y, Yo.transpose(3, 0, 1, 2))


def test_matmul_add_bias_folding(backend, oracle, tmp_path):
    """MatMul followed by Add of a constant vector (how nn.Linear is exported for
    inputs of rank > 2) becomes the FC layer's bias."""
    rng = np.random.default_rng(10)
    W = datagen.magnitude_prune(rng.standard_normal((12, 20)).astype(np.float32), .6)
    b = rng.standard_normal(12).astype(np.float32)
    nodes = [ow.node("MatMul", ["x", "Wt"], ["mm"]), ow.node("Add", ["mm", "b"], ["z"]), ow.node("Relu", ["z"], ["y"])]
    payload = ow.model(nodes, [("x", (6, 20))], [("y", (6, 12))], [("Wt", np.ascontiguousarray(W.T)), ("b", b)])
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "f.onnx"), payload))
    assert len(model.describe()) == 1 and "bias=1" in model.describe()[0] and "act=relu" in model.describe()[0]
    X = rng.standard_normal((6, 20)).astype(np.float32)
    assert np.array_equal(model.run(X), oracle.matmul(oracle.encode(W), np.ascontiguousarray(X.T), b, "relu").T)


def test_python_runtime_wrappers(oracle, tmp_path):
    """python/cpp_backend.py and python/sparse_onnx.py (the reference's python/ package)."""
    from python.cpp_backend import encode, matmul, matvec
    from python.sparse_onnx import OnnxSparseModel
    rng = np.random.default_rng(13)
    Ws = [datagen.magnitude_prune(rng.standard_normal((24, 16)).astype(np.float32), .6),
          datagen.magnitude_prune(rng.standard_normal((8, 24)).astype(np.float32), .6)]
    bs = [rng.standard_normal(24).astype(np.float32), rng.standard_normal(8).astype(np.float32)]
    path = ow.save(str(tmp_path / "g.onnx"), ow.mlp_model(Ws, ["Relu", None], 4, bs, use_gemm=True))
    model = OnnxSparseModel(path)
    # the reference's plan entries are (op, E, b, attrs) (python/sparse_onnx.py:27-32)
    assert [op for op, E, b, attrs in model.layers] == ["matmul", "relu", "matmul"]
    assert all(attrs == {} for op, E, b, attrs in model.layers) and model.layers[1][1] is None
    x = rng.standard_normal(16).astype(np.float32)
    y = model.run(x)                                          # 1-D input: matvec path
    ref = Ws[1].astype(np.float64) @ np.maximum(Ws[0].astype(np.float64) @ x + bs[0], 0) + bs[1]
    assert y.shape == (8,) and rel_err(y, ref) <= 1e-5
    X = rng.standard_normal((16, 5)).astype(np.float32)       # (n, C) input: matmul path
    Y = model.run(X)
    H = oracle.matmul(oracle.encode(Ws[0]), X, bs[0], "relu")
    assert np.array_equal(Y, oracle.matmul(oracle.encode(Ws[1]), H, bs[1]))
    E = encode(Ws[0])
    assert np.array_equal(matmul(E, X, bs[0]), oracle.matmul(oracle.encode(Ws[0]), X, bs[0]))
    assert rel_err(matvec(E, x, bs[0]), Ws[0].astype(np.float64) @ x + bs[0]) <= 1e-5


def torch_resnet(t, X, width=64):
    import torch
    import torch.nn.functional as F
    T = {k: torch.from_numpy(v).double() for k, v in t.items()}
    x = F.relu(F.conv2d(torch.from_numpy(X).double(), T["stem_w"], T["stem_b"], stride=2, padding=3))
    x = F.max_pool2d(x, 3, 2, 1)
    cin = width
    for s, cout in enumerate((width, 2 * width, 4 * width, 8 * width)):
        for b in range(2):
            stride = 2 if (s > 0 and b == 0) else 1
            nm = "s%db%d" % (s, b)
            y = F.relu(F.conv2d(x, T[nm + "c1_w"], T[nm + "c1_b"], stride=stride, padding=1))
            y = F.conv2d(y, T[nm + "c2_w"], T[nm + "c2_b"], padding=1)
            skip = x if (stride == 1 and cin == cout) else F.conv2d(x, T[nm + "proj_w"], T[nm + "proj_b"], stride=stride)
            x, cin = F.relu(y + skip), cout
    return (x.mean(dim=(2, 3)) @ T["fc_w"].T + T["fc_b"]).numpy()


def test_resnet18_shaped(backend, oracle, tmp_path):
    """Config 5 topology at reduced size (B=4, 64x64, width 32) against the oracle
    chain (bit-exact) and torch fp64 (1e-5 relative, the reference's atol=1e-4)."""
    from graph_oracle import run_graph
    payload, t = datagen.resnet18_onnx(seed=47, batch=4, hw=64, sparsity=0.8, classes=100, width=32)
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "r18.onnx"), payload))
    desc = model.describe()
    # every residual Add (and the ReLU after it) is fused into the convolution before it
    assert sum(d.startswith("Conv") for d in desc) == 20 and sum("+residual" in d for d in desc) == 8
    assert not any(d.startswith("Add") or d.startswith("Relu") for d in desc)
    assert model.output_shape() == [4, 100]
    X = np.random.default_rng(1).standard_normal((4, 3, 64, 64)).astype(np.float32)
    Y = model.run(X)
    Yo = run_graph(oracle, payload, X)
    assert np.array_equal(Y, Yo)
    Yt = torch_resnet(t, X, width=32)
    assert rel_err(Y, Yt) <= 1e-5 and np.allclose(Y, Yt, atol=1e-4)


@pytest.mark.parametrize("name", ["mlp_gemm", "cnn_gap", "cnn_flatten_fc", "resnet_tiny"])
def test_torch_exported_models(backend, oracle, name):
    """Real `torch.onnx.export` files (tests/golden/torch_export, the topologies of the
    reference's tests/full_test.py, tests/test_cnn.py and tests/test_resnet.py) against
    PyTorch's own output (the reference's atol=1e-4) and the oracle chain."""
    from graph_oracle import run_graph
    d = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "torch_export")
    exp = np.load(os.path.join(d, "expected.npz"))
    X, Yt = exp[name + "__input"], exp[name + "__output"]
    path = os.path.join(d, name + ".onnx")
    model = backend.SparseOnnxModel(path)
    assert model.output_shape() == list(Yt.shape)
    Y = model.run(X)
    assert Y.shape == Yt.shape
    assert rel_err(Y, Yt) <= 1e-5 and np.allclose(Y, Yt, atol=1e-4)
    Yo = run_graph(oracle, open(path, "rb").read(), X)
    if name in ("cnn_gap", "resnet_tiny"):      # only exact layers (conv, ReLU, pools, add, FC)
        assert np.array_equal(Y, Yo)
    else:                                       # sigmoid / tanh: device libm vs glibc
        assert rel_err(Y, Yo) <= 1e-6
    # a second batch through the same model object, in Fortran order
    Y2 = model.run(np.asfortranarray(X[::-1].copy()))
    assert rel_err(Y2, Yt[::-1]) <= 1e-5


def test_resnet18_full_size_batch_independence(backend, oracle, tmp_path):
    """Config 5 at its real size (ResNet-18-shaped, 224x224, 80 % sparse): every image's output is
    independent of the batch it travels in.  Batches of 32, 16, 8 and 3 take differently tuned
    convolution kernels (channels per wave, batch tile, gather kernel), and all must give the same
    bits; the oracle pins those bits for the first image."""
    payload, _ = datagen.resnet18_onnx(seed=47, batch=32, hw=224, sparsity=0.8)
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "r18.onnx"), payload))
    X = np.random.default_rng(3).standard_normal((32, 3, 224, 224)).astype(np.float32)
    Y = model.run(X)
    assert Y.shape == (32, 1000) and np.isfinite(Y).all()
    for B in (16, 8, 3):
        assert np.array_equal(model.run(X[:B]), Y[:B]), B
    assert np.array_equal(model.run(X), Y)                       # back to 32 after the resizes
    from graph_oracle import run_graph
    assert np.array_equal(run_graph(oracle, payload, X[:1]), Y[:1])


def test_cpp_caller_of_the_reference_headers(oracle, tmp_path):
    """tests/cpp/dropin_consumer.cpp is a C++ program written against the reference's headers
    (host pointers, as its benchmark drivers call the kernels): encoder round trip, ellpack_matmul
    and the fused-ReLU instantiation bit for bit, ellpack_matvec within 1e-5, the in-place activations, the four
    conv2d_* entry points of conv_kernels.hpp on their three layouts (with and without the RBM plan), and
    SparseOnnxModel::run / resize_buffers on a Gemm+ReLU chain bit for bit against the oracle."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "dropin_consumer")
    assert os.path.exists(exe), "tests/cpp/dropin_consumer is not built (run __graft_entry__.build())"
    rng = np.random.default_rng(12)
    dims, B = (40, 96, 70, 13), 20
    Ws = [datagen.magnitude_prune(rng.standard_normal((o, i)).astype(np.float32), .75) for i, o in zip(dims[:-1], dims[1:])]
    bs = [rng.standard_normal(o).astype(np.float32) for o in dims[1:]]
    acts = ["Relu", "Relu", None]
    path = ow.save(str(tmp_path / "mlp.onnx"), ow.mlp_model(Ws, acts, B, bs, True))
    X = rng.standard_normal((B, 40)).astype(np.float32)
    Yo = oracle_mlp(oracle, Ws, acts, X, bs)                       # (B, 13)
    np.ascontiguousarray(X.T).tofile(str(tmp_path / "in.bin"))     # [features x B], the C++ contract
    np.ascontiguousarray(Yo.T).tofile(str(tmp_path / "expected.bin"))
    r = subprocess.run([exe, path, str(tmp_path / "in.bin"), str(tmp_path / "expected.bin"), str(B)],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("ok  ") == 19 and "FAIL" not in r.stdout


def _run_device(model, ctx, X_bm):
    """X_bm (B, features...) -> (B, out features...) through SparseOnnxModel::run_device on HBM buffers
    allocated through the C ABI."""
    B = X_bm.shape[0]
    Xf = np.ascontiguousarray(X_bm.reshape(B, -1).T)               # [features x B], the C++ contract
    out_features = int(np.prod(model.output_shape()[1:]))
    dX = ctx.array(Xf)
    dY = ctx.array(np.full((out_features + 64, B), np.nan, np.float32))   # 64 guard rows behind the output
    model.run_device(dX.ptr, B, dY.ptr)
    got = dY.download()
    dX.free()
    dY.free()
    assert np.isnan(got[out_features:]).all(), "run_device wrote past its [out_features x B] output"
    return np.ascontiguousarray(got[:out_features].T).reshape([B] + list(model.output_shape()[1:]))


def test_run_device_mlp_wide_hidden_layers(backend, ctx, oracle, tmp_path):
    """run_device on a chain whose hidden tensors are wider than its output and share the output's
    arena slot (slots are recycled after a tensor's last reader): the caller's [out x B] buffer
    receives the last layer only, and the result has run()'s bits.  Batch 24 is not padded, 10 is
    (no convolutions: never), so both run_device paths with an MLP and both with a CNN are taken."""
    rng = np.random.default_rng(21)
    dims, B = (60, 256, 256, 256, 10), 24
    Ws = [datagen.magnitude_prune(rng.standard_normal((o, i)).astype(np.float32), .8) for i, o in zip(dims[:-1], dims[1:])]
    acts = ["Relu", "Relu", "Relu", None]
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "mlp.onnx"), ow.mlp_model(Ws, acts, B)))
    X = rng.standard_normal((B, 60)).astype(np.float32)
    Y = model.run(X)
    assert np.array_equal(Y, oracle_mlp(oracle, Ws, acts, X))
    assert np.array_equal(_run_device(model, ctx, X), Y)
    assert np.array_equal(_run_device(model, ctx, X[:10]), Y[:10])     # another batch: resize, then run
    assert np.array_equal(_run_device(model, ctx, X), Y)


@pytest.mark.parametrize("B", [32, 5])
def test_run_device_cnn(backend, ctx, tmp_path, B):
    """run_device on a ResNet-shaped stack at a batch carried as is (32) and one carried padded (5)."""
    payload, _ = datagen.resnet18_onnx(seed=5, batch=B, hw=32, sparsity=0.8, classes=10, width=16)
    model = backend.SparseOnnxModel(ow.save(str(tmp_path / "r18.onnx"), payload))
    X = np.random.default_rng(2).standard_normal((B, 3, 32, 32)).astype(np.float32)
    Y = model.run(X)
    assert np.array_equal(_run_device(model, ctx, X), Y)
    assert np.array_equal(_run_device(model, ctx, X), Y)


@pytest.mark.parametrize("B", [32, 16, 6])
def test_model_runs_the_row_block_merged_plan(backend, oracle, tmp_path, B):
    """The loader builds the row-block-merged plan for convolutions with Cout >= 32 and K >= 64 (the
    reference's rule, src/sparse_onnx.cpp:499-502) and hands it to the device library.  With the RBM kernel
    forced on every launch it fits, forbidden, and left to the library's choice, a ResNet-shaped model gives
    the same bits, and they are the oracle chain's."""
    from graph_oracle import run_graph
    payload, _ = datagen.resnet18_onnx(seed=11, batch=B, hw=64, sparsity=0.8, classes=10, width=32)
    X = np.random.default_rng(4).standard_normal((B, 3, 64, 64)).astype(np.float32)
    outs = {}
    try:
        for mode in ("1", "0", None):
            if mode is None:
                os.environ.pop("SPARSEOPS_CONV_RBM", None)
            else:
                os.environ["SPARSEOPS_CONV_RBM"] = mode
            backend.reload_tuning()
            model = backend.SparseOnnxModel(ow.save(str(tmp_path / "r18.onnx"), payload))
            outs[mode] = model.run(X)
            assert np.array_equal(model.run(X), outs[mode])
    finally:
        os.environ.pop("SPARSEOPS_CONV_RBM", None)
        backend.reload_tuning()
    assert np.array_equal(outs["1"], outs["0"]) and np.array_equal(outs[None], outs["0"])
    assert np.array_equal(outs["0"][:2], run_graph(oracle, payload, X[:2]))


def test_deep_mlp_records_the_row_block_merged_kernel(backend, oracle, tmp_path):
    """Nine 1536-wide layers at batch 256: a chain long enough to be recorded into a launch graph, whose large
    layers run on the row-block-merged matmul (workspace and records prepared by resize_buffers, outside the
    recording).  Replays, an eager model (SPARSEOPS_NO_GRAPH=1) and a second batch size agree bit for bit with
    one another; against the in-order CPU chain the result is within the tolerance of that kernel."""
    rng = np.random.default_rng(91)
    Ws = [datagen.magnitude_prune((rng.standard_normal((1536, 1536)) * 0.07).astype(np.float32), .9) for _ in range(9)]
    acts = ["Relu"] * 8 + [None]
    path = ow.save(str(tmp_path / "deep.onnx"), ow.mlp_model(Ws, acts, 256))
    X = rng.standard_normal((256, 1536)).astype(np.float32)
    Yo = oracle_mlp(oracle, Ws, acts, X)
    outs = {}
    os.environ["SPARSEOPS_MATMUL_RBM"] = "1"                   # 1536-row layers do not cover the chip: ask for the kernel
    try:
        for no_graph in ("0", "1"):
            os.environ["SPARSEOPS_NO_GRAPH"] = no_graph
            backend.reload_tuning()
            model = backend.SparseOnnxModel(path)
            outs[no_graph] = [model.run(X) for _ in range(3)]
            if no_graph == "0":
                model.resize_buffers(128)                      # other width: records rewritten, graph re-recorded
                half = [model.run(X[:128]) for _ in range(2)]
                model.resize_buffers(256)
                outs["back"] = [model.run(X)]
    finally:
        del os.environ["SPARSEOPS_NO_GRAPH"], os.environ["SPARSEOPS_MATMUL_RBM"]
        backend.reload_tuning()
    assert not np.array_equal(outs["0"][0], Yo)                # the in-order kernels would give the CPU chain's bits
    for Y in outs["0"] + outs["1"] + outs["back"]:
        assert np.array_equal(Y, outs["0"][0])
    assert np.array_equal(half[0], half[1])
    assert rel_err(outs["0"][0], Yo) <= 1e-4 and rel_err(half[0], Yo[:128]) <= 1e-4
