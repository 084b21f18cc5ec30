"""The dependency-free ONNX writer (python/onnx_wire.py), the C++ wire reader
(src/onnx_wire.cpp, seen through sparseops_backend.parse_onnx) and the loader's
error behaviour.  The writer is cross-checked against an independent encoder:
google.protobuf dynamic messages built from a descriptor of the same onnx.proto
fields."""
import os

import numpy as np
import pytest

import onnx_wire as ow


def small_cnn_bytes(rng, B=2):
    Wc = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    bc = rng.standard_normal(4).astype(np.float32)
    Wf = rng.standard_normal((5, 4 * 4 * 4)).astype(np.float32)
    bf = rng.standard_normal(5).astype(np.float32)
    nodes = [ow.node("Conv", ["x", "Wc", "bc"], ["c1"], kernel_shape=[3, 3], pads=[1, 1, 1, 1], strides=[1, 1],
                     dilations=[1, 1], group=1),
             ow.node("Relu", ["c1"], ["r1"]),
             ow.node("MaxPool", ["r1"], ["p1"], kernel_shape=[2, 2], strides=[2, 2], pads=[0, 0, 0, 0]),
             ow.node("Flatten", ["p1"], ["f1"], axis=1),
             ow.node("Gemm", ["f1", "Wf", "bf"], ["y"], alpha=1.0, beta=1.0, transB=1)]
    inits = [("Wc", Wc), ("bc", bc), ow.tensor("Wf", Wf, raw=False), ("bf", bf)]
    return ow.model(nodes, [("x", (B, 3, 8, 8))], [("y", (B, 5))], inits), dict(Wc=Wc, bc=bc, Wf=Wf, bf=bf)


def test_python_round_trip():
    rng = np.random.default_rng(0)
    payload, t = small_cnn_bytes(rng)
    m = ow.read_model(payload)
    assert [n["op_type"] for n in m["nodes"]] == ["Conv", "Relu", "MaxPool", "Flatten", "Gemm"]
    assert m["nodes"][0]["attrs"]["pads"] == [1, 1, 1, 1] and m["nodes"][0]["attrs"]["group"] == 1
    assert m["nodes"][4]["attrs"]["transB"] == 1 and m["nodes"][4]["attrs"]["alpha"] == 1.0
    assert m["inputs"] == [("x", (2, 3, 8, 8))] and m["outputs"] == [("y", (2, 5))]
    for k, v in t.items():
        assert np.array_equal(m["initializers"][k], v), k


def test_cpp_reader_matches_writer(backend, tmp_path):
    rng = np.random.default_rng(1)
    payload, t = small_cnn_bytes(rng)
    path = ow.save(str(tmp_path / "m.onnx"), payload)
    m = backend.parse_onnx(path)
    assert m["ir_version"] == 8 and m["opset_import"] == [("", 14)]
    assert [n["op_type"] for n in m["nodes"]] == ["Conv", "Relu", "MaxPool", "Flatten", "Gemm"]
    assert m["nodes"][0]["input"] == ["x", "Wc", "bc"] and m["nodes"][0]["output"] == ["c1"]
    assert m["nodes"][0]["attrs"]["kernel_shape"] == [3, 3] and m["nodes"][0]["attrs"]["group"] == 1
    assert m["nodes"][3]["attrs"]["axis"] == 1 and m["nodes"][4]["attrs"]["beta"] == 1.0
    assert m["inputs"] == [("x", (2, 3, 8, 8))] and m["outputs"] == [("y", (2, 5))]
    for k, v in t.items():       # raw_data and packed float_data both decode
        assert np.array_equal(m["initializers"][k], v), k


def onnx_subset_messages():
    """Message classes for the onnx.proto subset, built at run time (proto2)."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    fd = descriptor_pb2.FileDescriptorProto(name="onnx_subset.proto", package="onnxs", syntax="proto2")

    def msg(name, fields, parent=None):
        m = (parent.nested_type if parent is not None else fd.message_type).add(name=name)
        for fname, num, typ, label, tname in fields:
            f = m.field.add(name=fname, number=num, type=typ, label=label)
            if tname:
                f.type_name = tname
        return m
    O, R = F.LABEL_OPTIONAL, F.LABEL_REPEATED
    t = msg("TensorProto", [("dims", 1, F.TYPE_INT64, R, None), ("data_type", 2, F.TYPE_INT32, O, None),
                            ("float_data", 4, F.TYPE_FLOAT, R, None), ("name", 8, F.TYPE_STRING, O, None),
                            ("raw_data", 9, F.TYPE_BYTES, O, None)])
    t.field[2].options.packed = True
    msg("AttributeProto", [("name", 1, F.TYPE_STRING, O, None), ("f", 2, F.TYPE_FLOAT, O, None),
                           ("i", 3, F.TYPE_INT64, O, None), ("s", 4, F.TYPE_BYTES, O, None),
                           ("floats", 7, F.TYPE_FLOAT, R, None), ("ints", 8, F.TYPE_INT64, R, None),
                           ("type", 20, F.TYPE_INT32, O, None)])
    msg("NodeProto", [("input", 1, F.TYPE_STRING, R, None), ("output", 2, F.TYPE_STRING, R, None),
                      ("name", 3, F.TYPE_STRING, O, None), ("op_type", 4, F.TYPE_STRING, O, None),
                      ("attribute", 5, F.TYPE_MESSAGE, R, ".onnxs.AttributeProto")])
    shp = msg("TensorShapeProto", [("dim", 1, F.TYPE_MESSAGE, R, ".onnxs.TensorShapeProto.Dimension")])
    msg("Dimension", [("dim_value", 1, F.TYPE_INT64, O, None), ("dim_param", 2, F.TYPE_STRING, O, None)], shp)
    tp = msg("TypeProto", [("tensor_type", 1, F.TYPE_MESSAGE, O, ".onnxs.TypeProto.Tensor")])
    msg("Tensor", [("elem_type", 1, F.TYPE_INT32, O, None), ("shape", 2, F.TYPE_MESSAGE, O, ".onnxs.TensorShapeProto")], tp)
    msg("ValueInfoProto", [("name", 1, F.TYPE_STRING, O, None), ("type", 2, F.TYPE_MESSAGE, O, ".onnxs.TypeProto")])
    msg("GraphProto", [("node", 1, F.TYPE_MESSAGE, R, ".onnxs.NodeProto"), ("name", 2, F.TYPE_STRING, O, None),
                       ("initializer", 5, F.TYPE_MESSAGE, R, ".onnxs.TensorProto"),
                       ("input", 11, F.TYPE_MESSAGE, R, ".onnxs.ValueInfoProto"),
                       ("output", 12, F.TYPE_MESSAGE, R, ".onnxs.ValueInfoProto")])
    msg("OperatorSetIdProto", [("domain", 1, F.TYPE_STRING, O, None), ("version", 2, F.TYPE_INT64, O, None)])
    msg("ModelProto", [("ir_version", 1, F.TYPE_INT64, O, None), ("producer_name", 2, F.TYPE_STRING, O, None),
                       ("graph", 7, F.TYPE_MESSAGE, O, ".onnxs.GraphProto"),
                       ("opset_import", 8, F.TYPE_MESSAGE, R, ".onnxs.OperatorSetIdProto")])
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    return {n: message_factory.GetMessageClass(pool.FindMessageTypeByName("onnxs." + n))
            for n in ("ModelProto", "TensorProto", "NodeProto")}


def test_writer_against_protobuf_runtime(backend, tmp_path):
    M = onnx_subset_messages()
    rng = np.random.default_rng(2)
    payload, t = small_cnn_bytes(rng)
    pm = M["ModelProto"]()
    pm.ParseFromString(payload)                      # libprotobuf accepts what the writer emits
    assert pm.ir_version == 8 and pm.opset_import[0].version == 14
    g = pm.graph
    assert [n.op_type for n in g.node] == ["Conv", "Relu", "MaxPool", "Flatten", "Gemm"]
    assert list(g.node[0].attribute[1].ints) == [1, 1, 1, 1] and g.node[0].attribute[1].name == "pads"
    assert [d.dim_value for d in g.input[0].type.tensor_type.shape.dim] == [2, 3, 8, 8]
    init = {i.name: i for i in g.initializer}
    assert np.array_equal(np.frombuffer(init["Wc"].raw_data, np.float32).reshape(4, 3, 3, 3), t["Wc"])
    assert np.array_equal(np.array(init["Wf"].float_data, np.float32).reshape(5, 64), t["Wf"])
    # and the other way round: bytes produced by libprotobuf are read by both readers
    again = pm.SerializeToString()
    m2 = ow.read_model(again)
    assert np.array_equal(m2["initializers"]["Wf"], t["Wf"]) and m2["outputs"] == [("y", (2, 5))]
    path = ow.save(str(tmp_path / "pb.onnx"), again)
    m3 = backend.parse_onnx(path)
    assert np.array_equal(m3["initializers"]["Wc"], t["Wc"]) and m3["nodes"][2]["attrs"]["strides"] == [2, 2]
    # unpacked repeated fields (older writers) are accepted too
    tp = M["TensorProto"]()
    tp.ParseFromString(ow.tensor("z", np.arange(6, dtype=np.float32).reshape(2, 3), raw=False))
    assert list(tp.float_data) == [0, 1, 2, 3, 4, 5] and list(tp.dims) == [2, 3]


def load_error(backend, tmp_path, payload, match):
    path = ow.save(str(tmp_path / "bad.onnx"), payload)
    with pytest.raises(RuntimeError, match=match):
        backend.SparseOnnxModel(path)


def test_loader_errors(backend, tmp_path):
    W = np.ones((4, 3), np.float32)
    ok_in, ok_out = [("x", (2, 4))], [("y", (2, 3))]
    with pytest.raises(RuntimeError, match="Failed to open/parse ONNX file"):
        backend.SparseOnnxModel(str(tmp_path / "missing.onnx"))
    load_error(backend, tmp_path, b"\x0a\xff\xff\xff", "Failed to open/parse ONNX file")          # truncated
    good = ow.model([ow.node("MatMul", ["x", "W"], ["y"])], ok_in, ok_out, [("W", W)])
    load_error(backend, tmp_path, good[:len(good) // 2], "Failed to open/parse ONNX file")
    load_error(backend, tmp_path, ow.model([ow.node("Softmax", ["x"], ["y"])], ok_in, ok_out, []),
               "Unsupported ONNX op: Softmax")
    load_error(backend, tmp_path, ow.model([ow.node("MatMul", ["x", "W"], ["y"])], [("x", ("N", 4))], ok_out, [("W", W)]),
               "Dynamic dims not supported")
    load_error(backend, tmp_path, ow.model([ow.node("MatMul", ["x", "Wmissing"], ["y"])], ok_in, ok_out, [("W", W)]),
               "Weight 'Wmissing' not found")
    load_error(backend, tmp_path, ow.model([ow.node("MatMul", ["x", "W"], ["y"])], ok_in, ok_out + [("z", (2, 3))], [("W", W)]),
               "Expected exactly one graph output")
    load_error(backend, tmp_path, ow.model([ow.node("MatMul", ["x", "W"], ["y"])], [("x", (4,))], ok_out, [("W", W)]),
               "rank")
    load_error(backend, tmp_path, ow.model([], [], ok_out, []), "No non-initializer input")
    load_error(backend, tmp_path, ow.model([ow.node("MatMul", ["x", "W"], ["y"])], [("x", (2, 5))], ok_out, [("W", W)]),
               "features")
    Wc = np.ones((4, 2, 3, 3), np.float32)
    load_error(backend, tmp_path, ow.model([ow.node("Conv", ["x", "Wc"], ["y"], group=2)], [("x", (1, 2, 8, 8))],
                                           [("y", (1, 4, 6, 6))], [("Wc", Wc)]), "Grouped conv not supported")
    load_error(backend, tmp_path, ow.model([ow.node("Conv", ["x", "Wc"], ["y"])], [("x", (1, 3, 8, 8))],
                                           [("y", (1, 4, 6, 6))], [("Wc", Wc)]), "Conv Cin mismatch")
    load_error(backend, tmp_path, ow.model([ow.node("MaxPool", ["x"], ["y"], kernel_shape=[2, 2])], ok_in, ok_out, []),
               "Pool input must be 4D")


def test_valid_model_without_gpu_fails_loudly(backend, tmp_path):
    if backend.device_available():
        pytest.skip("a GPU is present")
    W = np.ones((4, 3), np.float32)
    path = ow.save(str(tmp_path / "ok.onnx"), ow.model([ow.node("MatMul", ["x", "W"], ["y"])], [("x", (2, 4))],
                                                       [("y", (2, 3))], [("W", W)]))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        backend.SparseOnnxModel(path)


# Real `torch.onnx.export` output (TorchScript exporter, opset 14), written once by
# tests/golden/make_torch_onnx.py together with PyTorch's own outputs.
TORCH_EXPORTS = {
    "mlp_gemm": ["Gemm", "Relu", "Gemm", "Sigmoid", "Gemm", "Tanh", "Gemm"],
    "cnn_gap": ["Conv", "Relu", "MaxPool", "Conv", "Relu", "GlobalAveragePool", "Flatten", "Gemm"],
    "cnn_flatten_fc": ["Conv", "Relu", "MaxPool", "Conv", "Tanh", "Flatten", "Gemm", "Relu", "Gemm"],
    "resnet_tiny": None,
}
EXPORT_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "torch_export")


@pytest.mark.parametrize("name", sorted(TORCH_EXPORTS))
def test_torch_exported_graph_parses(backend, name):
    """Both wire readers on files the builder's writer did not produce."""
    path = os.path.join(EXPORT_DIR, name + ".onnx")
    exp = np.load(os.path.join(EXPORT_DIR, "expected.npz"))
    m = backend.parse_onnx(path)
    mp = ow.read_model(open(path, "rb").read())
    ops = [n["op_type"] for n in m["nodes"]]
    assert ops == [n["op_type"] for n in mp["nodes"]]
    if TORCH_EXPORTS[name] is not None:
        assert ops == TORCH_EXPORTS[name]
    else:   # BatchNorm folded into the convolutions; 2 + 2 basic blocks, one projection
        assert ops.count("Conv") == 10 and ops.count("Add") == 4 and "BatchNormalization" not in ops
    assert m["inputs"] == [("input", exp[name + "__input"].shape)]
    assert m["outputs"] == [("output", exp[name + "__output"].shape)]
    assert sorted(m["initializers"]) == sorted(mp["initializers"])
    for k, v in mp["initializers"].items():
        assert np.array_equal(m["initializers"][k], v), k
    for a, b in zip(m["nodes"], mp["nodes"]):
        assert a["input"] == b["input"] and a["output"] == b["output"] and a["attrs"] == b["attrs"]


@pytest.mark.parametrize("name", sorted(TORCH_EXPORTS))
def test_torch_exported_graph_through_the_oracle_chain(oracle, name):
    """The oracle's layer chain over the exported graph reproduces PyTorch's output,
    which pins the graph semantics the GPU tests compare against (Gemm transB + bias,
    Flatten of a 4-D tensor into an FC, folded BatchNorm, residual Add)."""
    from graph_oracle import run_graph
    exp = np.load(os.path.join(EXPORT_DIR, "expected.npz"))
    payload = open(os.path.join(EXPORT_DIR, name + ".onnx"), "rb").read()
    Y = run_graph(oracle, payload, exp[name + "__input"])
    Yt = exp[name + "__output"]
    assert Y.shape == Yt.shape
    assert np.abs(Y - Yt).max() / np.abs(Yt).max() <= 1e-5 and np.allclose(Y, Yt, atol=1e-4)


@pytest.mark.parametrize("name", sorted(TORCH_EXPORTS))
def test_mutated_model_files_raise_cleanly(backend, tmp_path, name):
    """A model file is outside input: truncations, flipped bytes and oversized varints in a real
    exported graph must end in RuntimeError (or load), never in a crash or a hang.  (The same
    mutations were run against the loader built with -fsanitize=address,undefined.)"""
    good = open(os.path.join(EXPORT_DIR, name + ".onnx"), "rb").read()
    rng = np.random.default_rng(len(good))
    path = str(tmp_path / "mutated.onnx")
    loaded = 0
    for it in range(80):
        s = bytearray(good)
        kind = it % 4
        if kind == 0:
            s = s[:int(rng.integers(0, len(s) + 1))]
        elif kind == 1:
            for _ in range(int(rng.integers(1, 5))):
                s[int(rng.integers(0, len(s)))] = int(rng.integers(0, 256))
        elif kind == 2:       # the graph structure sits in the first kilobytes
            for _ in range(int(rng.integers(1, 4))):
                s[int(rng.integers(0, min(len(s), 2048)))] = int(rng.integers(0, 256))
        else:
            p = int(rng.integers(0, min(len(s) - 10, 4096)))
            s[p:p + 10] = b"\xff" * 9 + b"\x01"
        with open(path, "wb") as f:
            f.write(bytes(s))
        try:
            backend.SparseOnnxModel(path)
            loaded += 1
        except RuntimeError:
            pass
    assert loaded < 80


def test_loader_under_sanitizers(tmp_path):
    """The host ONNX loader, built with AddressSanitizer + UndefinedBehaviorSanitizer
    (`make -C sparse-ops_amd asan`, tests/cpp/fuzz_onnx.cpp), on 2000 mutations of the four
    torch-exported models: truncations, flipped bytes, oversized varints, repeated slices.  Every
    file must end in a loaded model or an exception; any sanitizer report fails the run."""
    import glob
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    binary = os.path.join(root, "tests", "cpp", "fuzz_onnx_asan")
    if not os.path.exists(binary):
        subprocess.run(["make", "-C", os.path.join(root, "sparse-ops_amd"), "asan"], check=True, stdout=subprocess.DEVNULL)
    models = sorted(glob.glob(os.path.join(root, "tests", "golden", "torch_export", "*.onnx")))
    assert len(models) == 4
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    out = subprocess.run([binary, "500", str(tmp_path)] + models, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                         errors="replace", env=env, timeout=300)        # messages quote mutated names: any bytes
    assert out.returncode == 0, out.stdout[-4000:]
    assert "2000 mutated files, no crash" in out.stdout
    assert "AddressSanitizer" not in out.stdout and "runtime error" not in out.stdout, out.stdout[-4000:]
