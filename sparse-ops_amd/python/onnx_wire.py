"""Dependency-free ONNX writer and reader (protobuf wire format, no `onnx` package).

The reference's scripts export models with torch.onnx and read them with the
`onnx` package (tests/onnx/create_model.py, python/sparse_onnx.py:1-4); neither is
available in a ROCm image, so models are written and read here directly against
the field numbers of onnx.proto.  Only what the sparse runtime consumes is
covered: ModelProto{ir_version=1, producer_name=2, graph=7, opset_import=8},
GraphProto{node=1, name=2, initializer=5, input=11, output=12},
NodeProto{input=1, output=2, name=3, op_type=4, attribute=5},
AttributeProto{name=1, f=2, i=3, s=4, floats=7, ints=8, type=20},
TensorProto{dims=1, data_type=2, float_data=4, name=8, raw_data=9},
ValueInfoProto{name=1, type=2}, TypeProto{tensor_type=1{elem_type=1, shape=2}},
TensorShapeProto{dim=1{dim_value=1, dim_param=2}}.
"""
import struct

import numpy as np

FLOAT = 1
ATTR_FLOAT, ATTR_INT, ATTR_STRING, ATTR_FLOATS, ATTR_INTS = 1, 2, 3, 6, 7


# ------------------------------------------------------------------ writer

def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _key(field, wt):
    return _varint((field << 3) | wt)


def _len(field, payload):
    return _key(field, 2) + _varint(len(payload)) + payload


def _str(field, s):
    return _len(field, s.encode() if isinstance(s, str) else s)


def _int(field, v):
    return _key(field, 0) + _varint(v)


def tensor(name, array, raw=True):
    a = np.ascontiguousarray(array, dtype=np.float32)
    out = b"".join(_int(1, d) for d in a.shape) + _int(2, FLOAT)
    if raw:
        out += _len(9, a.tobytes())
    else:
        out += _len(4, a.tobytes())      # packed repeated float
    return out + _str(8, name)


def attribute(name, value):
    out = _str(1, name)
    if isinstance(value, float):
        return out + _key(2, 5) + struct.pack("<f", value) + _int(20, ATTR_FLOAT)
    if isinstance(value, (int, np.integer)):
        return out + _int(3, int(value)) + _int(20, ATTR_INT)
    if isinstance(value, (str, bytes)):
        return out + _str(4, value) + _int(20, ATTR_STRING)
    vals = list(value)
    if vals and isinstance(vals[0], float):
        return out + _len(7, struct.pack("<%df" % len(vals), *vals)) + _int(20, ATTR_FLOATS)
    return out + b"".join(_int(8, int(v)) for v in vals) + _int(20, ATTR_INTS)


def node(op_type, inputs, outputs, name="", **attrs):
    out = b"".join(_str(1, i) for i in inputs) + b"".join(_str(2, o) for o in outputs)
    if name:
        out += _str(3, name)
    out += _str(4, op_type)
    for k, v in attrs.items():
        out += _len(5, attribute(k, v))
    return out


def value_info(name, shape, elem_type=FLOAT):
    dims = b""
    for d in shape:
        dims += _len(1, _str(2, d) if isinstance(d, str) else _int(1, d))
    tensor_type = _int(1, elem_type) + _len(2, dims)
    return _str(1, name) + _len(2, _len(1, tensor_type))


def model(nodes, inputs, outputs, initializers, graph_name="g", opset=14, initializers_as_inputs=False):
    """nodes: list of node() payloads; inputs/outputs: list of (name, shape);
    initializers: list of (name, ndarray) or tensor() payloads."""
    g = b"".join(_len(1, n) for n in nodes) + _str(2, graph_name)
    inits = [t if isinstance(t, bytes) else tensor(*t) for t in initializers]
    g += b"".join(_len(5, t) for t in inits)
    if initializers_as_inputs:          # old exporters list weights among graph inputs
        for t in initializers:
            if not isinstance(t, bytes):
                g += _len(11, value_info(t[0], np.shape(t[1])))
    g += b"".join(_len(11, value_info(n, s)) for n, s in inputs)
    g += b"".join(_len(12, value_info(n, s)) for n, s in outputs)
    opset_import = _str(1, "") + _int(2, opset)
    return _int(1, 8) + _str(2, "sparseops-amd") + _len(7, g) + _len(8, opset_import)


def save(path, payload):
    with open(path, "wb") as f:
        f.write(payload)
    return path


def mlp_model(weights, acts, batch, biases=None, use_gemm=False):
    """MatMul (weights stored N x M, no bias -- src/sparse_onnx.cpp:198-201) or
    Gemm (transB=1, weights M x N, bias) chain with the given activation op names
    ('Relu' | 'Sigmoid' | 'Tanh' | None) after each layer.  weights[l] is (out, in)."""
    nodes, inits = [], []
    cur = "input"
    for l, W in enumerate(weights):
        out = "fc%d" % l
        if use_gemm:
            inits.append(("W%d" % l, W))
            ins = [cur, "W%d" % l]
            if biases is not None and biases[l] is not None:
                inits.append(("b%d" % l, biases[l]))
                ins.append("b%d" % l)
            nodes.append(node("Gemm", ins, [out], alpha=1.0, beta=1.0, transB=1))
        else:
            inits.append(("W%d" % l, np.ascontiguousarray(W.T)))
            nodes.append(node("MatMul", [cur, "W%d" % l], [out]))
        cur = out
        if acts[l]:
            nodes.append(node(acts[l], [cur], ["act%d" % l]))
            cur = "act%d" % l
    n_in, n_out = weights[0].shape[1], weights[-1].shape[0]
    return model(nodes, [("input", (batch, n_in))], [(cur, (batch, n_out))], inits)


# ------------------------------------------------------------------ reader

def _read_varint(buf, pos):
    v = shift = 0
    while True:
        b = buf[pos]
        pos += 1
        v |= (b & 0x7F) << shift
        if not b & 0x80:
            return v, pos
        shift += 7


def fields(buf):
    """Yield (field, wire_type, value) for every field of a message; value is an int
    for varint/fixed and a memoryview for length-delimited fields."""
    buf = memoryview(buf)
    pos = 0
    while pos < len(buf):
        key, pos = _read_varint(buf, pos)
        f, wt = key >> 3, key & 7
        if wt == 0:
            v, pos = _read_varint(buf, pos)
        elif wt == 1:
            v = struct.unpack_from("<Q", buf, pos)[0]
            pos += 8
        elif wt == 2:
            n, pos = _read_varint(buf, pos)
            if pos + n > len(buf):
                raise ValueError("truncated protobuf")
            v = buf[pos:pos + n]
            pos += n
        elif wt == 5:
            v = struct.unpack_from("<I", buf, pos)[0]
            pos += 4
        else:
            raise ValueError("unsupported wire type %d" % wt)
        yield f, wt, v


def _signed(v):
    return v - (1 << 64) if v >= (1 << 63) else v


def read_tensor(buf):
    dims, raw, floats, name, dtype = [], None, [], "", 0
    for f, wt, v in fields(buf):
        if f == 1:
            if wt == 0:
                dims.append(_signed(v))
            else:
                p = 0
                while p < len(v):
                    d, p = _read_varint(v, p)
                    dims.append(_signed(d))
        elif f == 2:
            dtype = v
        elif f == 4:
            floats.append(np.frombuffer(v, dtype="<f4") if wt == 2 else
                          np.array([struct.unpack("<f", struct.pack("<I", v))[0]], dtype=np.float32))
        elif f == 8:
            name = bytes(v).decode()
        elif f == 9:
            raw = bytes(v)
    if raw:
        arr = np.frombuffer(raw, dtype="<f4")
    elif floats:
        arr = np.concatenate(floats)
    else:
        arr = np.zeros(0, dtype=np.float32)
    return name, arr.astype(np.float32).reshape(dims), dtype


def read_model(payload):
    """-> dict(nodes=[dict(op_type, input, output, attrs)], initializers={name: array},
    inputs=[(name, shape)], outputs=[(name, shape)])"""
    graph = None
    for f, wt, v in fields(payload):
        if f == 7 and wt == 2:
            graph = v
    if graph is None:
        raise ValueError("no graph in model")
    out = {"nodes": [], "initializers": {}, "inputs": [], "outputs": []}

    def read_vi(buf):
        name, shape = "", []
        for f, wt, v in fields(buf):
            if f == 1:
                name = bytes(v).decode()
            elif f == 2:
                for f2, _, v2 in fields(v):
                    if f2 != 1:
                        continue
                    for f3, _, v3 in fields(v2):
                        if f3 != 2:
                            continue
                        for f4, _, v4 in fields(v3):
                            if f4 != 1:
                                continue
                            dim = None
                            for f5, wt5, v5 in fields(v4):
                                dim = v5 if f5 == 1 else bytes(v5).decode()
                            shape.append(dim)
        return name, tuple(shape)

    for f, wt, v in fields(graph):
        if f == 1:
            n = {"op_type": "", "input": [], "output": [], "attrs": {}}
            for f2, wt2, v2 in fields(v):
                if f2 == 1:
                    n["input"].append(bytes(v2).decode())
                elif f2 == 2:
                    n["output"].append(bytes(v2).decode())
                elif f2 == 4:
                    n["op_type"] = bytes(v2).decode()
                elif f2 == 5:
                    an, val, ints, fl = "", None, [], []
                    for f3, wt3, v3 in fields(v2):
                        if f3 == 1:
                            an = bytes(v3).decode()
                        elif f3 == 2:
                            val = struct.unpack("<f", struct.pack("<I", v3))[0]
                        elif f3 == 3:
                            val = _signed(v3)
                        elif f3 == 4:
                            val = bytes(v3)
                        elif f3 == 7:
                            fl.extend(np.frombuffer(v3, dtype="<f4").tolist() if wt3 == 2 else
                                      [struct.unpack("<f", struct.pack("<I", v3))[0]])
                        elif f3 == 8:
                            if wt3 == 0:
                                ints.append(_signed(v3))
                            else:
                                p = 0
                                while p < len(v3):
                                    d, p = _read_varint(v3, p)
                                    ints.append(_signed(d))
                    n["attrs"][an] = ints if ints else (fl if fl else val)
            out["nodes"].append(n)
        elif f == 5:
            name, arr, _ = read_tensor(v)
            out["initializers"][name] = arr
        elif f == 11:
            out["inputs"].append(read_vi(v))
        elif f == 12:
            out["outputs"].append(read_vi(v))
    return out
