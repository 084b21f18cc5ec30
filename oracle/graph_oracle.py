"""Executes an ONNX graph (as written by python/onnx_wire.py) with the CPU oracle's
kernels, layer by layer, on the [features x B] / [C][H][W][B] layout -- the checker
for SparseOnnxModel on arbitrary graphs.  Test infrastructure only."""
import numpy as np

import onnx_wire as ow


def run_graph(oracle, payload, X):
    """X: (B, ...) C-order input.  Returns the (B, ...) C-order output."""
    from oracle import conv_geom
    g = ow.read_model(payload)
    init = g["initializers"]
    B = X.shape[0]
    in_name = [n for n, _ in g["inputs"] if n not in init][0]
    vals = {in_name: np.ascontiguousarray(np.moveaxis(X.astype(np.float32), 0, -1))}   # (..., B)
    for n in g["nodes"]:
        op, a = n["op_type"], n["attrs"]
        x = vals.get(n["input"][0])
        if op in ("MatMul", "Gemm"):
            W = init[n["input"][1]]
            if op == "MatMul" or a.get("transB", 1) == 0:
                W = np.ascontiguousarray(W.T)
            b = init[n["input"][2]] if len(n["input"]) > 2 else None
            y = oracle.matmul(oracle.encode(W), x.reshape(-1, B), b)
        elif op == "Conv":
            W = init[n["input"][1]]
            b = init[n["input"][2]] if len(n["input"]) > 2 else None
            Cout, Cin, kH, kW = W.shape
            geom = conv_geom(Cin, Cout, kH, kW, x.shape[1], x.shape[2], tuple(a.get("strides", [1, 1])),
                             tuple(a.get("pads", [0, 0, 0, 0])[:2]), tuple(a.get("dilations", [1, 1])))
            y = oracle.conv2d_pf(oracle.encode(W.reshape(Cout, -1)), geom, x, B, b)
        elif op in ("Relu", "Sigmoid", "Tanh"):
            y = oracle.act(x, op.lower())
        elif op == "Add":
            other = vals.get(n["input"][1])
            if other is None:                       # constant operand: the bias of the preceding FC layer
                y = x + init[n["input"][1]].reshape(-1, 1)
            else:
                y = oracle.add(x, other)
        elif op == "MaxPool":
            pads = a.get("pads", [0, 0, 0, 0])
            y = oracle.maxpool_pf(x, x.shape[0], x.shape[1], x.shape[2], B, tuple(a["kernel_shape"]),
                                  tuple(a.get("strides", [1, 1])), tuple(pads[:2]))
        elif op == "GlobalAveragePool":
            y = oracle.gap_pf(x, x.shape[0], x.shape[1], x.shape[2], B)
        elif op == "Flatten":
            y = x.reshape(-1, B)
        elif op == "Identity":
            y = x
        else:
            raise NotImplementedError(op)
        vals[n["output"][0]] = y
    out = vals[g["outputs"][0][0]]
    return np.ascontiguousarray(np.moveaxis(out, -1, 0))
