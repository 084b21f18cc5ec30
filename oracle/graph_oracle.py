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


class RefGraph:
    """The same graph with the reference's own compiled kernels where oracle/_ref has them:
    every Conv through conv2d_rbm_fmajor_implicit (src/layers/conv_kernels.cpp:66-147; the
    reference's variant that is correct for strided layers) on its Fortran (B,C,H,W) layout, with
    Conv+Relu fused the way its loader fuses them (src/sparse_onnx.cpp:573-620); every FC through
    ellpack_matmul.  MaxPool, Add, GlobalAveragePool and unfused activations run on the plain-C
    port (the reference's versions are private members of a class that cannot be built here).
    The constructor does the load-time work (encode, RBM plans); run() returns the output and the
    seconds spent inside kernels (layout shuffles between the two conventions are not counted)."""

    def __init__(self, ref, oracle, payload, in_hw):
        from oracle import conv_geom
        self.ref, self.oracle = ref, oracle
        g = self.g = ow.read_model(payload)
        init = g["initializers"]
        uses = {}
        for n in g["nodes"]:
            for t in n["input"]:
                uses[t] = uses.get(t, 0) + 1
        for t, _ in g["outputs"]:
            uses[t] = uses.get(t, 0) + 1
        self.in_name = [n for n, _ in g["inputs"] if n not in init][0]
        self.steps = []
        hw = {self.in_name: tuple(in_hw)}
        nodes = g["nodes"]
        skip = set()
        for i, n in enumerate(nodes):
            if i in skip:
                continue
            op, a = n["op_type"], n["attrs"]
            src, out = n["input"][0], n["output"][0]
            if op == "Conv":
                W = init[n["input"][1]]
                b = init[n["input"][2]] if len(n["input"]) > 2 else None
                Cout, Cin, kH, kW = W.shape
                H, Wi = hw[src]
                geom = conv_geom(Cin, Cout, kH, kW, H, Wi, tuple(a.get("strides", [1, 1])),
                                 tuple(a.get("pads", [0, 0, 0, 0])[:2]), tuple(a.get("dilations", [1, 1])))
                fuse = (i + 1 < len(nodes) and nodes[i + 1]["op_type"] == "Relu" and nodes[i + 1]["input"][0] == out
                        and uses.get(out, 0) == 1)
                if fuse:
                    skip.add(i + 1)
                    out = nodes[i + 1]["output"][0]
                plan = ref.conv_plan(W.reshape(Cout, -1), geom, b, fuse, 3)
                self.steps.append(("conv", src, out, (plan, geom)))
                hw[out] = (geom.H_out, geom.W_out)
            elif op in ("MatMul", "Gemm"):
                W = init[n["input"][1]]
                if op == "MatMul" or a.get("transB", 1) == 0:
                    W = np.ascontiguousarray(W.T)
                b = init[n["input"][2]] if len(n["input"]) > 2 else None
                self.steps.append(("fc", src, out, (ref.encode(W), b)))
            elif op == "MaxPool":
                pads = a.get("pads", [0, 0, 0, 0])
                k, s, p = tuple(a["kernel_shape"]), tuple(a.get("strides", [1, 1])), tuple(pads[:2])
                H, Wi = hw[src]
                hw[out] = ((H + 2 * p[0] - k[0]) // s[0] + 1, (Wi + 2 * p[1] - k[1]) // s[1] + 1)
                self.steps.append(("maxpool", src, out, (k, s, p)))
            elif op == "Add":
                self.steps.append(("add", src, out, n["input"][1]))
                hw[out] = hw.get(src)
            elif op in ("Relu", "Sigmoid", "Tanh"):
                self.steps.append(("act", src, out, op.lower()))
                hw[out] = hw.get(src)
            elif op == "GlobalAveragePool":
                self.steps.append(("gap", src, out, None))
            elif op in ("Flatten", "Identity"):
                self.steps.append(("alias", src, out, None))
                hw[out] = hw.get(src)
            else:
                raise NotImplementedError(op)

    def run(self, X):
        import time
        ref, orc, init = self.ref, self.oracle, self.g["initializers"]
        B = X.shape[0]
        vals = {self.in_name: np.ascontiguousarray(np.moveaxis(X.astype(np.float32), 0, -1))}   # [C][H][W][B]
        spent = 0.0
        for kind, src, out, arg in self.steps:
            x = vals[src]
            if kind == "conv":
                plan, geom = arg
                xf = np.ascontiguousarray(x.transpose(2, 1, 0, 3)).ravel()             # Fortran (B,C,H,W)
                dst = np.empty(geom.Cout * geom.H_out * geom.W_out * B, dtype=np.float32)
                t0 = time.perf_counter()
                ref.conv_run(plan, geom, xf, B, out=dst)
                spent += time.perf_counter() - t0
                y = np.ascontiguousarray(dst.reshape(geom.W_out, geom.H_out, geom.Cout, B).transpose(2, 1, 0, 3))
            elif kind == "fc":
                h, b = arg
                x2 = x.reshape(-1, B)
                t0 = time.perf_counter()
                y = ref.matmul(h, x2, b)
                spent += time.perf_counter() - t0
            elif kind == "alias":
                y = x.reshape(-1, B) if x.ndim == 4 else x
            else:
                t0 = time.perf_counter()
                if kind == "maxpool":
                    k, s, p = arg
                    y = orc.maxpool_pf(x, x.shape[0], x.shape[1], x.shape[2], B, k, s, p)
                elif kind == "add":
                    other = vals.get(arg)
                    y = orc.add(x, other) if other is not None else x + init[arg].reshape(-1, 1)
                elif kind == "act":
                    y = orc.act(x, arg)
                else:
                    y = orc.gap_pf(x, x.shape[0], x.shape[1], x.shape[2], B)
                spent += time.perf_counter() - t0
            vals[out] = y
        res = vals[self.g["outputs"][0][0]]
        return np.ascontiguousarray(np.moveaxis(res, -1, 0)), spent

    def close(self):
        for kind, _, _, arg in self.steps:
            if kind == "conv":
                self.ref.conv_plan_free(arg[0])
        self.steps = []
