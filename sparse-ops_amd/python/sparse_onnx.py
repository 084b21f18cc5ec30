"""Pure-Python ONNX runner on top of the ELLPACK kernels: the reference's
OnnxSparseModel (python/sparse_onnx.py:6-53) without the `onnx` package -- the graph
is read by the bundled wire-format reader.  A 1-D input runs through matvec, a 2-D
(n, C) input through matmul, activations in numpy, exactly as the reference does;
as there, Gemm/MatMul weights are encoded as stored (out x in for a PyTorch Gemm)."""
import numpy as np

try:
    from . import onnx_wire
    from .cpp_backend import encode, matmul, matvec
except ImportError:          # imported as top-level modules (sys.path points at this directory)
    import onnx_wire
    from cpp_backend import encode, matmul, matvec


class OnnxSparseModel:
    def __init__(self, onnx_path: str):
        with open(onnx_path, "rb") as f:
            graph = onnx_wire.read_model(f.read())
        self._initializers = {k: v.astype(np.float32) for k, v in graph["initializers"].items()}
        self.layers = []
        for node in graph["nodes"]:
            op = node["op_type"]
            if op in ("Gemm", "MatMul"):
                W = self._initializers[node["input"][1]]
                b = self._initializers[node["input"][2]] if op == "Gemm" and len(node["input"]) > 2 else None
                self.layers.append(("matmul", encode(W), b))
            elif op in ("Relu", "Sigmoid", "Tanh"):
                self.layers.append((op.lower(), None, None))
            else:
                raise NotImplementedError("Unsupported op %s" % op)

    def run(self, x: np.ndarray) -> np.ndarray:
        v = x.astype(np.float32)
        for op, E, b in self.layers:
            if op == "matmul":
                v = matvec(E, v, b) if v.ndim == 1 else matmul(E, v, b)
            elif op == "relu":
                v = np.maximum(v, 0)
            elif op == "sigmoid":
                v = (1 / (1 + np.exp(-v))).astype(np.float32)
            elif op == "tanh":
                v = np.tanh(v)
        return v
