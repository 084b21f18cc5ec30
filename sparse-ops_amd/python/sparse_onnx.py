"""Pure-Python ONNX runner on top of the ELLPACK kernels.

Same class, constructor and `run` as the reference's OnnxSparseModel
(python/sparse_onnx.py:6-53), without the `onnx` package: the file is read by the bundled
wire-format reader.  Behaviour kept from the reference: Gemm/MatMul weights are encoded as they
are stored (out x in for a PyTorch Gemm), a Gemm's third input is its bias, a 1-D input goes
through matvec and a 2-D (n, C) input through matmul, Relu/Sigmoid/Tanh run in numpy, any other
operator raises NotImplementedError when the model is built."""
import numpy as np

try:
    from . import onnx_wire
    from .cpp_backend import encode, matmul, matvec
except ImportError:          # imported as top-level modules (sys.path points at this directory)
    import onnx_wire
    from cpp_backend import encode, matmul, matvec


def _product_step(E, bias):
    def step(v):
        return (matvec if v.ndim == 1 else matmul)(E, v, bias)
    return step


_ELEMENTWISE = {
    "Relu": lambda v: np.maximum(v, 0),
    "Sigmoid": lambda v: 1 / (1 + np.exp(-v)),
    "Tanh": np.tanh,
}


class OnnxSparseModel:
    def __init__(self, onnx_path: str):
        with open(onnx_path, "rb") as f:
            graph = onnx_wire.read_model(f.read())
        self._initializers = {name: arr.astype(np.float32) for name, arr in graph["initializers"].items()}
        self.layers = []      # (op, Ellpack or None, bias or None, attrs), one per node: the reference's plan, same arity
        self._steps = []      # what run() calls, in order
        for node in graph["nodes"]:
            kind, operands = node["op_type"], node["input"]
            if kind in ("Gemm", "MatMul"):
                E = encode(self._initializers[operands[1]])
                bias = self._initializers[operands[2]] if kind == "Gemm" and len(operands) > 2 else None
                self.layers.append(("matmul", E, bias, {}))
                self._steps.append(_product_step(E, bias))
            elif kind in _ELEMENTWISE:
                self.layers.append((kind.lower(), None, None, {}))
                self._steps.append(_ELEMENTWISE[kind])
            else:
                raise NotImplementedError("Unsupported op %s" % kind)

    def run(self, x: np.ndarray) -> np.ndarray:
        v = np.asarray(x, dtype=np.float32)
        for step in self._steps:
            v = step(v)
        return v
