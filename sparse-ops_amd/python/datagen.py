"""Seeded synthetic inputs for the benchmark configurations and the tests.

Everything is generated with numpy's PCG64 generator from an explicit seed, so the
same arrays are produced on every machine with the same numpy.  Matrices that are
too large to hold densely are generated row by row directly in ELLPACK form.
"""
import numpy as np


class EllpackHost:
    """Plain-array ELLPACK as the encoder lays it out (include/ellpack_encoder.hpp:6-23)."""

    def __init__(self, m, n, r, Wd, idx, nnz):
        self.m, self.n, self.r = int(m), int(n), int(r)
        self.Wd = np.ascontiguousarray(Wd, dtype=np.float32).reshape(self.m, self.r)
        self.idx = np.ascontiguousarray(idx, dtype=np.uint32).reshape(self.m, self.r)
        self.nnz = np.ascontiguousarray(nnz, dtype=np.uint32).reshape(self.m)

    @property
    def total_nnz(self):
        return int(self.nnz.sum(dtype=np.int64))


def save_ellpack(path, E):
    """Write E in the format bench/bench_vendor --ellpack-file reads: b"SOELLPK1", uint32 m, n, r, 0,
    then nnz[m], idx[m*r] (uint32) and Wd[m*r] (float32), little endian."""
    with open(path, "wb") as f:
        f.write(b"SOELLPK1")
        f.write(np.array([E.m, E.n, E.r, 0], dtype="<u4").tobytes())
        f.write(E.nnz.astype("<u4").tobytes())
        f.write(E.idx.astype("<u4").tobytes())
        f.write(E.Wd.astype("<f4").tobytes())


def load_ellpack(path):
    with open(path, "rb") as f:
        if f.read(8) != b"SOELLPK1":
            raise ValueError("%s is not an ELLPACK file" % path)
        m, n, r, _ = np.frombuffer(f.read(16), dtype="<u4")
        nnz = np.frombuffer(f.read(4 * int(m)), dtype="<u4")
        idx = np.frombuffer(f.read(4 * int(m) * int(r)), dtype="<u4")
        Wd = np.frombuffer(f.read(4 * int(m) * int(r)), dtype="<f4")
    return EllpackHost(m, n, r, Wd, idx, nnz)


def encode_dense(W):
    """numpy ELLPACK encoder: same layout rules as convert_to_ellpack
    (src/ellpack_encoder.cpp:6-44), vectorised."""
    W = np.ascontiguousarray(W, dtype=np.float32)
    m, n = W.shape
    mask = W != 0
    nnz = mask.sum(axis=1).astype(np.uint32)
    r = int(nnz.max()) if m else 0
    Wd = np.zeros((m, r), dtype=np.float32)
    idx = np.zeros((m, r), dtype=np.uint32)
    rows, cols = np.nonzero(mask)
    if rows.size:
        starts = np.concatenate(([0], np.cumsum(nnz[:-1], dtype=np.int64)))
        pos = np.arange(rows.size) - starts[rows]
        Wd[rows, pos] = W[rows, cols]
        idx[rows, pos] = cols
    return EllpackHost(m, n, r, Wd, idx, nnz)


def rows_to_ellpack(m, n, row_cols, row_vals):
    nnz = np.array([len(c) for c in row_cols], dtype=np.uint32)
    r = int(nnz.max()) if m else 0
    Wd = np.zeros((m, r), dtype=np.float32)
    idx = np.zeros((m, r), dtype=np.uint32)
    for i, (c, v) in enumerate(zip(row_cols, row_vals)):
        Wd[i, :len(c)] = v
        idx[i, :len(c)] = c
    return EllpackHost(m, n, r, Wd, idx, nnz)


def bernoulli_dense(rng, m, n, keep, scale=1.0):
    """W ~ N(0, scale) with an i.i.d. Bernoulli(keep) mask
    (the reference benchmark's generator, benchmark-mkl/common/data_gen.cpp:55-61)."""
    W = (rng.standard_normal((m, n), dtype=np.float32) * np.float32(scale))
    W[rng.random((m, n), dtype=np.float32) >= keep] = 0.0
    return W


def config1(seed=42):
    """1024x1024, 90 % Bernoulli sparsity, X 1024x64, bias N(0, 0.1)."""
    rng = np.random.default_rng(seed)
    W = bernoulli_dense(rng, 1024, 1024, 0.1)
    X = rng.standard_normal((1024, 64), dtype=np.float32)
    bias = rng.standard_normal(1024, dtype=np.float32) * np.float32(0.1)
    return encode_dense(W), X, bias, W


def config2a(seed=43, m=16384, n=16384, keep=0.05):
    """matvec, uniform Bernoulli 95 % sparsity, generated in chunks of rows."""
    rng = np.random.default_rng(seed)
    cols, vals = [], []
    chunk = 512
    for i0 in range(0, m, chunk):
        rows = min(chunk, m - i0)
        mask = rng.random((rows, n), dtype=np.float32) < keep
        for i in range(rows):
            c = np.flatnonzero(mask[i]).astype(np.uint32)
            cols.append(c)
            vals.append(rng.standard_normal(c.size, dtype=np.float32))
    E = rows_to_ellpack(m, n, cols, vals)
    x = rng.standard_normal(n, dtype=np.float32)
    bias = rng.standard_normal(m, dtype=np.float32) * np.float32(0.1)
    return E, x, bias


def uniform_ellpack(seed, m, n, keep, chunk=4096):
    """Bernoulli(keep) mask with N(0,1) values, built straight into ELLPACK arrays (for matrices
    whose dense form would not fit).  A Bernoulli row is drawn through its gaps: the distances
    between consecutive nonzeros are i.i.d. Geometric(keep), so the cost is O(nnz), not O(m n)."""
    rng = np.random.default_rng(seed)
    kmax = int(n * keep + 10 * np.sqrt(n * keep * (1 - keep)) + 16)
    Wd = np.zeros((m, kmax), dtype=np.float32)
    idx = np.zeros((m, kmax), dtype=np.uint32)
    nnz = np.zeros(m, dtype=np.uint32)
    for i0 in range(0, m, chunk):
        rows = min(chunk, m - i0)
        cols = np.cumsum(rng.geometric(keep, size=(rows, kmax)), axis=1, dtype=np.int64) - 1
        live = cols < n
        assert not live[:, -1].any(), "kmax too small for this draw"
        nnz[i0:i0 + rows] = live.sum(axis=1)
        idx[i0:i0 + rows] = np.where(live, cols, 0)
        Wd[i0:i0 + rows] = np.where(live, rng.standard_normal((rows, kmax), dtype=np.float32), np.float32(0))
    r = int(nnz.max()) if m else 0
    x = rng.standard_normal(n, dtype=np.float32)
    bias = rng.standard_normal(m, dtype=np.float32) * np.float32(0.1)
    return EllpackHost(m, n, r, Wd[:, :r], idx[:, :r], nnz), x, bias


def config2b(seed=44, m=16384, n=16384, s=1.2, cap=2048):
    """matvec, skewed: per-row nnz = min(Zipf(s), cap) (clipped, so a fifth of the
    rows sit at the cap and r = cap), columns uniform without replacement, ascending."""
    rng = np.random.default_rng(seed)
    counts = np.minimum(rng.zipf(s, size=m), cap).astype(np.int64)
    cols, vals = [], []
    for i in range(m):
        k = int(counts[i])
        if k * 8 < n:
            c = np.unique(rng.integers(0, n, size=k + k // 4 + 8))
            while c.size < k:
                c = np.unique(np.concatenate((c, rng.integers(0, n, size=k))))
            c = np.sort(rng.permutation(c)[:k])
        else:
            c = np.sort(rng.permutation(n)[:k])
        cols.append(c.astype(np.uint32))
        vals.append(rng.standard_normal(k, dtype=np.float32))
    E = rows_to_ellpack(m, n, cols, vals)
    x = rng.standard_normal(n, dtype=np.float32)
    bias = rng.standard_normal(m, dtype=np.float32) * np.float32(0.1)
    return E, x, bias


def topk_rows(W, k):
    """Keep the k largest |w| of every row (ties: lower column wins)."""
    m, n = W.shape
    order = np.argsort(-np.abs(W), axis=1, kind="stable")[:, :k]
    out = np.zeros_like(W)
    rows = np.arange(m)[:, None]
    out[rows, order] = W[rows, order]
    return out


def config3(seed=45, m=4096, n=4096, C=256, density=0.1):
    """Large FC: W ~ N(0, 0.02), per-row top-10 % magnitude pruning (uniform r),
    X n x C ~ N(0,1), bias ~ N(0, 0.1)."""
    rng = np.random.default_rng(seed)
    W = rng.standard_normal((m, n), dtype=np.float32) * np.float32(0.02)
    W = topk_rows(W, int(round(n * density + 0.4)))   # 4096 -> 410
    X = rng.standard_normal((n, C), dtype=np.float32)
    bias = rng.standard_normal(m, dtype=np.float32) * np.float32(0.1)
    return encode_dense(W), X, bias


def magnitude_prune(W, sparsity):
    """Zero everything below the `sparsity` quantile of |W| (unstructured)."""
    thr = np.quantile(np.abs(W), sparsity)
    out = W.copy()
    out[np.abs(out) < thr] = 0.0
    return out


def config4_weights(seed=46, dims=(784, 4096, 4096, 4096, 10), sparsity=0.9):
    """MLP weights W_l (out x in) ~ N(0, 1/sqrt(fan_in)), 90 % magnitude-pruned."""
    rng = np.random.default_rng(seed)
    Ws = []
    for fin, fout in zip(dims[:-1], dims[1:]):
        W = rng.standard_normal((fout, fin), dtype=np.float32) * np.float32(1.0 / np.sqrt(fin))
        Ws.append(magnitude_prune(W, sparsity))
    return Ws


def config4_input(seed=46, batch=256, features=784):
    rng = np.random.default_rng(seed + 1000)
    return rng.random((batch, features), dtype=np.float32)


def he_sparse_conv(rng, cout, cin, k, sparsity=0.8):
    fan_in = cin * k * k
    W = rng.standard_normal((cout, cin, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / fan_in))
    W[rng.random(W.shape, dtype=np.float32) < sparsity] = 0.0
    return W


def resnet18_onnx(seed=47, batch=32, hw=224, sparsity=0.8, classes=1000, width=64):
    """ResNet-18-shaped graph without BatchNorm (as a constant-folded export has it,
    the reference's tests/test_resnet.py:57-70): 7x7/2 stem + 3x3/2 max-pool, four
    stages of two basic blocks (3x3 convs, 1x1 stride-2 projection on the first skip
    of stages 2-4), Add + ReLU, global average pool, Flatten, Gemm.  Conv weights
    He-initialised with i.i.d. Bernoulli sparsity.  Returns (onnx bytes, tensors)."""
    import onnx_wire as ow
    rng = np.random.default_rng(seed)
    t, nodes = {}, []

    def conv(x, name, cin, cout, k, stride, pad, relu):
        t[name + "_w"] = he_sparse_conv(rng, cout, cin, k, sparsity)
        t[name + "_b"] = rng.standard_normal(cout, dtype=np.float32) * np.float32(0.01)
        nodes.append(ow.node("Conv", [x, name + "_w", name + "_b"], [name], kernel_shape=[k, k],
                             pads=[pad] * 4, strides=[stride, stride], dilations=[1, 1], group=1))
        if relu:
            nodes.append(ow.node("Relu", [name], [name + "_r"]))
            return name + "_r"
        return name

    x = conv("input", "stem", 3, width, 7, 2, 3, True)
    nodes.append(ow.node("MaxPool", [x], ["pool"], kernel_shape=[3, 3], strides=[2, 2], pads=[1, 1, 1, 1]))
    x, cin = "pool", width
    for s, cout in enumerate((width, 2 * width, 4 * width, 8 * width)):
        for b in range(2):
            stride = 2 if (s > 0 and b == 0) else 1
            nm = "s%db%d" % (s, b)
            y = conv(x, nm + "c1", cin, cout, 3, stride, 1, True)
            y = conv(y, nm + "c2", cout, cout, 3, 1, 1, False)
            skip = x if (stride == 1 and cin == cout) else conv(x, nm + "proj", cin, cout, 1, stride, 0, False)
            nodes.append(ow.node("Add", [y, skip], [nm + "add"]))
            nodes.append(ow.node("Relu", [nm + "add"], [nm + "out"]))
            x, cin = nm + "out", cout
    nodes.append(ow.node("GlobalAveragePool", [x], ["gap"]))
    nodes.append(ow.node("Flatten", ["gap"], ["flat"], axis=1))
    t["fc_w"] = (rng.standard_normal((classes, cin), dtype=np.float32) * np.float32(1.0 / np.sqrt(cin)))
    t["fc_b"] = rng.standard_normal(classes, dtype=np.float32) * np.float32(0.01)
    nodes.append(ow.node("Gemm", ["flat", "fc_w", "fc_b"], ["logits"], alpha=1.0, beta=1.0, transB=1))
    payload = ow.model(nodes, [("input", (batch, 3, hw, hw))], [("logits", (batch, classes))], list(t.items()))
    return payload, t
