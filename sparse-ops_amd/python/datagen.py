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
