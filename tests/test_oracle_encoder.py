"""Pins the oracle's encoder (oracle.c: orc_ellpack_count/pack/decode) and the
shipped host encoder (sparseops_backend.convert_to_ellpack) against: the
reference's hand-written known answer, numpy closed forms, the round-trip
invariant, the special cases the reference tests, the compiled reference, and the
committed reference vectors."""
import numpy as np
import pytest

from conftest import sparse_matrix


def closed_form(W):
    mask = W != 0
    nnz = mask.sum(axis=1)
    r = int(nnz.max()) if W.shape[0] else 0
    Wd = np.zeros((W.shape[0], r), np.float32)
    idx = np.zeros((W.shape[0], r), np.uint32)
    for i in range(W.shape[0]):
        c = np.flatnonzero(mask[i])
        Wd[i, :c.size] = W[i, c]
        idx[i, :c.size] = c
    return r, Wd, idx, nnz.astype(np.uint32)


KAT = np.array([[1, 0, 0, 2], [0, 3, 0, 0], [0, 0, 4, 0], [0, 0, 0, 5]], dtype=np.float32)


def encoders(oracle, backend):
    def host(W):
        return backend.convert_to_ellpack(W)
    return [("oracle", oracle.encode), ("host", host)]


def test_known_answer_4x4(oracle, backend):
    # tests/unit/test_ellpack_encoder.py:51-77 of the reference
    for name, enc in encoders(oracle, backend):
        E = enc(KAT)
        assert (E.m, E.n, E.r) == (4, 4, 2), name
        assert E.Wd.shape == (4, 2)
        assert np.array_equal(E.Wd, [[1, 2], [3, 0], [4, 0], [5, 0]]), name
        assert np.array_equal(E.idx, [[0, 3], [1, 0], [2, 0], [3, 0]]), name
        assert np.array_equal(E.nnz, [2, 1, 1, 1]), name


@pytest.mark.parametrize("m,n,sp", [(64, 64, .3), (128, 128, .3), (32, 32, .3), (64, 32, .3), (32, 64, .9),
                                    (1, 1, 0.), (1, 1000, .1), (1000, 1, .1), (7, 5, 1.0), (10, 10, 0.)])
def test_closed_form_and_round_trip(oracle, backend, m, n, sp):
    rng = np.random.default_rng(m * 1000 + n)
    W = sparse_matrix(rng, m, n, sp, signed=False)
    r, Wd, idx, nnz = closed_form(W)
    assert r == np.max(np.count_nonzero(W, axis=1))           # :31-39
    for name, enc in encoders(oracle, backend):
        E = enc(W)
        assert (E.m, E.n, E.r) == (m, n, r), name
        assert np.array_equal(E.Wd, Wd) and np.array_equal(E.idx, idx) and np.array_equal(E.nnz, nnz), name
    assert np.array_equal(oracle.decode(oracle.encode(W)), W)   # :13-20, exact
    assert np.array_equal(backend.decode_from_ellpack(backend.convert_to_ellpack(W)), W)


def test_all_zero_and_empty(oracle, backend):
    for name, enc in encoders(oracle, backend):
        E = enc(np.zeros((32, 32), np.float32))               # :41-49
        assert (E.m, E.n, E.r) == (32, 32, 0), name
        assert E.Wd.shape == (32, 0)
        E = enc(np.zeros((0, 0), np.float32))
        assert (E.m, E.n, E.r) == (0, 0, 0), name
    assert backend.decode_from_ellpack(backend.convert_to_ellpack(np.zeros((3, 4), np.float32))).shape == (3, 4)


def test_negative_zero_dropped_nan_kept(oracle, backend):
    # v != 0.0f: -0.0f compares equal to zero, NaN compares unequal (src/ellpack_encoder.cpp:14,34)
    W = np.array([[-0.0, 1.0, np.nan], [0.0, -0.0, 0.0]], dtype=np.float32)
    for name, enc in encoders(oracle, backend):
        E = enc(W)
        assert E.r == 2 and list(E.nnz) == [2, 0], name
        assert list(E.idx[0]) == [1, 2] and E.Wd[0, 0] == 1.0 and np.isnan(E.Wd[0, 1]), name


def test_against_compiled_reference(oracle, backend, ref):
    rng = np.random.default_rng(7)
    for (m, n, sp) in [(300, 257, .9), (64, 1000, .5), (1000, 3, .2), (5, 5, 1.0)]:
        W = sparse_matrix(rng, m, n, sp)
        Er = ref.arrays(ref.encode(W))
        for name, enc in encoders(oracle, backend):
            E = enc(W)
            assert E.r == Er.r and np.array_equal(E.Wd, Er.Wd) and np.array_equal(E.idx, Er.idx) \
                and np.array_equal(E.nnz, Er.nnz), name
        assert np.array_equal(ref.decode(ref.encode(W)), W)


def test_against_reference_vectors(oracle, backend, golden):
    for key in ("enc", "encnan"):
        W = golden[key + "_W"]
        for name, enc in encoders(oracle, backend):
            E = enc(W)
            assert np.array_equal(E.Wd, golden[key + "_Wd"], equal_nan=True), name
            assert np.array_equal(E.idx, golden[key + "_idx"]) and np.array_equal(E.nnz, golden[key + "_nnz"]), name
    assert np.array_equal(oracle.decode(oracle.encode(golden["enc_W"])), golden["enc_decoded"])


def test_host_ellpack_properties(backend):
    E = backend.convert_to_ellpack(KAT)
    assert E.Xt.shape == (4, 2) and E.Xt.dtype == np.float32
    assert E.idx.dtype == np.uint32 and E.Wd.dtype == np.float32
    w = E.Wd
    w[0, 0] = 99                       # properties hand out copies (src/bindings.cpp:59-82)
    assert E.Wd[0, 0] == 1.0
    with pytest.raises(RuntimeError):
        backend.convert_to_ellpack(np.zeros(5, np.float32))


def test_datagen_encoder_matches(oracle):
    import datagen
    rng = np.random.default_rng(3)
    W = sparse_matrix(rng, 200, 300, .93)
    W[17] = 0
    E, Eo = datagen.encode_dense(W), oracle.encode(W)
    assert E.r == Eo.r and np.array_equal(E.Wd, Eo.Wd) and np.array_equal(E.idx, Eo.idx) and np.array_equal(E.nnz, Eo.nnz)


def test_datagen_gap_generator_is_a_valid_encoding(oracle):
    """uniform_ellpack builds ELLPACK arrays without the dense matrix: they must be exactly what
    the encoder makes of the matrix they describe, with the requested density."""
    import datagen
    E, x, b = datagen.uniform_ellpack(5, 300, 2000, 0.05)
    assert x.shape == (2000,) and b.shape == (300,)
    W = np.zeros((300, 2000), np.float32)
    for i in range(300):
        c = E.idx[i, :E.nnz[i]]
        assert (np.diff(c.astype(np.int64)) > 0).all() and (c < 2000).all()
        W[i, c] = E.Wd[i, :E.nnz[i]]
    Eo = oracle.encode(W)
    assert E.r == Eo.r and np.array_equal(E.Wd, Eo.Wd) and np.array_equal(E.idx, Eo.idx) and np.array_equal(E.nnz, Eo.nnz)
    assert abs(E.total_nnz / (300 * 2000) - 0.05) < 0.005


def test_benchmark_generator(backend):
    """sparseops_backend.benchmark_dense / benchmark_operand (bench/data_gen.hpp, the recipe of the reference's
    benchmark-mkl/common/data_gen.cpp:23-96): deterministic per seed, a Bernoulli(1 - sparsity) mask over N(0,1)
    values, a dense last row with `irregular`, operand uniform in [-1, 1)."""
    W = backend.benchmark_dense(300, 400, 0.9, 11, False)
    assert W.shape == (300, 400) and W.dtype == np.float32
    assert np.array_equal(W, backend.benchmark_dense(300, 400, 0.9, 11, False))
    assert not np.array_equal(W, backend.benchmark_dense(300, 400, 0.9, 12, False))
    kept = np.count_nonzero(W) / W.size
    assert abs(kept - 0.1) < 0.01
    vals = W[W != 0]
    assert abs(vals.mean()) < 0.05 and abs(vals.std() - 1.0) < 0.05
    Wi = backend.benchmark_dense(50, 64, 0.9, 3, True)
    assert np.count_nonzero(Wi[-1]) == 64 and np.count_nonzero(Wi[:-1]) < 0.2 * Wi[:-1].size
    assert np.count_nonzero(backend.benchmark_dense(16, 16, 1.0, 1, False)) == 0
    X = backend.benchmark_operand(128, 32, 5)
    assert X.shape == (128, 32) and X.min() >= -1.0 and X.max() < 1.0 and abs(X.mean()) < 0.05
    with pytest.raises(RuntimeError):
        backend.benchmark_dense(4, 4, 1.5, 1, False)
