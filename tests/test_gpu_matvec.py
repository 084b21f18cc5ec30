"""so_matvec (all three device layouts) and sparseops_backend.ellpack_matvec on the
GPU.  The in-row summation order differs from the reference's (wave reduction vs.
16 interleaved partials), so the bar is the fp32 tolerance: max|y - ref| / max|ref|
<= 1e-5 against both the fp64 product and the oracle."""
import numpy as np
import pytest

from conftest import as_oracle, rel_err, sparse_matrix
from test_oracle_kernels import MATVEC_CASES

import datagen
import hipabi

pytestmark = pytest.mark.gpu
TOL = 1e-5
ALL = hipabi.LAYOUT_ROW | hipabi.LAYOUT_SLOT | hipabi.LAYOUT_BINS


def gpu_matvec(ctx, E, x, bias, layouts=ALL, which=(hipabi.LAYOUT_ROW, hipabi.LAYOUT_SLOT, hipabi.LAYOUT_BINS, 0)):
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, layouts)
    dx, dy = ctx.array(x), ctx.empty((E.m,))
    dB = ctx.array(bias) if bias is not None else None
    out = {}
    for lay in which:
        dy.upload(np.full(E.m, np.nan, np.float32))      # every row must be written
        ctx.matvec(dE, dx, dB, dy, lay)
        out[lay] = dy.download()
    dE.free()
    return out


@pytest.mark.parametrize("m,n,sp", MATVEC_CASES + [(257, 4097, .5), (5000, 64, .2), (100, 50000, .99)])
def test_matvec_all_layouts(ctx, oracle, m, n, sp):
    rng = np.random.default_rng(m * 13 + n)
    W = sparse_matrix(rng, m, n, sp)
    x = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    E = datagen.encode_dense(W)
    y64 = W.astype(np.float64) @ x + b
    yo = oracle.matvec(as_oracle(E), x, b)
    for lay, y in gpu_matvec(ctx, E, x, b).items():
        assert y.shape == (m,)
        assert rel_err(y, y64) <= TOL, lay
        assert rel_err(y, yo) <= TOL, lay
    for lay, y in gpu_matvec(ctx, E, x, None, which=(hipabi.LAYOUT_ROW, hipabi.LAYOUT_BINS)).items():
        assert rel_err(y, W.astype(np.float64) @ x) <= TOL, lay


def test_matvec_every_row_written_once(ctx):
    """Binned launches must cover every row exactly once: y starts as NaN."""
    rng = np.random.default_rng(3)
    counts = np.minimum(rng.zipf(1.3, size=3000), 400)
    n = 1000
    cols = [np.sort(rng.permutation(n)[:k]).astype(np.uint32) for k in counts]
    vals = [rng.standard_normal(k).astype(np.float32) for k in counts]
    E = datagen.rows_to_ellpack(3000, n, cols, vals)
    x = rng.standard_normal(n).astype(np.float32)
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, ALL)
    dx = ctx.array(x)
    W = np.zeros((3000, n))
    for i in range(3000):
        W[i, cols[i]] = vals[i]
    for lay in (hipabi.LAYOUT_ROW, hipabi.LAYOUT_SLOT, hipabi.LAYOUT_BINS):
        dy = ctx.array(np.full(3000, np.nan, np.float32))
        ctx.matvec(dE, dx, None, dy, lay)
        y = dy.download()
        assert np.isfinite(y).all(), lay
        assert rel_err(y, W @ x) <= TOL, lay


@pytest.mark.parametrize("lanes", [8, 16, 32, 64])
@pytest.mark.parametrize("m,n,kmax", [(3001, 1000, 203), (517, 4099, 700), (64, 300, 17), (70000, 256, 40)])
def test_matvec_rows_lanes_per_row(ctx, lanes, m, n, kmax):
    """The row kernel shares a row among 8, 16, 32 or 64 lanes (picked by the longest row and the
    row count; forced here): ragged rows including empty ones, odd r, rows longer than one pass."""
    rng = np.random.default_rng(lanes + m)
    counts = rng.integers(0, kmax + 1, size=m)
    counts[::7] = 0
    counts[1] = kmax
    cols = [np.sort(rng.choice(n, size=k, replace=False)).astype(np.uint32) for k in counts]
    vals = [rng.standard_normal(k).astype(np.float32) for k in counts]
    E = datagen.rows_to_ellpack(m, n, cols, vals)
    assert E.r == kmax
    x = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    y64 = b.astype(np.float64)
    for i in range(m):
        y64[i] += vals[i].astype(np.float64) @ x[cols[i]]
    with ctx.tuning(SPARSEOPS_MATVEC_LANES=lanes):
        y = gpu_matvec(ctx, E, x, b, layouts=hipabi.LAYOUT_ROW, which=(hipabi.LAYOUT_ROW,))[hipabi.LAYOUT_ROW]
    assert np.isfinite(y).all()
    assert rel_err(y, y64) <= TOL
    y_auto = gpu_matvec(ctx, E, x, b, layouts=hipabi.LAYOUT_ROW, which=(hipabi.LAYOUT_ROW,))[hipabi.LAYOUT_ROW]
    assert rel_err(y_auto, y64) <= TOL


def test_matvec_reference_vectors(ctx, golden):
    E = datagen.encode_dense(golden["enc_W"])
    for lay, y in gpu_matvec(ctx, E, golden["mv_x"], golden["mm_bias"]).items():
        assert rel_err(y, golden["mv_y"]) <= TOL, lay


def test_matvec_padding_is_not_read(ctx):
    W = np.zeros((5, 8), np.float32)
    W[0, 1:7] = 1
    W[2, 3] = 2
    x = np.ones(8, np.float32)
    x[0] = np.inf
    for lay, y in gpu_matvec(ctx, datagen.encode_dense(W), x, None).items():
        assert np.array_equal(y, [6, 0, 2, 0, 0]), lay


def test_matvec_config2a_and_2b(ctx, oracle):
    """Full-size configurations: 16384 x 16384 at 95 % uniform sparsity, and the
    skewed variant with Zipf(1.2) row lengths clipped at 2048."""
    E, x, b = datagen.config2a()
    assert 880 < E.r < 1000 and abs(E.total_nnz - 0.05 * 16384 ** 2) < 5e4
    yo = oracle.matvec(as_oracle(E), x, b)
    for lay, y in gpu_matvec(ctx, E, x, b, layouts=hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS,
                             which=(hipabi.LAYOUT_ROW, hipabi.LAYOUT_BINS)).items():
        assert rel_err(y, yo) <= TOL, lay
    E, x, b = datagen.config2b()
    assert E.r == 2048 and E.total_nnz < E.m * E.r // 3
    yo = oracle.matvec(as_oracle(E), x, b)
    for lay, y in gpu_matvec(ctx, E, x, b, layouts=hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS,
                             which=(hipabi.LAYOUT_ROW, hipabi.LAYOUT_BINS, 0)).items():
        assert rel_err(y, yo) <= TOL, lay
    # linearity in x is size-independent: E(2x) = 2 E(x) exactly (scaling by 2 is exact in fp32)
    y1 = gpu_matvec(ctx, E, x, None, layouts=hipabi.LAYOUT_BINS, which=(hipabi.LAYOUT_BINS,))[hipabi.LAYOUT_BINS]
    y2 = gpu_matvec(ctx, E, 2 * x, None, layouts=hipabi.LAYOUT_BINS, which=(hipabi.LAYOUT_BINS,))[hipabi.LAYOUT_BINS]
    assert np.array_equal(y2, 2 * y1)


def test_matvec_degenerate(ctx):
    E = datagen.encode_dense(np.zeros((0, 0), np.float32))
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, 0, 0, 0, ALL)
    ctx.matvec(dE, ctx.empty((0,)), None, ctx.empty((0,)), 0)          # no launch, no error
    E = datagen.encode_dense(np.zeros((32, 32), np.float32))
    b = np.arange(32, dtype=np.float32)
    for lay, y in gpu_matvec(ctx, E, np.ones(32, np.float32), b).items():
        assert np.array_equal(y, b), lay
    with pytest.raises(hipabi.SoError):
        dE2 = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, 32, 32, 0, hipabi.LAYOUT_ROW)
        ctx.matvec(dE2, ctx.empty((32,)), None, ctx.empty((32,)), hipabi.LAYOUT_SLOT)   # layout not uploaded


# ---- columns in 16 bits (SO_LAYOUT_IDX16): same kernels, 6 bytes per nonzero, same bits

def both_column_widths(ctx, E, x, b, layouts, which):
    """y from the handle's 16-bit columns and, on the same handle, from its 32-bit ones."""
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, layouts | hipabi.LAYOUT_IDX16)
    assert dE.layouts() & hipabi.LAYOUT_IDX16
    dx, dy = ctx.array(x), ctx.empty((E.m,))
    dB = ctx.array(b) if b is not None else None
    out = {}
    for lay in which:
        dy.upload(np.full(E.m, np.nan, np.float32))
        ctx.matvec(dE, dx, dB, dy, lay)
        y16 = dy.download()
        with ctx.tuning(SPARSEOPS_MATVEC_IDX16="0"):
            dy.upload(np.full(E.m, np.nan, np.float32))
            ctx.matvec(dE, dx, dB, dy, lay)
        out[lay] = (y16, dy.download())
    # the 32-bit arrays are untouched: the download is still the upload
    Wd, idx, nnz = dE.download(hipabi.LAYOUT_ROW)
    assert np.array_equal(Wd.view(np.uint32), E.Wd.view(np.uint32)) and np.array_equal(idx, E.idx) and np.array_equal(nnz, E.nnz)
    dE.free()
    return out


@pytest.mark.parametrize("lanes", [0, 8, 16, 32, 64])
@pytest.mark.parametrize("m,n,kmax", [(3001, 1000, 203), (517, 65536, 1300), (64, 300, 17), (20000, 256, 40), (300, 40000, 2600)])
def test_matvec_16_bit_columns(ctx, lanes, m, n, kmax):
    """Ragged rows (empty ones, odd r, rows of several passes, columns up to 65535) through the row kernel at
    every lanes-per-row setting, through the binned kernel and the lane-per-row kernel: the 16-bit columns give the bits of the 32-bit ones."""
    rng = np.random.default_rng(lanes * 7 + m)
    counts = np.minimum(rng.zipf(1.3, size=m) * 3, kmax)
    counts[::7] = 0
    counts[1] = kmax
    cols = [np.sort(rng.choice(n, size=k, replace=False)).astype(np.uint32) for k in counts]
    cols[1][-1] = n - 1                                    # the last column is used (65535 when n = 65536)
    if kmax > 1:
        cols[1][-2] = min(cols[1][-2], n - 2)
    vals = [rng.standard_normal(k).astype(np.float32) for k in counts]
    E = datagen.rows_to_ellpack(m, n, cols, vals)
    x = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    y64 = b.astype(np.float64)
    for i in range(m):
        y64[i] += vals[i].astype(np.float64) @ x[cols[i]]
    with ctx.tuning(SPARSEOPS_MATVEC_LANES=lanes or None):
        res = both_column_widths(ctx, E, x, b, ALL, (hipabi.LAYOUT_ROW, hipabi.LAYOUT_BINS, hipabi.LAYOUT_SLOT, 0))
    for lay, (y16, y32) in res.items():
        assert np.isfinite(y16).all(), lay
        if lay:                                # left to itself (0) the library may take another kernel on 16-bit columns
            assert np.array_equal(y16, y32), lay
        assert rel_err(y16, y64) <= TOL and rel_err(y32, y64) <= TOL, lay


def test_matvec_16_bit_columns_full_size(ctx, oracle):
    """Configurations 2a and 2b with the compact columns: the oracle's result within tolerance, the 32-bit
    kernels' bits."""
    for gen, layouts, which in ((datagen.config2a, hipabi.LAYOUT_ROW, (hipabi.LAYOUT_ROW,)),
                                (datagen.config2b, hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS, (hipabi.LAYOUT_BINS, hipabi.LAYOUT_ROW))):
        E, x, b = gen()
        yo = oracle.matvec(as_oracle(E), x, b)
        for lay, (y16, y32) in both_column_widths(ctx, E, x, b, layouts, which).items():
            assert np.array_equal(y16, y32), lay
            assert rel_err(y16, yo) <= TOL, lay


def test_matvec_16_bit_columns_need_few_columns(ctx):
    W = np.zeros((4, 65537), np.float32)
    W[2, 65536] = 1.0
    E = datagen.encode_dense(W)
    with pytest.raises(hipabi.SoError, match="65536"):
        ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, hipabi.LAYOUT_ROW | hipabi.LAYOUT_IDX16)
    # without the flag the same matrix is fine, and an empty one takes the flag
    y = gpu_matvec(ctx, E, np.arange(65537, dtype=np.float32), None, layouts=hipabi.LAYOUT_ROW, which=(hipabi.LAYOUT_ROW,))
    assert np.array_equal(y[hipabi.LAYOUT_ROW], [0, 0, 65536, 0])
    E0 = datagen.encode_dense(np.zeros((3, 5), np.float32))
    dE = ctx.upload_ellpack(E0.Wd, E0.idx, E0.nnz, 3, 5, E0.r, hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS | hipabi.LAYOUT_IDX16)
    dy = ctx.array(np.full(3, np.nan, np.float32))
    ctx.matvec(dE, ctx.array(np.ones(5, np.float32)), None, dy, 0)
    assert np.array_equal(dy.download(), [0, 0, 0])
    dE.free()


@pytest.mark.parametrize("n,long_rows", [(20000, (20000, 4097, 9000)), (70000, (70000, 33000)), (5000, (5000,) * 40)])
def test_matvec_binned_very_long_rows(ctx, n, long_rows):
    """Rows of more than 4096 nonzeros get a whole workgroup in the binned kernel (16 waves share the row, their
    partial sums meet in LDS): a few such rows among short ones, a fully dense row, more such rows than the launch
    has workgroups for them at once would need, x staged in LDS or not, both column widths."""
    rng = np.random.default_rng(n)
    m = 700
    counts = np.minimum(rng.zipf(1.4, size=m) * 2, 300)
    counts[::9] = 0
    where = rng.choice(m, size=len(long_rows), replace=False)
    counts[where] = long_rows
    cols = [np.sort(rng.choice(n, size=k, replace=False)).astype(np.uint32) for k in counts]
    vals = [rng.standard_normal(k).astype(np.float32) for k in counts]
    E = datagen.rows_to_ellpack(m, n, cols, vals)
    x = rng.standard_normal(n).astype(np.float32)
    b = rng.standard_normal(m).astype(np.float32)
    y64 = b.astype(np.float64)
    for i in range(m):
        y64[i] += vals[i].astype(np.float64) @ x[cols[i]]
    lay = hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS
    if n <= 65536:
        for which, (y16, y32) in both_column_widths(ctx, E, x, b, lay, (hipabi.LAYOUT_BINS, hipabi.LAYOUT_ROW)).items():
            assert np.isfinite(y16).all() and np.array_equal(y16, y32), which
            assert rel_err(y16, y64) <= TOL, which
    else:
        for which, y in gpu_matvec(ctx, E, x, b, layouts=lay, which=(hipabi.LAYOUT_BINS, hipabi.LAYOUT_ROW)).items():
            assert np.isfinite(y).all() and rel_err(y, y64) <= TOL, which
    # the same launch twice gives the same bits (the partial sums are added in a fixed order)
    y1 = gpu_matvec(ctx, E, x, b, layouts=lay, which=(hipabi.LAYOUT_BINS,))[hipabi.LAYOUT_BINS]
    y2 = gpu_matvec(ctx, E, x, b, layouts=lay, which=(hipabi.LAYOUT_BINS,))[hipabi.LAYOUT_BINS]
    assert np.array_equal(y1, y2)


# ---- the drop-in module: the reference's unit cases (tests/unit/test_matvec.py:12-46), seeded

@pytest.mark.parametrize("m,n,sp", MATVEC_CASES)
def test_backend_matvec(backend, m, n, sp):
    rng = np.random.default_rng(m + n)
    W = sparse_matrix(rng, m, n, sp, signed=False)
    E = backend.convert_to_ellpack(W)
    x = rng.random(n).astype(np.float32)
    b = rng.random(m).astype(np.float32)
    y = backend.ellpack_matvec(E, x, b)
    assert y.shape == (m,)
    y64 = W.astype(np.float64) @ x + b
    assert rel_err(y, y64) <= TOL
    assert np.allclose(y, y64, rtol=1e-5, atol=1e-5 * max(1.0, np.abs(y64).max() if m else 1.0))
    if m:
        assert rel_err(backend.ellpack_matvec(E, x, None), W.astype(np.float64) @ x) <= TOL


def test_backend_matvec_skewed(backend):
    rng = np.random.default_rng(11)
    W = sparse_matrix(rng, 800, 900, .995)
    W[7] = rng.standard_normal(900)                 # one dense row: r = 900, mean nnz ~ 5
    E = backend.convert_to_ellpack(W)
    x = rng.standard_normal(900).astype(np.float32)
    assert rel_err(backend.ellpack_matvec(E, x, None), W.astype(np.float64) @ x) <= TOL
