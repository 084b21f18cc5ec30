"""bench/bench_vendor -- the counterpart of the reference's benchmark-mkl drivers
(benchmark-mkl/matmul/main_matmul.cpp:49-139, matvec/main_matvec.cpp:49-132) -- runs on the GPU
and every comparator (this library's kernels, rocSPARSE CSR, rocBLAS dense) agrees with so_matmul /
so_matvec to 1e-5 of the largest output (the reference's own harness prints the same kind of
difference and asserts nothing; 1e-5 is its unit tests' tolerance, tests/unit/test_matmul.py:48)."""

import os
import re
import subprocess

import numpy as np
import pytest

import datagen

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "sparse-ops_amd", "bench", "bench_vendor")
DIFF = re.compile(r"max rel diff(?: vs so_\w+)? ([0-9.e+-]+)\s*$")
TOL = 1e-5


def run_vendor(args):
    out = subprocess.run([BIN] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    assert out.returncode == 0, out.stdout
    diffs = [float(m.group(1)) for m in map(DIFF.search, out.stdout.splitlines()) if m]
    return out.stdout, diffs


@pytest.mark.parametrize("irregular", [0, 1])
def test_vendor_matmul(irregular):
    text, diffs = run_vendor(["matmul", "--M", "384", "--N", "512", "--C", "64", "--sparsity", "0.9", "--runs", "3",
                              "--seed", "7", "--irregular", str(irregular)])
    assert len(diffs) >= 4, text               # two of ours, at least one rocSPARSE algorithm, rocBLAS
    assert "rocBLAS dense SGEMM" in text and "rocSPARSE CSR SpMM" in text
    assert max(diffs) <= TOL, text
    if irregular:
        assert "ELLPACK r 512" in text         # the dense last row sets r


@pytest.mark.parametrize("irregular", [0, 1])
def test_vendor_matvec(irregular):
    text, diffs = run_vendor(["matvec", "--M", "1024", "--N", "768", "--sparsity", "0.95", "--runs", "3", "--seed", "9",
                              "--irregular", str(irregular)])
    assert len(diffs) >= 4, text
    assert "rocBLAS dense SGEMV" in text and "rocSPARSE CSR SpMV" in text
    assert max(diffs) <= TOL, text


def test_vendor_runs_a_datagen_matrix(tmp_path):
    """--ellpack-file: the benchmark configurations' generator (per-row top-k, as config 3) feeds the harness."""
    E, _, _ = datagen.config3(m=256, n=320, C=64)
    path = str(tmp_path / "m.ellpack")
    datagen.save_ellpack(path, E)
    back = datagen.load_ellpack(path)
    assert (back.m, back.n, back.r) == (E.m, E.n, E.r) and np.array_equal(back.idx, E.idx) and np.array_equal(back.Wd, E.Wd)
    text, diffs = run_vendor(["matmul", "--ellpack-file", path, "--C", "64", "--runs", "3"])
    assert "Matrix dims:     256 x 320" in text and "nnz %d, ELLPACK r %d" % (E.total_nnz, E.r) in text
    assert len(diffs) >= 4 and max(diffs) <= TOL, text
    text, diffs = run_vendor(["matvec", "--ellpack-file", path, "--runs", "3"])
    assert len(diffs) >= 4 and max(diffs) <= TOL, text


@pytest.mark.parametrize("irregular", [0, 1])
def test_vendor_and_python_draw_the_same_matrix(irregular):
    """One generator (bench/data_gen.hpp) behind the harness and sparseops_backend.benchmark_dense:
    the same seed gives the same matrix, so the harness's nnz and ELLPACK r are those of the Python side's."""
    import sparseops_backend as sb
    W = sb.benchmark_dense(384, 512, 0.9, 7, bool(irregular))
    E = datagen.encode_dense(W)
    text, _ = run_vendor(["matmul", "--M", "384", "--N", "512", "--C", "64", "--sparsity", "0.9", "--runs", "2",
                          "--seed", "7", "--irregular", str(irregular)])
    assert "nnz %d, ELLPACK r %d" % (np.count_nonzero(W), E.r) in text, text
