"""The C-ABI library loads without a GPU, exports every symbol the header declares,
and reports a missing device as a status code (never an abort)."""
import ctypes as ct
import os
import re

import numpy as np
import pytest

from conftest import ROOT

import hipabi

HEADER = os.path.join(ROOT, "include", "sparseops_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(so_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = hipabi.load_library()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), "missing export: " + n
    assert sorted(hipabi.SYMBOLS) == names, "python binding and header disagree"


def test_header_is_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "sparseops_hip.h"\nint main(void){so_conv_geom g; (void)g; return SO_OK;}\n')
    import subprocess
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    "-c", str(src), "-o", str(tmp_path / "t.o")], check=True)


def has_gpu():
    lib = hipabi.load_library()
    n = ct.c_int()
    return lib.so_device_count(ct.byref(n)) == hipabi.SO_OK and n.value > 0


def test_no_device_is_a_status_not_a_crash():
    if has_gpu():
        pytest.skip("a GPU is present")
    lib = hipabi.load_library()
    n = ct.c_int(5)
    assert lib.so_device_count(ct.byref(n)) == hipabi.SO_ERR_NO_DEVICE and n.value == 0
    assert b"no HIP device" in lib.so_last_error()
    h = ct.c_void_p()
    assert lib.so_init(0, ct.byref(h)) == hipabi.SO_ERR_NO_DEVICE and not h.value
    with pytest.raises(hipabi.SoError) as e:
        hipabi.Context()
    assert e.value.status == hipabi.SO_ERR_NO_DEVICE


def test_null_arguments_are_rejected():
    lib = hipabi.load_library()
    assert lib.so_device_count(None) == hipabi.SO_ERR_INVALID
    assert lib.so_init(0, None) == hipabi.SO_ERR_INVALID
    assert lib.so_matmul(None, None, None, 1, None, None, 0) == hipabi.SO_ERR_INVALID
    assert lib.so_matvec(None, None, None, None, None, 0) == hipabi.SO_ERR_INVALID
    assert lib.so_sync(None) == hipabi.SO_ERR_INVALID
    assert lib.so_destroy(None) == hipabi.SO_OK and lib.so_ellpack_free(None, None) == hipabi.SO_OK


def test_backend_fails_loudly_without_device(backend):
    if has_gpu():
        pytest.skip("a GPU is present")
    assert backend.device_available() is False
    E = backend.convert_to_ellpack(np.eye(4, dtype=np.float32))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        backend.ellpack_matmul(E, np.ones((4, 2), np.float32), np.zeros(4, np.float32))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        backend.ellpack_matvec(E, np.ones(4, np.float32), np.zeros(4, np.float32))


def test_backend_argument_errors(backend):
    # src/bindings.cpp:116-124 of the reference: same checks, same exception type
    E = backend.convert_to_ellpack(np.eye(4, dtype=np.float32))
    with pytest.raises(RuntimeError, match="X must be 2D"):
        backend.ellpack_matmul(E, np.ones(4, np.float32), np.zeros(4, np.float32))
    with pytest.raises(RuntimeError, match="Input row count must equal E.n"):
        backend.ellpack_matmul(E, np.ones((5, 2), np.float32), np.zeros(4, np.float32))
    with pytest.raises(RuntimeError, match="Bias length must equal E.m"):
        backend.ellpack_matmul(E, np.ones((4, 2), np.float32), np.zeros(3, np.float32))
    with pytest.raises(RuntimeError, match="Input length must equal E.n"):
        backend.ellpack_matvec(E, np.ones(5, np.float32), np.zeros(4, np.float32))


def test_product_does_not_touch_the_oracle():
    """Nothing under sparse-ops_amd/ or include/ may reference oracle/."""
    bad = []
    for base in (os.path.join(ROOT, "sparse-ops_amd"), os.path.join(ROOT, "include")):
        for dp, _, files in os.walk(base):
            for f in files:
                if f.endswith((".py", ".cpp", ".hpp", ".h", ".hip", "Makefile")):
                    text = open(os.path.join(dp, f), errors="ignore").read()
                    if re.search(r"\boracle\b|liboracle|_ref/", text):
                        bad.append(os.path.join(dp, f))
    assert not bad, bad
