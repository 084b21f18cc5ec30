"""ctypes front-end to the CPU checkers.  TEST INFRASTRUCTURE ONLY.

`Oracle` wraps liboracle.so (oracle.c, this repository's restatement of the
reference's arithmetic); `Ref` wraps _ref/libsparseops_ref.so (the reference's
own kernels compiled from its sources by oracle/Makefile), when that library was
built and the host CPU has AVX-512F.  Only tests, the smoke check and the
benchmark's cpu_baseline leg may import this module; the shipped library never
does.
"""
import ctypes as ct
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ACT = {"none": 0, "relu": 1, "sigmoid": 2, "tanh": 3}

_f32p = ct.POINTER(ct.c_float)
_u32p = ct.POINTER(ct.c_uint32)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_f32p)


def _up(a):
    return a.ctypes.data_as(_u32p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def host_has_avx512f():
    try:
        with open("/proc/cpuinfo") as f:
            return " avx512f" in f.read()
    except OSError:
        return False


def build(with_ref=True):
    """(Re)build liboracle.so and, when the reference tree is present, _ref."""
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True, capture_output=True)
    if with_ref:
        subprocess.run(["make", "-C", _HERE, "ref"], check=True, capture_output=True)


class ConvGeom(ct.Structure):
    _fields_ = [(k, ct.c_uint32) for k in (
        "Cin", "Cout", "kH", "kW", "stride_h", "stride_w", "pad_h", "pad_w",
        "dil_h", "dil_w", "H_in", "W_in", "H_out", "W_out")]


class PoolGeom(ct.Structure):
    _fields_ = [(k, ct.c_uint32) for k in ("C", "H", "W", "H_out", "W_out")] + \
               [(k, ct.c_int32) for k in ("kH", "kW", "sH", "sW", "padH0", "padW0")]


def conv_geom(Cin, Cout, kH, kW, H, W, stride=(1, 1), pad=(0, 0), dil=(1, 1)):
    """Output size as the reference's loader computes it (src/sparse_onnx.cpp:428-429)."""
    Ho = (H + 2 * pad[0] - (dil[0] * (kH - 1) + 1)) // stride[0] + 1
    Wo = (W + 2 * pad[1] - (dil[1] * (kW - 1) + 1)) // stride[1] + 1
    return ConvGeom(Cin, Cout, kH, kW, stride[0], stride[1], pad[0], pad[1],
                    dil[0], dil[1], H, W, Ho, Wo)


class EllpackArrays:
    """Plain-array ELLPACK: Wd (m,r) f32, idx (m,r) u32, nnz (m,) u32."""

    def __init__(self, m, n, r, Wd, idx, nnz):
        self.m, self.n, self.r = int(m), int(n), int(r)
        self.Wd = np.ascontiguousarray(Wd, dtype=np.float32).reshape(self.m, self.r)
        self.idx = np.ascontiguousarray(idx, dtype=np.uint32).reshape(self.m, self.r)
        self.nnz = np.ascontiguousarray(nnz, dtype=np.uint32).reshape(self.m)

    @property
    def total_nnz(self):
        return int(self.nnz.sum(dtype=np.int64))


class RbmArrays:
    """build_rbm_from_ellpack's result (RBMPlan, include/rbm_conv.hpp:8-27) with the per-block vectors
    laid end to end: block b = rows [b*Ct_max, ...) owns union columns krel[block_union[b] :
    block_union[b+1]]; union column u owns pairs colptr[u] : colptr[u+1] (colptr made absolute over
    all blocks), pair p = (pair_row[p], pair_w[p])."""

    def __init__(self, M, N, Ct_max, block_union, krel, colptr, pair_row, pair_w):
        self.M, self.N, self.Ct_max = int(M), int(N), int(Ct_max)
        self.block_union = np.ascontiguousarray(block_union, dtype=np.uint32)
        self.krel = np.ascontiguousarray(krel, dtype=np.uint32)
        self.colptr = np.ascontiguousarray(colptr, dtype=np.uint32)
        self.pair_row = np.ascontiguousarray(pair_row, dtype=np.uint16)
        self.pair_w = np.ascontiguousarray(pair_w, dtype=np.float32)
        self.nblocks = len(self.block_union) - 1

    def same_as(self, o):
        return ((self.M, self.N, self.Ct_max) == (o.M, o.N, o.Ct_max) and
                all(np.array_equal(getattr(self, k), getattr(o, k))
                    for k in ("block_union", "krel", "colptr", "pair_row")) and
                np.array_equal(self.pair_w.view(np.uint32), o.pair_w.view(np.uint32)))


class Oracle:
    def __init__(self, path=None):
        path = path or os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build(with_ref=False)
        L = self.lib = ct.CDLL(path)
        L.orc_ellpack_count.restype = ct.c_uint32
        L.orc_ellpack_count.argtypes = [_f32p, ct.c_uint32, ct.c_uint32, _u32p]
        L.orc_ellpack_pack.argtypes = [_f32p, ct.c_uint32, ct.c_uint32, ct.c_uint32, _f32p, _u32p]
        L.orc_ellpack_decode.argtypes = [_f32p, _u32p, _u32p, ct.c_uint32, ct.c_uint32, ct.c_uint32, _f32p]
        L.orc_act.argtypes = [_f32p, ct.c_size_t, ct.c_int, _f32p]
        mm = [_f32p, _u32p, _u32p, ct.c_uint32, ct.c_uint32, ct.c_uint32, _f32p, ct.c_uint32, _f32p, ct.c_int, _f32p]
        L.orc_matmul.argtypes = mm
        L.orc_matmul_scalar.argtypes = mm
        L.orc_matvec.argtypes = [_f32p, _u32p, _u32p, ct.c_uint32, ct.c_uint32, ct.c_uint32, _f32p, _f32p, _f32p]
        L.orc_conv2d_pf.argtypes = [_f32p, _u32p, _u32p, ct.c_uint32, ct.POINTER(ConvGeom), _f32p,
                                    ct.c_uint32, _f32p, ct.c_int, _f32p]
        _u16p = ct.POINTER(ct.c_uint16)
        L.orc_rbm_build.argtypes = [_f32p, _u32p, _u32p, ct.c_uint32, ct.c_uint32, ct.c_uint32, _u32p, _u32p, _u32p,
                                    _u16p, _f32p, ct.POINTER(ct.c_uint64)]
        L.orc_conv2d_rbm_pf.argtypes = [_u32p, _u32p, _u32p, _u16p, _f32p, ct.c_uint32, ct.POINTER(ConvGeom), _f32p,
                                        ct.c_uint32, _f32p, ct.c_int, _f32p]
        L.orc_maxpool_pf.argtypes = [ct.POINTER(PoolGeom), _f32p, ct.c_uint32, _f32p]
        L.orc_gap_pf.argtypes = [ct.c_uint32, ct.c_uint32, ct.c_uint32, _f32p, ct.c_uint32, _f32p]
        L.orc_add.argtypes = [_f32p, _f32p, ct.c_size_t, _f32p]
        L.orc_num_threads.restype = ct.c_int
        L.orc_set_num_threads.argtypes = [ct.c_int]

    # -- encoder
    def encode(self, W):
        W = _f32(W)
        m, n = W.shape
        nnz = np.zeros(m, dtype=np.uint32)
        r = self.lib.orc_ellpack_count(_fp(W), m, n, _up(nnz)) if m else 0
        Wd = np.empty((m, r), dtype=np.float32)
        idx = np.empty((m, r), dtype=np.uint32)
        if m:
            self.lib.orc_ellpack_pack(_fp(W), m, n, r, _fp(Wd), _up(idx))
        return EllpackArrays(m, n, r, Wd, idx, nnz)

    def decode(self, E):
        W = np.empty((E.m, E.n), dtype=np.float32)
        self.lib.orc_ellpack_decode(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.m, E.n, E.r, _fp(W))
        return W

    # -- kernels
    def matmul(self, E, X, bias=None, act="none", scalar=False):
        X = _f32(X)
        C = X.shape[1]
        bias = None if bias is None else _f32(bias)
        Y = np.empty((E.m, C), dtype=np.float32)
        fn = self.lib.orc_matmul_scalar if scalar else self.lib.orc_matmul
        fn(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.m, E.n, E.r, _fp(X), C, _fp(bias), ACT[act], _fp(Y))
        return Y

    def matvec(self, E, x, bias=None):
        x = _f32(x)
        bias = None if bias is None else _f32(bias)
        y = np.empty(E.m, dtype=np.float32)
        self.lib.orc_matvec(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.m, E.n, E.r, _fp(x), _fp(bias), _fp(y))
        return y

    def act(self, x, act):
        x = _f32(x)
        y = np.empty_like(x)
        self.lib.orc_act(_fp(x), x.size, ACT[act], _fp(y))
        return y

    def conv2d_pf(self, E, g, X, B, bias=None, act="none"):
        """X: [Cin][H][W][B] flat; returns [Cout][Ho][Wo][B]."""
        X = _f32(X)
        bias = None if bias is None else _f32(bias)
        Y = np.empty((g.Cout, g.H_out, g.W_out, B), dtype=np.float32)
        self.lib.orc_conv2d_pf(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.r, ct.byref(g), _fp(X), B,
                               _fp(bias), ACT[act], _fp(Y))
        return Y

    def rbm_build(self, E, Ct_max=8):
        """build_rbm_from_ellpack restated (orc_rbm_build) -> RbmArrays."""
        nb = (E.m + Ct_max - 1) // Ct_max
        sizes = (ct.c_uint64 * 2)()
        bu = np.zeros(nb + 1, dtype=np.uint32)
        self.lib.orc_rbm_build(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.m, E.r, Ct_max, _up(bu), None, None, None, None, sizes)
        U, P = int(sizes[0]), int(sizes[1])
        krel, colptr = np.zeros(U, np.uint32), np.zeros(U + 1, np.uint32)
        prow, pw = np.zeros(P, np.uint16), np.zeros(P, np.float32)
        self.lib.orc_rbm_build(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.m, E.r, Ct_max, _up(bu), _up(krel), _up(colptr),
                               prow.ctypes.data_as(ct.POINTER(ct.c_uint16)), _fp(pw), sizes)
        return RbmArrays(E.m, E.n, Ct_max, bu, krel, colptr, prow, pw)

    def conv2d_rbm_pf(self, R, g, X, B, bias=None, act="none"):
        """conv2d_rbm_fmajor_implicit restated on [C][H][W][B] (orc_conv2d_rbm_pf)."""
        assert R.Ct_max <= 64
        X = _f32(X)
        bias = None if bias is None else _f32(bias)
        Y = np.empty((g.Cout, g.H_out, g.W_out, B), dtype=np.float32)
        self.lib.orc_conv2d_rbm_pf(_up(R.block_union), _up(R.krel), _up(R.colptr),
                                   R.pair_row.ctypes.data_as(ct.POINTER(ct.c_uint16)), _fp(R.pair_w), R.Ct_max,
                                   ct.byref(g), _fp(X), B, _fp(bias), ACT[act], _fp(Y))
        return Y

    def maxpool_pf(self, X, C, H, W, B, k, s, pad):
        X = _f32(X)
        Ho = (H + 2 * pad[0] - k[0]) // s[0] + 1
        Wo = (W + 2 * pad[1] - k[1]) // s[1] + 1
        p = PoolGeom(C, H, W, Ho, Wo, k[0], k[1], s[0], s[1], pad[0], pad[1])
        Y = np.empty((C, Ho, Wo, B), dtype=np.float32)
        self.lib.orc_maxpool_pf(ct.byref(p), _fp(X), B, _fp(Y))
        return Y

    def gap_pf(self, X, C, H, W, B):
        X = _f32(X)
        Y = np.empty((C, B), dtype=np.float32)
        self.lib.orc_gap_pf(C, H, W, _fp(X), B, _fp(Y))
        return Y

    def add(self, A, Bv):
        A, Bv = _f32(A), _f32(Bv)
        D = np.empty_like(A)
        self.lib.orc_add(_fp(A), _fp(Bv), A.size, _fp(D))
        return D

    def num_threads(self):
        return self.lib.orc_num_threads()

    def set_num_threads(self, n):
        self.lib.orc_set_num_threads(n)


class Ref:
    """The reference's own kernels (compiled from its sources).  `Ref.available()`
    says whether the library exists and this host can execute it."""

    PATH = os.path.join(_HERE, "_ref", "libsparseops_ref.so")

    @classmethod
    def available(cls):
        return os.path.exists(cls.PATH) and host_has_avx512f()

    def __init__(self):
        if not self.available():
            raise RuntimeError("reference library not built or host lacks avx512f")
        L = self.lib = ct.CDLL(self.PATH)
        L.ref_encode.restype = ct.c_void_p
        L.ref_encode.argtypes = [_f32p, ct.c_uint32, ct.c_uint32]
        L.ref_from_arrays.restype = ct.c_void_p
        L.ref_from_arrays.argtypes = [_f32p, _u32p, _u32p, ct.c_uint32, ct.c_uint32, ct.c_uint32]
        L.ref_free.argtypes = [ct.c_void_p]
        L.ref_dims.argtypes = [ct.c_void_p, _u32p, _u32p, _u32p]
        L.ref_copy.argtypes = [ct.c_void_p, _f32p, _u32p, _u32p]
        L.ref_decode.argtypes = [ct.c_void_p, _f32p]
        L.ref_matmul.argtypes = [ct.c_void_p, _f32p, ct.c_uint32, _f32p, _f32p]
        L.ref_matmul_fused.argtypes = [ct.c_void_p, _f32p, ct.c_uint32, _f32p, _f32p, ct.c_int, ct.c_int]
        L.ref_matvec.argtypes = [ct.c_void_p, _f32p, _f32p, _f32p]
        for nm in ("ref_relu_inplace", "ref_sigmoid_inplace", "ref_tanh_inplace"):
            getattr(L, nm).argtypes = [_f32p, ct.c_size_t]
        L.ref_conv.argtypes = [_f32p, _u32p, _f32p, ct.c_int, ct.c_int, _f32p, ct.c_uint32, _f32p]
        L.ref_conv_plan.restype = ct.c_void_p
        L.ref_conv_plan.argtypes = [_f32p, _u32p, _f32p, ct.c_int, ct.c_int]
        L.ref_conv_run.argtypes = [ct.c_void_p, _f32p, ct.c_uint32, _f32p]
        L.ref_conv_plan_free.argtypes = [ct.c_void_p]
        L.ref_rbm_sizes.argtypes = [ct.c_void_p, ct.c_uint32, _u32p]
        L.ref_rbm_copy.argtypes = [ct.c_void_p, ct.c_uint32, _u32p, _u32p, _u32p, ct.POINTER(ct.c_uint16), _f32p]

    class Handle:
        def __init__(self, lib, h):
            self.lib, self.h = lib, h
            m, n, r = ct.c_uint32(), ct.c_uint32(), ct.c_uint32()
            lib.ref_dims(h, ct.byref(m), ct.byref(n), ct.byref(r))
            self.m, self.n, self.r = m.value, n.value, r.value

        def __del__(self):
            if self.h:
                self.lib.ref_free(self.h)
                self.h = None

    def encode(self, W):
        W = _f32(W)
        return Ref.Handle(self.lib, self.lib.ref_encode(_fp(W), W.shape[0], W.shape[1]))

    def from_arrays(self, E):
        return Ref.Handle(self.lib, self.lib.ref_from_arrays(_fp(E.Wd), _up(E.idx), _up(E.nnz), E.m, E.n, E.r))

    def arrays(self, h):
        Wd = np.empty((h.m, h.r), dtype=np.float32)
        idx = np.empty((h.m, h.r), dtype=np.uint32)
        nnz = np.empty(h.m, dtype=np.uint32)
        self.lib.ref_copy(h.h, _fp(Wd), _up(idx), _up(nnz))
        return EllpackArrays(h.m, h.n, h.r, Wd, idx, nnz)

    def decode(self, h):
        W = np.empty((h.m, h.n), dtype=np.float32)
        self.lib.ref_decode(h.h, _fp(W))
        return W

    def matmul(self, h, X, bias=None, out=None):
        X = _f32(X)
        bias = None if bias is None else _f32(bias)
        Y = out if out is not None else np.empty((h.m, X.shape[1]), dtype=np.float32)
        self.lib.ref_matmul(h.h, _fp(X), X.shape[1], _fp(bias), _fp(Y))
        return Y

    def matmul_fused(self, h, X, bias=None, use_mask=True, fuse_relu=False):
        X = _f32(X)
        bias = None if bias is None else _f32(bias)
        Y = np.empty((h.m, X.shape[1]), dtype=np.float32)
        self.lib.ref_matmul_fused(h.h, _fp(X), X.shape[1], _fp(bias), _fp(Y), int(use_mask), int(fuse_relu))
        return Y

    def matvec(self, h, x, bias=None, out=None):
        x = _f32(x)
        bias = None if bias is None else _f32(bias)
        y = out if out is not None else np.empty(h.m, dtype=np.float32)
        self.lib.ref_matvec(h.h, _fp(x), _fp(bias), _fp(y))
        return y

    def act_inplace(self, x, act):
        y = _f32(x).copy()
        getattr(self.lib, "ref_%s_inplace" % act)(_fp(y), y.size)
        return y

    def rbm_build(self, h, Ct_max=8):
        """The reference's own build_rbm_from_ellpack on the handle's matrix -> RbmArrays."""
        sizes = np.zeros(3, dtype=np.uint32)
        self.lib.ref_rbm_sizes(h.h, Ct_max, _up(sizes))
        nb, U, P = (int(v) for v in sizes)
        bu, krel, colptr = np.zeros(nb + 1, np.uint32), np.zeros(U, np.uint32), np.zeros(U + 1, np.uint32)
        prow, pw = np.zeros(P, np.uint16), np.zeros(P, np.float32)
        self.lib.ref_rbm_copy(h.h, Ct_max, _up(bu), _up(krel), _up(colptr), prow.ctypes.data_as(ct.POINTER(ct.c_uint16)), _fp(pw))
        return RbmArrays(h.m, h.n, Ct_max, bu, krel, colptr, prow, pw)

    def conv(self, Wdense, g, src, B, bias=None, fuse_relu=False, variant=0):
        Wdense, src = _f32(Wdense), _f32(src)
        bias = None if bias is None else _f32(bias)
        geom = np.array([getattr(g, k) for k, _ in ConvGeom._fields_], dtype=np.uint32)
        dst = np.empty(g.Cout * g.H_out * g.W_out * B, dtype=np.float32)
        self.lib.ref_conv(_fp(Wdense), _up(geom), _fp(bias), int(fuse_relu), variant, _fp(src), B, _fp(dst))
        return dst

    def conv_plan(self, Wdense, g, bias=None, fuse_relu=False, variant=0):
        """The load-time part of a convolution layer (encode, kmap, RBM plan) -> a handle for conv_run."""
        Wdense = _f32(Wdense)
        bias = None if bias is None else _f32(bias)
        geom = np.array([getattr(g, k) for k, _ in ConvGeom._fields_], dtype=np.uint32)
        return self.lib.ref_conv_plan(_fp(Wdense), _up(geom), _fp(bias), int(fuse_relu), variant)

    def conv_run(self, plan, g, src, B, out=None):
        src = _f32(src)
        dst = out if out is not None else np.empty(g.Cout * g.H_out * g.W_out * B, dtype=np.float32)
        self.lib.ref_conv_run(plan, _fp(src), B, _fp(dst))
        return dst

    def conv_plan_free(self, plan):
        self.lib.ref_conv_plan_free(plan)
