"""ctypes binding of the C ABI of libsparseops_hip.so (include/sparseops_hip.h).

This is the stub a maintainer of a Python caller would write; the tests and the
benchmark drive the HIP kernels through it with device-resident operands.
"""
import contextlib
import ctypes as ct
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libsparseops_hip.so")

SO_OK, SO_ERR_NO_DEVICE, SO_ERR_INVALID, SO_ERR_OOM, SO_ERR_HIP, SO_ERR_BOUNDS = range(6)
ACT = {"none": 0, "relu": 1, "sigmoid": 2, "tanh": 3}
LAYOUT_ROW, LAYOUT_SLOT, LAYOUT_BINS, LAYOUT_TILED, LAYOUT_RBM, LAYOUT_IDX16 = 1, 2, 4, 8, 16, 32

# Every symbol include/sparseops_hip.h declares.
SYMBOLS = (
    "so_device_count so_init so_destroy so_last_error so_device_info so_tuning_reload so_malloc so_free so_h2d so_d2h "
    "so_d2d so_fill_zero so_sync so_timer_begin so_timer_end so_ellpack_upload so_ellpack_free "
    "so_ellpack_dims so_ellpack_download so_ellpack_decode so_ellpack_encode so_ellpack_encode_noalloc so_matmul so_matmul_reserve so_matvec so_conv_plan_create so_conv_plan_free so_conv_plan_window so_conv_plan_tune so_conv2d_add "
    "so_conv2d so_maxpool so_gap so_add so_act so_transpose so_reverse_axes3 so_copy_rows so_graph_begin so_graph_end "
    "so_graph_launch so_graph_free so_rbm_upload so_rbm_free so_rbm_dims so_conv_plan_set_rbm so_conv_plan_rbm_info").split()

_vp = ct.c_void_p
_u32 = ct.c_uint32


class ConvGeom(ct.Structure):
    _fields_ = [(k, _u32) for k in (
        "Cin", "Cout", "kH", "kW", "stride_h", "stride_w", "pad_h", "pad_w",
        "dil_h", "dil_w", "H_in", "W_in", "H_out", "W_out")]


class PoolGeom(ct.Structure):
    _fields_ = [(k, _u32) for k in ("C", "H", "W", "H_out", "W_out")] + \
               [(k, ct.c_int32) for k in ("kH", "kW", "sH", "sW", "padH0", "padW0")]


def conv_geom(Cin, Cout, kH, kW, H, W, stride=(1, 1), pad=(0, 0), dil=(1, 1)):
    Ho = (H + 2 * pad[0] - (dil[0] * (kH - 1) + 1)) // stride[0] + 1
    Wo = (W + 2 * pad[1] - (dil[1] * (kW - 1) + 1)) // stride[1] + 1
    return ConvGeom(Cin, Cout, kH, kW, stride[0], stride[1], pad[0], pad[1], dil[0], dil[1], H, W, Ho, Wo)


class SoError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("so_status %d: %s" % (status, message))
        self.status = status


def load_library(path=None):
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise FileNotFoundError("libsparseops_hip.so is not built: %s (run __graft_entry__.build())" % path)
    lib = ct.CDLL(path)
    lib.so_last_error.restype = ct.c_char_p
    sig = {
        "so_device_count": [ct.POINTER(ct.c_int)],
        "so_init": [ct.c_int, ct.POINTER(_vp)],
        "so_destroy": [_vp],
        "so_device_info": [_vp, ct.c_char_p, ct.c_size_t, ct.POINTER(ct.c_int)],
        "so_tuning_reload": [_vp],
        "so_malloc": [_vp, ct.c_size_t, ct.POINTER(_vp)],
        "so_free": [_vp, _vp],
        "so_h2d": [_vp, _vp, _vp, ct.c_size_t],
        "so_d2h": [_vp, _vp, _vp, ct.c_size_t],
        "so_d2d": [_vp, _vp, _vp, ct.c_size_t],
        "so_fill_zero": [_vp, _vp, ct.c_size_t],
        "so_sync": [_vp],
        "so_timer_begin": [_vp],
        "so_timer_end": [_vp, ct.POINTER(ct.c_float)],
        "so_ellpack_upload": [_vp, _vp, _vp, _vp, _u32, _u32, _u32, ct.c_int, ct.POINTER(_vp)],
        "so_ellpack_free": [_vp, _vp],
        "so_ellpack_dims": [_vp, ct.POINTER(_u32), ct.POINTER(_u32), ct.POINTER(_u32),
                            ct.POINTER(ct.c_uint64), ct.POINTER(ct.c_int)],
        "so_ellpack_download": [_vp, _vp, ct.c_int, _vp, _vp, _vp],
        "so_ellpack_decode": [_vp, _vp, _vp],
        "so_ellpack_encode": [_vp, _vp, _u32, _u32, ct.POINTER(_vp)],
        "so_ellpack_encode_noalloc": [_vp, _vp, _u32, _u32, _u32, _vp, _vp, _vp, ct.POINTER(_u32), ct.POINTER(ct.c_uint64)],
        "so_matmul": [_vp, _vp, _vp, _u32, _vp, _vp, ct.c_int],
        "so_matmul_reserve": [_vp, _vp, _u32],
        "so_matvec": [_vp, _vp, _vp, _vp, _vp, ct.c_int],
        "so_conv_plan_create": [_vp, _vp, ct.POINTER(ConvGeom), ct.POINTER(_vp)],
        "so_conv_plan_free": [_vp, _vp],
        "so_conv_plan_window": [_vp, ct.POINTER(ct.c_uint32)],
        "so_conv_plan_tune": [_vp, _vp, ct.c_uint32],
        "so_conv2d": [_vp, _vp, _vp, _u32, _vp, _vp, ct.c_int],
        "so_conv2d_add": [_vp, _vp, _vp, ct.c_uint32, _vp, _vp, _vp, ct.c_int],
        "so_maxpool": [_vp, ct.POINTER(PoolGeom), _vp, _u32, _vp],
        "so_gap": [_vp, _u32, _u32, _u32, _vp, _u32, _vp],
        "so_add": [_vp, _vp, _vp, ct.c_size_t, _vp],
        "so_act": [_vp, ct.c_int, _vp, ct.c_size_t, _vp],
        "so_transpose": [_vp, _vp, _u32, _u32, _vp],
        "so_reverse_axes3": [_vp, _vp, _u32, _u32, _u32, _u32, _vp],
        "so_copy_rows": [_vp, _vp, ct.c_size_t, _u32, _u32, _vp, ct.c_size_t, ct.c_int],
        "so_graph_begin": [_vp],
        "so_graph_end": [_vp, ct.POINTER(_vp)],
        "so_graph_launch": [_vp, _vp],
        "so_graph_free": [_vp, _vp],
        "so_rbm_upload": [_vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, ct.POINTER(_vp)],
        "so_rbm_free": [_vp, _vp],
        "so_rbm_dims": [_vp, ct.POINTER(_u32), ct.POINTER(_u32), ct.POINTER(_u32), ct.POINTER(_u32),
                        ct.POINTER(ct.c_uint64), ct.POINTER(ct.c_uint64)],
        "so_conv_plan_set_rbm": [_vp, _vp, _vp],
        "so_conv_plan_rbm_info": [_vp, ct.POINTER(ct.c_uint64)],
    }
    for name, argtypes in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ct.c_int
    return lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_vp)


class DeviceArray:
    """A float32/uint32 array in HBM, owned by a Context."""

    def __init__(self, ctx, shape, dtype=np.float32):
        self.ctx, self.shape, self.dtype = ctx, tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = _vp()
        ctx._ck(ctx.lib.so_malloc(ctx.h, self.nbytes, ct.byref(p)))
        self.ptr = p.value

    def upload(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        assert host.nbytes == self.nbytes, (host.shape, self.shape)
        self.ctx._ck(self.ctx.lib.so_h2d(self.ctx.h, self.ptr, _ptr(host), self.nbytes))
        return self

    def download(self):
        out = np.empty(self.shape, dtype=self.dtype)
        self.ctx._ck(self.ctx.lib.so_d2h(self.ctx.h, _ptr(out), self.ptr, self.nbytes))
        return out

    def offset(self, elems):
        """A view of the flattened array that starts `elems` elements in; it does not own the memory."""
        total = self.nbytes // self.dtype.itemsize
        assert 0 <= elems <= total
        v = object.__new__(DeviceArray)
        v.ctx, v.shape, v.dtype = self.ctx, (total - elems,), self.dtype
        v.nbytes = (total - elems) * self.dtype.itemsize
        v.ptr = self.ptr + elems * self.dtype.itemsize
        v._view = True
        return v

    def free(self):
        if self.ptr and not getattr(self, "_view", False):
            self.ctx.lib.so_free(self.ctx.h, self.ptr)
        self.ptr = None


class DeviceEllpack:
    def __init__(self, ctx, handle, m, n, r):
        self.ctx, self.h, self.m, self.n, self.r = ctx, handle, m, n, r

    def decode(self):
        """-> the dense (m, n) matrix, decoded on the device."""
        dW = self.ctx.empty((self.m, self.n))
        self.ctx._ck(self.ctx.lib.so_ellpack_decode(self.ctx.h, self.h, dW.ptr))
        W = dW.download()
        dW.free()
        return W

    def layouts(self):
        """The mask of SO_LAYOUT_* the handle holds (so_ellpack_dims)."""
        lay = ct.c_int()
        self.ctx._ck(self.ctx.lib.so_ellpack_dims(self.h, None, None, None, None, ct.byref(lay)))
        return lay.value

    def download(self, layout=LAYOUT_ROW):
        shape = (self.m, self.r) if layout == LAYOUT_ROW else (self.r, self.m)
        Wd = np.empty(shape, dtype=np.float32)
        idx = np.empty(shape, dtype=np.uint32)
        nnz = np.empty(self.m, dtype=np.uint32)
        self.ctx._ck(self.ctx.lib.so_ellpack_download(self.ctx.h, self.h, layout, _ptr(Wd), _ptr(idx), _ptr(nnz)))
        return Wd, idx, nnz

    def free(self):
        if self.h:
            self.ctx.lib.so_ellpack_free(self.ctx.h, self.h)
            self.h = None


class Context:
    """One so_ctx.  Raises SoError(SO_ERR_NO_DEVICE) when no GPU is usable."""

    def __init__(self, device=0, lib=None):
        self.lib = lib or load_library()
        h = _vp()
        self.h = None
        self._ck(self.lib.so_init(device, ct.byref(h)))
        self.h = h.value

    def _ck(self, status):
        if status != SO_OK:
            raise SoError(status, self.lib.so_last_error().decode())

    def close(self):
        if self.h:
            self.lib.so_destroy(self.h)
            self.h = None

    def info(self):
        name = ct.create_string_buffer(64)
        cus = ct.c_int()
        self._ck(self.lib.so_device_info(self.h, name, 64, ct.byref(cus)))
        return name.value.decode(), cus.value

    def array(self, host, dtype=np.float32):
        host = np.ascontiguousarray(host, dtype=dtype)
        return DeviceArray(self, host.shape, dtype).upload(host)

    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    def sync(self):
        self._ck(self.lib.so_sync(self.h))

    def reload_tuning(self):
        """Read the SPARSEOPS_* tuning overrides from the environment again (they are read once,
        when the context is created)."""
        self._ck(self.lib.so_tuning_reload(self.h))

    @contextlib.contextmanager
    def tuning(self, **overrides):
        """with ctx.tuning(SPARSEOPS_MATMUL_TILED="1"): ...  -- set overrides (None unsets), reload,
        and put everything back afterwards."""
        saved = {k: os.environ.get(k) for k in overrides}
        try:
            for k, v in overrides.items():
                if v is None:
                    os.environ.pop(k, None)
                else:
                    os.environ[k] = str(v)
            self.reload_tuning()
            yield self
        finally:
            for k, v in saved.items():
                if v is None:
                    os.environ.pop(k, None)
                else:
                    os.environ[k] = v
            self.reload_tuning()

    def timer_begin(self):
        self._ck(self.lib.so_timer_begin(self.h))

    def timer_end(self):
        ms = ct.c_float()
        self._ck(self.lib.so_timer_end(self.h, ct.byref(ms)))
        return ms.value

    def upload_ellpack(self, Wd, idx, nnz, m, n, r, layouts=LAYOUT_ROW):
        Wd = np.ascontiguousarray(Wd, dtype=np.float32)
        idx = np.ascontiguousarray(idx, dtype=np.uint32)
        nnz = np.ascontiguousarray(nnz, dtype=np.uint32)
        h = _vp()
        self._ck(self.lib.so_ellpack_upload(self.h, _ptr(Wd), _ptr(idx), _ptr(nnz), m, n, r, layouts, ct.byref(h)))
        return DeviceEllpack(self, h.value, m, n, r)

    def encode_dense(self, dW, m, n):
        """Device-side convert_to_ellpack of the (m, n) fp32 DeviceArray dW -> DeviceEllpack (ROW layout)."""
        h = _vp()
        self._ck(self.lib.so_ellpack_encode(self.h, dW.ptr if dW is not None else None, m, n, ct.byref(h)))
        r = ct.c_uint32()
        self._ck(self.lib.so_ellpack_dims(h, None, None, ct.byref(r), None, None))
        return DeviceEllpack(self, h.value, m, n, r.value)

    def encode_dense_noalloc(self, dW, m, n, r_cap, dWd, dIdx, dNnz, want_counts=True):
        """so_ellpack_encode_noalloc into the caller's DeviceArrays -> (r, total nnz), or None without a wait."""
        r, total = ct.c_uint32(), ct.c_uint64()
        self._ck(self.lib.so_ellpack_encode_noalloc(
            self.h, dW.ptr if dW is not None else None, m, n, r_cap, dWd.ptr if dWd is not None else None,
            dIdx.ptr if dIdx is not None else None, dNnz.ptr if dNnz is not None else None,
            ct.byref(r) if want_counts else None, ct.byref(total) if want_counts else None))
        return (r.value, total.value) if want_counts else None

    def matmul(self, E, dX, C, dBias, dY, act="none"):
        self._ck(self.lib.so_matmul(self.h, E.h, dX.ptr, C, dBias.ptr if dBias else None, dY.ptr, ACT[act]))

    def matmul_reserve(self, E, C):
        self._ck(self.lib.so_matmul_reserve(self.h, E.h, C))

    def matvec(self, E, dx, dBias, dy, layout=0):
        self._ck(self.lib.so_matvec(self.h, E.h, dx.ptr, dBias.ptr if dBias else None, dy.ptr, layout))

    def conv_plan(self, E, geom):
        h = _vp()
        self._ck(self.lib.so_conv_plan_create(self.h, E.h, ct.byref(geom), ct.byref(h)))
        return h.value

    def conv_plan_tune(self, plan, B):
        self._ck(self.lib.so_conv_plan_tune(self.h, plan, B))

    def conv_plan_window(self, plan):
        """-> dict of the LDS-windowed kernel's parameters, or None when the plan has none."""
        out = (ct.c_uint32 * 8)()
        self._ck(self.lib.so_conv_plan_window(plan, out))
        keys = ("tile_h", "tile_w", "window_h", "window_w", "chunk_channels", "chunks", "channels_per_wave")
        return dict(zip(keys, out[:7])) if out[4] else None

    def upload_rbm(self, M, N, Ct_max, block_union, krel, colptr, pair_row, pair_w):
        """The flattened row-block-merged format (see so_rbm_upload) -> handle."""
        bu = np.ascontiguousarray(block_union, dtype=np.uint32)
        krel = np.ascontiguousarray(krel, dtype=np.uint32)
        colptr = np.ascontiguousarray(colptr, dtype=np.uint32)
        prow = np.ascontiguousarray(pair_row, dtype=np.uint16)
        pw = np.ascontiguousarray(pair_w, dtype=np.float32)
        h = _vp()
        self._ck(self.lib.so_rbm_upload(self.h, M, N, Ct_max, len(bu) - 1, _ptr(bu), _ptr(krel), _ptr(colptr),
                                        _ptr(prow), _ptr(pw), ct.byref(h)))
        return h.value

    def rbm_dims(self, rbm):
        M, N, Ct, nb = _u32(), _u32(), _u32(), _u32()
        U, P = ct.c_uint64(), ct.c_uint64()
        self._ck(self.lib.so_rbm_dims(rbm, ct.byref(M), ct.byref(N), ct.byref(Ct), ct.byref(nb), ct.byref(U), ct.byref(P)))
        return dict(M=M.value, N=N.value, Ct_max=Ct.value, nblocks=nb.value, union=U.value, pairs=P.value)

    def rbm_free(self, rbm):
        self.lib.so_rbm_free(self.h, rbm)

    def conv_plan_set_rbm(self, plan, rbm):
        self._ck(self.lib.so_conv_plan_set_rbm(self.h, plan, rbm))

    def conv_plan_rbm_info(self, plan):
        """-> dict(sets, pairs, slots, slots_per_record) of the plan's RBM streams, or None without streams."""
        out = (ct.c_uint64 * 4)()
        self._ck(self.lib.so_conv_plan_rbm_info(plan, out))
        return dict(sets=out[0], pairs=out[1], slots=out[2], slots_per_record=out[3]) if out[0] else None

    def conv_plan_free(self, plan):
        self.lib.so_conv_plan_free(self.h, plan)

    def conv2d(self, plan, dX, B, dBias, dY, act="none", residual=None):
        if residual is None:
            self._ck(self.lib.so_conv2d(self.h, plan, dX.ptr, B, dBias.ptr if dBias else None, dY.ptr, ACT[act]))
        else:
            self._ck(self.lib.so_conv2d_add(self.h, plan, dX.ptr, B, dBias.ptr if dBias else None, residual.ptr, dY.ptr, ACT[act]))

    def maxpool(self, C, H, W, k, s, pad, dX, B, dY):
        Ho = (H + 2 * pad[0] - k[0]) // s[0] + 1
        Wo = (W + 2 * pad[1] - k[1]) // s[1] + 1
        g = PoolGeom(C, H, W, Ho, Wo, k[0], k[1], s[0], s[1], pad[0], pad[1])
        self._ck(self.lib.so_maxpool(self.h, ct.byref(g), dX.ptr, B, dY.ptr))

    def gap(self, C, H, W, dX, B, dY):
        self._ck(self.lib.so_gap(self.h, C, H, W, dX.ptr, B, dY.ptr))

    def add(self, dA, dB, n, dD):
        self._ck(self.lib.so_add(self.h, dA.ptr, dB.ptr, n, dD.ptr))

    def act(self, act, dX, n, dY):
        self._ck(self.lib.so_act(self.h, ACT[act], dX.ptr, n, dY.ptr))

    def transpose(self, dSrc, rows, cols, dDst):
        self._ck(self.lib.so_transpose(self.h, dSrc.ptr, rows, cols, dDst.ptr))

    def reverse_axes3(self, dSrc, d0, d1, d2, inner, dDst):
        self._ck(self.lib.so_reverse_axes3(self.h, dSrc.ptr, d0, d1, d2, inner, dDst.ptr))

    def copy_rows(self, dSrc, src_stride, rows, cols, dDst, dst_stride, zero_fill=False):
        self._ck(self.lib.so_copy_rows(self.h, dSrc.ptr, src_stride, rows, cols, dDst.ptr, dst_stride, int(zero_fill)))

    def fill_zero(self, dA):
        self._ck(self.lib.so_fill_zero(self.h, dA.ptr, dA.nbytes))

    def graph_begin(self):
        self._ck(self.lib.so_graph_begin(self.h))

    def graph_end(self):
        g = _vp()
        self._ck(self.lib.so_graph_end(self.h, ct.byref(g)))
        return g.value

    def graph_launch(self, g):
        self._ck(self.lib.so_graph_launch(self.h, g))

    def graph_free(self, g):
        self.lib.so_graph_free(self.h, g)
