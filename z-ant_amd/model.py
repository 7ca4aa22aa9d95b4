"""Python handle of a zant_model: the GPU form of a library the reference's code generator would emit
(src/codeGen/predict.zig): nodes appended in ready order, one arena, one `run` per forward pass."""
import ctypes as C
import sys

import numpy as np

from .capi import Context, ZantError, dims, lib
from .tensor_math import ACT, PAD

F32, U8 = 0, 1


def _np(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


class HostPtr(C.c_void_p):
    """A void pointer that remembers the numpy array it points into (keeps it alive for the call; the code generator
    reads the array back to embed it)."""


def _hp(a):
    if a is None:
        return None
    p = HostPtr(a.ctypes.data)
    p.array = a
    return p


class Model:
    def __init__(self, ctx: Context):
        """ctx None: a dry-run model that validates the graph and answers shape queries on the host (no GPU is touched)
        but cannot be finalized."""
        self.ctx = ctx
        self._lib = lib  # every library call of this class goes through it (the code generator substitutes a recorder)
        h = C.c_void_p()
        rc = lib.zant_model_create(ctx.handle if ctx is not None else None, C.byref(h))
        if rc:
            raise ZantError(rc)
        self.handle = h

    def _id(self, rc):
        if rc < 0:
            raise ZantError(rc)
        return rc

    def input(self, shape, dtype=F32, scale=1.0, zp=0):
        d, r = dims(shape)
        return self._id(self._lib.zant_model_input(self.handle, dtype, d, r, scale, zp))

    def conv(self, x, w, bias, stride, pads=None, dilations=None, group=1, auto_pad=None):
        w = _np(w, np.float32); bias = _np(bias, np.float32)
        wd, _ = dims(w.shape); s, ns = dims(stride); p, npd = dims(pads); d, nd = dims(dilations)
        return self._id(self._lib.zant_model_conv(self.handle, x, _hp(w), wd, _hp(bias), s, ns, p, npd, d, nd,
                                            -1 if group is None else group, None if auto_pad is None else auto_pad.encode()))

    def relu(self, x):
        return self._id(self._lib.zant_model_relu(self.handle, x))

    def leaky_relu(self, x, slope):
        return self._id(self._lib.zant_model_leaky_relu(self.handle, x, slope))

    def maxpool(self, x, kernel, strides, dilations=(1, 1), pads=(0, 0, 0, 0), auto_pad="NOTSET", ceil_mode=False):
        k, _ = dims(kernel); s, _ = dims(strides); d, _ = dims(dilations); p, _ = dims(pads)
        return self._id(self._lib.zant_model_maxpool(self.handle, x, k, s, d, p, PAD[auto_pad], int(ceil_mode)))

    def avgpool(self, x, kernel, strides, pads=None, ceil_mode=False, count_include_pad=False):
        k, _ = dims(kernel); s, _ = dims(strides); p, _ = dims(pads)
        return self._id(self._lib.zant_model_avgpool(self.handle, x, k, s, p, int(ceil_mode), int(count_include_pad)))

    def batchnorm(self, x, gamma, beta, mean, var, epsilon=1e-5):
        g, b, mu, v = (_np(np.asarray(a).reshape(-1), np.float32) for a in (gamma, beta, mean, var))
        if not (g.size == b.size == mu.size == v.size):
            raise ZantError(-5)
        return self._id(self._lib.zant_model_batchnorm(self.handle, x, _hp(g), _hp(b), _hp(mu), _hp(v), g.size, epsilon))

    def reshape(self, x, new_shape):
        d, r = dims(new_shape)
        return self._id(self._lib.zant_model_reshape(self.handle, x, d, r))

    def gemm(self, a, b, c=None, alpha=1.0, beta=1.0, trans_a=False, trans_b=False):
        """gemm_lean: A (a rank-4 tensor {1, 1, rows, cols}), B and C in the reference's rank-4 form; B and C of lower
        rank are given leading ones (the C side reads four B dimensions)."""
        b = _np(b, np.float32); c = _np(c, np.float32)
        if b.ndim > 4 or (c is not None and c.ndim > 4):
            raise ZantError(-3)
        b = b.reshape((1,) * (4 - b.ndim) + b.shape)
        if c is not None:
            c = c.reshape((1,) * (4 - c.ndim) + c.shape)
        bd, _ = dims(b.shape); cd, cr = dims(None if c is None else c.shape)
        return self._id(self._lib.zant_model_gemm(self.handle, a, _hp(b), bd, _hp(c), cd, cr, alpha, beta, int(trans_a), int(trans_b)))

    def matmul(self, a, b):
        b = _np(b, np.float32)
        bd, br = dims(b.shape)
        return self._id(self._lib.zant_model_matmul(self.handle, a, _hp(b), bd, br))

    def add_const(self, x, c):
        c = _np(c, np.float32)
        cd, cr = dims(c.shape)
        return self._id(self._lib.zant_model_add_const(self.handle, x, _hp(c), cd, cr))

    def add(self, a, b):
        return self._id(self._lib.zant_model_add(self.handle, a, b))

    def softmax(self, x):
        return self._id(self._lib.zant_model_softmax(self.handle, x))

    def sigmoid(self, x):
        return self._id(self._lib.zant_model_sigmoid(self.handle, x))

    def reduce_mean(self, x, axes, keepdims=True):
        ad, na = dims(axes)
        return self._id(self._lib.zant_model_reduce_mean(self.handle, x, ad, na, int(keepdims)))

    def global_average_pool(self, x):
        """ONNX GlobalAveragePool of an NCHW tensor: the mean over H and W, rank kept."""
        return self.reduce_mean(x, [2, 3], True)

    def concat(self, xs, axis):
        arr = (C.c_int * max(len(xs), 1))(*xs)
        return self._id(self._lib.zant_model_concat(self.handle, arr, len(xs), axis))

    def resize_nearest(self, x, scales=None, sizes=None, coordinate_transformation_mode="half_pixel"):
        sc = (C.c_float * len(scales))(*scales) if scales is not None else None
        sd, _ = dims(sizes)
        n = len(scales) if scales is not None else (len(sizes) if sizes is not None else 0)
        mode = {"half_pixel": 0, "align_corners": 1}.get(coordinate_transformation_mode, 2)
        return self._id(self._lib.zant_model_resize_nearest(self.handle, x, sc, sd, n, mode))

    def tensor_shape(self, x):
        d = (C.c_int64 * 8)(); r = C.c_int()
        self._id(self._lib.zant_model_tensor_dims(self.handle, x, d, C.byref(r), None))
        return tuple(d)[:r.value]

    def quantize(self, x, scale, zp):
        return self._id(self._lib.zant_model_quantize(self.handle, x, scale, zp))

    def dequantize(self, x):
        return self._id(self._lib.zant_model_dequantize(self.handle, x))

    def qlinearconv(self, x, w, w_scale, bias, y_scale, y_zp, stride, pads, dilations=(1, 1), group=1):
        w = _np(w, np.int8); ws = np.atleast_1d(_np(w_scale, np.float32)); bias = _np(bias, np.int32)
        wd, _ = dims(w.shape); s, _ = dims(stride); p, _ = dims(pads); d, _ = dims(dilations)
        return self._id(self._lib.zant_model_qlinearconv(self.handle, x, _hp(w), wd, _hp(ws), ws.size, _hp(bias), y_scale, y_zp,
                                                   s, p, d, group))

    def qlinear_act(self, x, act, alpha, y_scale, y_zp):
        return self._id(self._lib.zant_model_qlinear_act(self.handle, x, ACT[act], alpha, y_scale, y_zp))

    def qlinear_add(self, a, b, y_scale, y_zp):
        return self._id(self._lib.zant_model_qlinear_add(self.handle, a, b, y_scale, y_zp))

    def qlinear_global_avgpool(self, x, y_scale, y_zp):
        return self._id(self._lib.zant_model_qlinear_global_avgpool(self.handle, x, y_scale, y_zp))

    def finalize(self):
        rc = self._lib.zant_model_finalize(self.handle)
        if rc:
            raise ZantError(rc)
        d = (C.c_int64 * 8)(); r = C.c_int(); dt = C.c_int()
        self._lib.zant_model_output_dims(self.handle, d, C.byref(r), C.byref(dt))
        self.out_shape = tuple(d[i] for i in range(r.value))
        self.out_dtype = np.float32 if dt.value == F32 else np.uint8
        return self

    @property
    def arena_bytes(self):
        return self._lib.zant_model_arena_bytes(self.handle)

    @property
    def unfused_bytes(self):
        return self._lib.zant_model_unfused_bytes(self.handle)

    @property
    def num_launches(self):
        return self._lib.zant_model_num_launches(self.handle)

    @property
    def input_ptr(self):
        return self._lib.zant_model_input_ptr(self.handle)

    @property
    def output_ptr(self):
        return self._lib.zant_model_output_ptr(self.handle)

    def run(self, input_dev_ptr=None, output_dev_ptr=None):
        """Device in / device out; asynchronous on the context's stream; allocates nothing.  With no pointers the
        input is taken from `input_ptr` and the result left at `output_ptr` (both inside the arena)."""
        rc = self._lib.zant_model_run(self.handle, None if input_dev_ptr is None else C.c_void_p(input_dev_ptr),
                                None if output_dev_ptr is None else C.c_void_p(output_dev_ptr))
        if rc:
            raise ZantError(rc)

    def profile(self):
        """One pass with per-kernel timing -> [(name, ms, ops, bytes)] per kernel-launching node."""
        n = self.num_launches
        ms = (C.c_float * n)(); ops = (C.c_double * n)(); by = (C.c_double * n)()
        rc = self._lib.zant_model_profile(self.handle, ms, ops, by, n)
        if rc < 0:
            raise ZantError(rc)
        return [(self._lib.zant_model_launch_name(self.handle, i).decode(), ms[i], ops[i], by[i]) for i in range(rc)]

    def launch_kernels(self):
        """Device function of each launch's main kernel as of the last profile() (a profiler's kernel-trace names)."""
        return [self._lib.zant_model_launch_kernel(self.handle, i).decode() for i in range(self.num_launches)]

    def predict_host(self, x):
        x = np.ascontiguousarray(x)
        y = np.zeros(self.out_shape, self.out_dtype)
        rc = self._lib.zant_model_predict_host(self.handle, _hp(x), _hp(y))
        if rc:
            raise ZantError(rc)
        return y

    def read_tensor(self, tid, shape, dtype):
        y = np.zeros(shape, dtype)
        rc = self._lib.zant_model_read_tensor(self.handle, tid, _hp(y), y.nbytes)
        if rc:
            raise ZantError(rc)
        return y

    def bind_predict(self):
        rc = self._lib.zant_model_bind_predict(self.handle)
        if rc:
            raise ZantError(rc)

    def close(self):
        if self.handle:
            self._lib.zant_model_destroy(self.handle)
            self.handle = None

    def __del__(self):
        if sys is None or sys.is_finalizing():  # the HIP runtime may already be gone at interpreter exit; the OS reclaims the rest
            return
        try:
            self.close()
        except Exception:
            pass
