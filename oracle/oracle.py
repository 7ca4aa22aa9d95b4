"""ctypes front end of the CPU oracle (oracle/libzant_oracle.so).

TEST INFRASTRUCTURE ONLY: the checker the HIP backend is compared against.
Nothing in the product package imports this module; only tests, the smoke
check and the benchmark's CPU-baseline leg do.

Function names follow the reference's lean operator names
(src/Core/Tensor/TensorMath/tensor_math_standard.zig:43-149); arrays are numpy.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libzant_oracle.so")

ERR = {
    0: "OK", -1: "InvalidDimensions", -2: "InvalidPadding", -3: "InputTensorsWrongShape",
    -4: "InputTensorDifferentShape", -5: "InputTensorDimensionMismatch", -6: "IncompatibleBroadcastShapes",
    -7: "InputTensorDifferentSize", -8: "EmptyTensor", -9: "ZeroSizeTensor", -10: "InvalidInput",
    -11: "InputArrayWrongSize", -12: "WrongStride", -13: "MemError", -14: "InvalidAxes", -15: "AxisOutOfBounds",
    -16: "MismatchedShape", -17: "MismatchedRank", -18: "EmptyTensorList", -19: "UnsupportedMode",
}
PAD = {"NOTSET": 0, "SAME_UPPER": 1, "SAME_LOWER": 2, "VALID": 3}
ACT = {None: 0, "none": 0, "relu": 1, "leaky": 2, "relu6": 3}


class OracleError(Exception):
    def __init__(self, code):
        self.code = code
        self.name = ERR.get(code, "Unknown")
        super().__init__(self.name)


def build():
    """Compile the oracle with its Makefile (gcc, no GPU needed)."""
    subprocess.check_call(["make", "-C", _HERE, "-s"])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()
_i64p = C.POINTER(C.c_int64)


def _dims(seq):
    if seq is None:
        return None, 0
    arr = (C.c_int64 * max(len(seq), 1))(*[int(v) for v in seq])
    return arr, len(seq)


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _chk(rc):
    if rc != 0:
        raise OracleError(rc)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


# ----------------------------------------------------------------------------- f32

def conv_out_shape(xshape, wshape, stride, pads=None, dilations=None, group=None, auto_pad=None):
    xd, _ = _dims(xshape); wd, _ = _dims(wshape)
    s, ns = _dims(stride); p, npd = _dims(pads); d, nd = _dims(dilations)
    out = (C.c_int64 * 4)()
    _chk(_lib.zo_conv_out_shape(xd, wd, s, ns, p, npd, d, nd, C.c_int64(-1 if group is None else group),
                                None if auto_pad is None else auto_pad.encode(), out))
    return tuple(out)


def conv_lean(x, w, y, bias, stride, pads=None, dilations=None, group=None, auto_pad=None):
    """OnnxConvLean: writes into the pre-shaped y (op_convolution.zig:42)."""
    if x.ndim != 4 or w.ndim != 4:
        raise OracleError(-1)
    x = _f32(x); w = _f32(w); bias = _f32(bias)
    assert y.dtype == np.float32 and y.flags.c_contiguous
    xd, _ = _dims(x.shape); wd, _ = _dims(w.shape); yd, _ = _dims(y.shape)
    s, ns = _dims(stride); p, npd = _dims(pads); d, nd = _dims(dilations)
    _chk(_lib.zo_conv_lean_f32(_ptr(x), xd, _ptr(w), wd, _ptr(bias), _ptr(y), yd, s, ns, p, npd, d, nd,
                               C.c_int64(-1 if group is None else group),
                               None if auto_pad is None else auto_pad.encode()))
    return y


def Conv(x, w, bias, stride, pads=None, dilations=None, group=None, auto_pad=None):
    """OnnxConv: allocates the output of the expected shape, then conv_lean (op_convolution.zig:647)."""
    if x.ndim != 4 or w.ndim != 4:
        raise OracleError(-1)
    shape = conv_out_shape(x.shape, w.shape, stride, pads, dilations, group, auto_pad)
    y = np.zeros(shape, np.float32)
    return conv_lean(x, w, y, bias, stride, pads, dilations, group, auto_pad)


def convolve_tensor_with_bias(x, w, bias, stride, dilations=None):
    x = _f32(x); w = _f32(w); bias = _f32(bias)
    d = [1, 1] if dilations is None else [dilations[0], dilations[1] if len(dilations) > 1 else 1]
    dkh, dkw = (w.shape[2] - 1) * d[0] + 1, (w.shape[3] - 1) * d[1] + 1
    if x.shape[2] < dkh or x.shape[3] < dkw:
        raise OracleError(-1)
    oh, ow = (x.shape[2] - dkh) // stride[0] + 1, (x.shape[3] - dkw) // stride[1] + 1
    y = np.zeros((x.shape[0], w.shape[0], oh, ow), np.float32)
    xd, _ = _dims(x.shape); wd, _ = _dims(w.shape); s, _ = _dims(stride[:2]); dd, _ = _dims(d)
    out = (C.c_int64 * 4)()
    _chk(_lib.zo_convolve_with_bias_f32(_ptr(x), xd, _ptr(w), wd, _ptr(bias), s, dd, _ptr(y), out))
    return y


def conv_direct(x, w, bias, stride, pads, dilations, group=1):
    """Independent 7-loop convolution with double accumulation (pins the restatement)."""
    x = _f32(x); w = _f32(w); bias = _f32(bias)
    dkh, dkw = (w.shape[2] - 1) * dilations[0] + 1, (w.shape[3] - 1) * dilations[1] + 1
    oh = (x.shape[2] + pads[0] + pads[2] - dkh) // stride[0] + 1
    ow = (x.shape[3] + pads[1] + pads[3] - dkw) // stride[1] + 1
    y = np.zeros((x.shape[0], w.shape[0], oh, ow), np.float32)
    xd, _ = _dims(x.shape); wd, _ = _dims(w.shape); yd, _ = _dims(y.shape)
    s, _ = _dims(stride); p, _ = _dims(pads); d, _ = _dims(dilations)
    _chk(_lib.zo_conv_direct_f64acc(_ptr(x), xd, _ptr(w), wd, _ptr(bias), _ptr(y), yd, s, p, d, C.c_int64(group)))
    return y


def mat_mul_lean(a, b, y):
    a = _f32(a); b = _f32(b)
    ad, ar = _dims(a.shape); bd, br = _dims(b.shape)
    _chk(_lib.zo_mat_mul_lean_f32(_ptr(a), ad, ar, _ptr(b), bd, br, _ptr(y)))
    return y


def mat_mul(a, b):
    ad, ar = _dims(a.shape); bd, br = _dims(b.shape)
    _chk(_lib.zo_mat_mul_check(ad, ar, bd, br))
    y = np.zeros(tuple(a.shape[:-2]) + (a.shape[-2], b.shape[-1]), np.float32)
    return mat_mul_lean(a, b, y)


def gemm_lean(a, b, c, alpha, beta, trans_a, trans_b, y):
    a = _f32(a); b = _f32(b); c = _f32(c)
    ad, _ = _dims(a.shape); bd, _ = _dims(b.shape); yd, _ = _dims(y.shape)
    cd, cr = _dims(None if c is None else c.shape)
    _chk(_lib.zo_gemm_lean_f32(_ptr(a), ad, _ptr(b), bd, _ptr(c), cd, cr, C.c_float(alpha), C.c_float(beta),
                               int(trans_a), int(trans_b), _ptr(y), yd))
    return y


def gemm(a, b, c, alpha, beta, trans_a, trans_b):
    ad, ar = _dims(a.shape); bd, br = _dims(b.shape)
    cd, cr = _dims(None if c is None else c.shape)
    out = (C.c_int64 * 4)()
    _chk(_lib.zo_gemm_check(ad, ar, bd, br, cd, cr, int(c is not None), int(trans_a), int(trans_b), out))
    y = np.zeros(tuple(out), np.float32)
    return gemm_lean(a, b, c, alpha, beta, trans_a, trans_b, y)


def maxpool_out_shape(xshape, kernel, strides, dilations, pads, auto_pad="NOTSET", ceil_mode=False):
    xd, _ = _dims(xshape); k, _ = _dims(kernel); s, _ = _dims(strides); d, _ = _dims(dilations); p, _ = _dims(pads)
    out = (C.c_int64 * 4)()
    _chk(_lib.zo_maxpool_out_shape(xd, k, s, d, p, PAD[auto_pad], int(ceil_mode), out))
    return tuple(out)


def onnx_maxpool_lean(x, y, kernel, strides, dilations, pads, auto_pad="NOTSET"):
    xd, _ = _dims(x.shape); yd, _ = _dims(y.shape)
    k, _ = _dims(kernel); s, _ = _dims(strides); d, _ = _dims(dilations); p, npd = _dims(pads)
    x = np.ascontiguousarray(x)
    if x.dtype == np.uint8:
        _chk(_lib.zo_maxpool_lean_u8(_ptr(x), xd, _ptr(y), yd, k, s, d, p, npd, PAD[auto_pad]))
    else:
        x = _f32(x)
        _chk(_lib.zo_maxpool_lean_f32(_ptr(x), xd, _ptr(y), yd, k, s, d, p, npd, PAD[auto_pad]))
    return y


def onnx_maxpool(x, kernel, strides, dilations, pads, auto_pad="NOTSET", ceil_mode=False):
    shape = maxpool_out_shape(x.shape, kernel, strides, dilations, pads, auto_pad, ceil_mode)
    y = np.zeros(shape, x.dtype if x.dtype == np.uint8 else np.float32)
    return onnx_maxpool_lean(x, y, kernel, strides, dilations, pads, auto_pad)


def avgpool_out_shape(xshape, kernel, strides, pads=(0, 0, 0, 0), ceil_mode=False):
    """pool_forward's output size (op_pooling.zig:239-240) with ONNX AveragePool's pads and ceil_mode; a last window
    that would start in the bottom / right padding is dropped, as ONNX and torch do."""
    out = []
    for ax in range(2):
        n = xshape[2 + ax] + pads[ax] + pads[2 + ax] - kernel[ax]
        if n < 0:
            raise OracleError(-1)
        o = (-(-n // strides[ax]) if ceil_mode else n // strides[ax]) + 1
        if ceil_mode and (o - 1) * strides[ax] >= xshape[2 + ax] + pads[ax]:
            o -= 1
        out.append(o)
    return (xshape[0], xshape[1], out[0], out[1])


def avgpool_lean(x, y, kernel, strides, pads=(0, 0, 0, 0), count_include_pad=False):
    x = _f32(x)
    xd, _ = _dims(x.shape); yd, _ = _dims(y.shape)
    k, _ = _dims(kernel); s, _ = _dims(strides); p, _ = _dims(pads)
    _chk(_lib.zo_avgpool_f32(_ptr(x), xd, _ptr(y), yd, k, s, p, int(count_include_pad)))
    return y


def avgpool(x, kernel, strides, pads=(0, 0, 0, 0), ceil_mode=False, count_include_pad=False):
    """pool_forward(.Avg) for pads 0 / floor; ONNX AveragePool otherwise."""
    if x.ndim != 4:
        raise OracleError(-5)
    y = np.zeros(avgpool_out_shape(x.shape, kernel, strides, pads, ceil_mode), np.float32)
    return avgpool_lean(x, y, kernel, strides, pads, count_include_pad)


def batchnorm(x, gamma, beta, mean, var, epsilon=1e-5):
    """Inference BatchNormalization with the features on axis 1."""
    x = _f32(x)
    if x.ndim < 2:
        raise OracleError(-1)
    g, b, m, v = (_f32(np.asarray(a).reshape(-1)) for a in (gamma, beta, mean, var))
    F = x.shape[1]
    if not (g.size == b.size == m.size == v.size == F):
        raise OracleError(-5)
    y = np.zeros(x.shape, np.float32)
    inner = int(np.prod(x.shape[2:])) if x.ndim > 2 else 1
    _chk(_lib.zo_batchnorm_f32(_ptr(x), C.c_int64(x.shape[0]), C.c_int64(F), C.c_int64(inner), _ptr(g), _ptr(b), _ptr(m),
                               _ptr(v), C.c_float(epsilon), _ptr(y)))
    return y


def ReLU_lean(x, y):
    x = _f32(x)
    _chk(_lib.zo_relu_lean_f32(_ptr(x), _ptr(y), C.c_int64(x.size)))
    return y


def ReLU(x):
    if x.size == 0:
        raise OracleError(-9)
    return ReLU_lean(x, np.zeros(x.shape, np.float32))  # fromShape zero-fills (tensor.zig:128)


def leakyReLU_lean(x, slope, y):
    x = _f32(x)
    _chk(_lib.zo_leaky_relu_lean_f32(_ptr(x), C.c_float(slope), _ptr(y), C.c_int64(x.size)))
    return y


def leakyReLU(x, slope):
    if x.size == 0:
        raise OracleError(-9)
    return leakyReLU_lean(x, slope, np.zeros(x.shape, np.float32))


def softmax_lean(x, y):
    x = _f32(x)
    _chk(_lib.zo_softmax_lean_f32(_ptr(x), _ptr(y), C.c_int64(x.shape[0]), C.c_int64(x.shape[1])))
    return y


def softmax(x):
    if x.size == 0:
        raise OracleError(-9)
    return softmax_lean(x, np.zeros(x.shape, np.float32))


def sigmoid_lean(x, y):
    x = _f32(x)
    _chk(_lib.zo_sigmoid_lean_f32(_ptr(x), _ptr(y), C.c_int64(x.size)))
    return y


def sigmoid(x):
    if x.size == 0:
        raise OracleError(-9)
    return sigmoid_lean(x, np.zeros(x.shape, np.float32))


def reduce_mean(x, axes=None, keepdims=True, noop_with_empty_axes=False):
    x = _f32(x)
    xd, xr = _dims(x.shape)
    ax = (C.c_int64 * max(len(axes), 1))(*axes) if axes is not None else None
    na = len(axes) if axes is not None else 0
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    _chk(_lib.zo_reduce_mean_f32(_ptr(x), xd, xr, ax, na, int(keepdims), int(noop_with_empty_axes), None, yd, C.byref(yr)))
    y = np.zeros(tuple(yd)[:yr.value], np.float32)
    _chk(_lib.zo_reduce_mean_f32(_ptr(x), xd, xr, ax, na, int(keepdims), int(noop_with_empty_axes), _ptr(y), yd, C.byref(yr)))
    return y


def _tensor_list(tensors):
    n = len(tensors)
    keep = [_dims(t.shape) for t in tensors]
    ptrs = (C.c_void_p * max(n, 1))(*[t.ctypes.data for t in tensors])
    dims = (C.POINTER(C.c_int64) * max(n, 1))(*[C.cast(d, C.POINTER(C.c_int64)) for d, _ in keep])
    ranks = (C.c_int * max(n, 1))(*[r for _, r in keep])
    return ptrs, dims, ranks, keep


def concatenate(tensors, axis):
    tensors = [np.ascontiguousarray(t) for t in tensors]
    ptrs, dims, ranks, keep = _tensor_list(tensors)
    es = tensors[0].itemsize if tensors else 4
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    _chk(_lib.zo_concatenate(ptrs, dims, ranks, len(tensors), C.c_int64(axis), C.c_size_t(es), None, yd, C.byref(yr)))
    y = np.zeros(tuple(yd)[:yr.value], tensors[0].dtype)
    _chk(_lib.zo_concatenate(ptrs, dims, ranks, len(tensors), C.c_int64(axis), C.c_size_t(es), _ptr(y), yd, C.byref(yr)))
    return y


COORD = {"half_pixel": 0, "align_corners": 1, "asymmetric": 2}


def resize(x, mode, scales, sizes, coordinate_transformation_mode="half_pixel"):
    """Only the "nearest" mode is restated; other known modes raise NotImplementedError, unknown ones UnsupportedMode."""
    x = np.ascontiguousarray(x)
    if (scales is None) == (sizes is None):
        raise OracleError(-10)  # before the mode is looked at (lib_shape_math.zig:23-28)
    if mode in ("linear", "cubic"):
        raise NotImplementedError(mode)
    if mode != "nearest":
        raise OracleError(-19)
    xd, xr = _dims(x.shape)
    sc = (C.c_float * max(len(scales), 1))(*scales) if scales is not None else None
    sz = (C.c_int64 * max(len(sizes), 1))(*sizes) if sizes is not None else None
    n = len(scales) if scales is not None else len(sizes)
    cm = COORD.get(coordinate_transformation_mode, 2)
    yd = (C.c_int64 * 8)()
    _chk(_lib.zo_resize_nearest(_ptr(x), xd, xr, C.c_size_t(x.itemsize), sc, sz, n, cm, None, yd))
    y = np.zeros(tuple(yd)[:x.ndim], x.dtype)
    _chk(_lib.zo_resize_nearest(_ptr(x), xd, xr, C.c_size_t(x.itemsize), sc, sz, n, cm, _ptr(y), yd))
    return y


def sum_tensors_lean(a, b, y=None):
    a = _f32(a); b = _f32(b)
    ad, ar = _dims(a.shape); bd, br = _dims(b.shape)
    if y is None:
        if a.size == b.size:
            shape = a.shape
        else:
            try:
                shape = np.broadcast_shapes(a.shape, b.shape)
            except ValueError:
                raise OracleError(-6)
        y = np.zeros(shape, np.float32)
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    _chk(_lib.zo_sum_tensors_lean_f32(_ptr(a), ad, ar, _ptr(b), bd, br, _ptr(y), yd, C.byref(yr)))
    return y


def add_bias(t, bias):
    assert t.dtype == np.float32 and t.flags.c_contiguous
    bias = _f32(bias)
    td, tr = _dims(t.shape); bd, br = _dims(bias.shape)
    _chk(_lib.zo_add_bias_f32(_ptr(t), td, tr, _ptr(bias), bd, br))
    return t


def reshape_lean(x, new_shape):
    x = np.ascontiguousarray(x)
    xd, xr = _dims(x.shape); nd, nr = _dims(new_shape)
    out = (C.c_int64 * max(nr, 1))()
    y = np.empty(x.size, x.dtype)
    _chk(_lib.zo_reshape_lean(_ptr(x), xd, xr, C.c_size_t(x.itemsize), nd, nr, _ptr(y), out))
    return y.reshape(tuple(out)[:nr])


# ----------------------------------------------------------------------------- int8 family

def quantize_linear(x, y_scale, y_zp=None, axis=1, signed=False):
    """signed (or an int8 zero point): int8 output saturating to [-128, 127]; otherwise uint8."""
    x = _f32(x); y_scale = np.atleast_1d(_f32(y_scale))
    signed = signed or (y_zp is not None and np.asarray(y_zp).dtype == np.int8)
    dt = np.int8 if signed else np.uint8
    zp = None if y_zp is None else np.atleast_1d(np.ascontiguousarray(y_zp, dtype=dt))
    y = np.zeros(x.shape, dt)
    xd, r = _dims(x.shape)
    fn = _lib.zo_quantize_linear_f32_i8 if signed else _lib.zo_quantize_linear_f32_u8
    _chk(fn(_ptr(x), xd, r, _ptr(y_scale), _ptr(zp), C.c_int64(y_scale.size), axis, _ptr(y)))
    return y


def dequantize_linear(x, x_scale, x_zp=None, axis=1):
    """x: uint8, int8 or int32 (the zero point has x's type)."""
    x = np.ascontiguousarray(x)
    if x.dtype not in (np.uint8, np.int8, np.int32):
        x = x.astype(np.uint8)
    x_scale = np.atleast_1d(_f32(x_scale))
    zp = None if x_zp is None else np.atleast_1d(np.ascontiguousarray(x_zp, dtype=x.dtype))
    y = np.zeros(x.shape, np.float32)
    xd, r = _dims(x.shape)
    fn = {np.dtype(np.uint8): _lib.zo_dequantize_linear_u8_f32, np.dtype(np.int8): _lib.zo_dequantize_linear_i8_f32,
          np.dtype(np.int32): _lib.zo_dequantize_linear_i32_f32}[x.dtype]
    _chk(fn(_ptr(x), xd, r, _ptr(x_scale), _ptr(zp), C.c_int64(x_scale.size), axis, _ptr(y)))
    return y


def qconv_out_shape(xshape, wshape, stride, pads, dilations):
    dkh, dkw = (wshape[2] - 1) * dilations[0] + 1, (wshape[3] - 1) * dilations[1] + 1
    oh = (xshape[2] + pads[0] + pads[2] - dkh) // stride[0] + 1
    ow = (xshape[3] + pads[1] + pads[3] - dkw) // stride[1] + 1
    return (xshape[0], wshape[0], oh, ow)


def qconv_acc(x, x_zp, w, w_zp, bias, stride, pads, dilations, group=1):
    x = np.ascontiguousarray(x, np.uint8); w = np.ascontiguousarray(w, np.int8)
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    wz = None if w_zp is None else np.ascontiguousarray(w_zp, np.int8)
    shape = qconv_out_shape(x.shape, w.shape, stride, pads, dilations)
    acc = np.zeros(shape, np.int32)
    xd, _ = _dims(x.shape); wd, _ = _dims(w.shape); yd, _ = _dims(shape)
    s, _ = _dims(stride); p, _ = _dims(pads); d, _ = _dims(dilations)
    _chk(_lib.zo_qconv_acc_i32(_ptr(x), xd, C.c_uint8(x_zp), _ptr(w), wd, _ptr(wz), _ptr(bias), _ptr(acc), yd, s, p, d,
                               C.c_int64(group)))
    return acc


def qlinearconv(x, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp, bias, stride, pads, dilations, group=1,
                act=None, act_alpha=0.0, act_scale=1.0, act_zp=0):
    x = np.ascontiguousarray(x, np.uint8); w = np.ascontiguousarray(w, np.int8)
    ws = np.atleast_1d(_f32(w_scale))
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    wz = None if w_zp is None else np.ascontiguousarray(w_zp, np.int8)
    shape = qconv_out_shape(x.shape, w.shape, stride, pads, dilations)
    y = np.zeros(shape, np.uint8)
    xd, _ = _dims(x.shape); wd, _ = _dims(w.shape); yd, _ = _dims(shape)
    s, _ = _dims(stride); p, _ = _dims(pads); d, _ = _dims(dilations)
    _chk(_lib.zo_qlinearconv_u8i8(_ptr(x), xd, C.c_float(x_scale), C.c_uint8(x_zp), _ptr(w), wd, _ptr(ws),
                                  C.c_int64(ws.size), _ptr(wz), C.c_float(y_scale), C.c_uint8(y_zp), _ptr(bias),
                                  _ptr(y), yd, s, p, d, C.c_int64(group), ACT[act], C.c_float(act_alpha),
                                  C.c_float(act_scale), C.c_uint8(act_zp)))
    return y


def qlinear_act(x, x_scale, x_zp, act, alpha, y_scale, y_zp):
    x = np.ascontiguousarray(x, np.uint8)
    y = np.zeros(x.shape, np.uint8)
    _chk(_lib.zo_qlinear_act_u8(_ptr(x), C.c_int64(x.size), C.c_float(x_scale), C.c_uint8(x_zp), ACT[act],
                                C.c_float(alpha), C.c_float(y_scale), C.c_uint8(y_zp), _ptr(y)))
    return y


def qlinear_add(a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp):
    a = np.ascontiguousarray(a, np.uint8); b = np.ascontiguousarray(b, np.uint8)
    if a.shape != b.shape:
        raise OracleError(-7)
    y = np.zeros(a.shape, np.uint8)
    _chk(_lib.zo_qlinear_add_u8(_ptr(a), C.c_float(a_scale), C.c_uint8(a_zp), _ptr(b), C.c_float(b_scale),
                                C.c_uint8(b_zp), C.c_float(y_scale), C.c_uint8(y_zp), _ptr(y), C.c_int64(a.size)))
    return y


def qlinear_global_avgpool(x, x_scale, x_zp, y_scale, y_zp):
    x = np.ascontiguousarray(x, np.uint8)
    y = np.zeros((x.shape[0], x.shape[1], 1, 1), np.uint8)
    xd, _ = _dims(x.shape)
    _chk(_lib.zo_qlinear_global_avgpool_u8(_ptr(x), xd, C.c_float(x_scale), C.c_uint8(x_zp), C.c_float(y_scale),
                                           C.c_uint8(y_zp), _ptr(y)))
    return y
