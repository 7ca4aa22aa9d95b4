"""Host-side mirror of the reference's operator interface over libzant_hip.so.

Names, argument order and error behaviour follow the reference's façade
(src/Core/Tensor/TensorMath/tensor_math_standard.zig:43-149): every operator has a ``*_lean`` form that
writes into a caller-supplied, pre-shaped output and a standard form that validates, allocates the output
and calls the lean one.  Tensors are contiguous torch tensors on the GPU (torch only supplies the memory
and the stream); ``None`` stands for Zig's ``null``.  Errors are raised as ``ZantError`` whose ``name`` is
the Zig error name.  Nothing here computes on the CPU.
"""
import ctypes as C

import torch

from .capi import Context, ZantError, dims, lib

PAD = {"NOTSET": 0, "SAME_UPPER": 1, "SAME_LOWER": 2, "VALID": 3}
ACT = {None: 0, "none": 0, "relu": 1, "leaky": 2, "relu6": 3, "softmax": 4}

_ctx = {}


def context(device=None):
    """The per-device context, created on torch's current stream so torch copies and our kernels order."""
    dev = torch.cuda.current_device() if device is None else device
    stream = torch.cuda.current_stream(dev).cuda_stream
    key = (dev, stream)
    if key not in _ctx:
        _ctx[key] = Context(dev, stream)
    return _ctx[key]


def _p(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("tensors must live on the GPU: this backend has no CPU path")
    if not t.is_contiguous():
        raise ValueError("tensors must be contiguous")
    return C.c_void_p(t.data_ptr())


def _enc(s):
    return None if s is None else s.encode()


def _grp(g):
    return -1 if g is None else int(g)


# ------------------------------------------------------------------------------------------ Conv

def get_convolution_output_shape(xshape, wshape, stride, pads=None, dilations=None, auto_pad=None, group=None):
    xd, _ = dims(xshape); wd, _ = dims(wshape)
    s, ns = dims(stride); p, npd = dims(pads); d, nd = dims(dilations)
    out = (C.c_int64 * 4)()
    rc = lib.zant_hip_conv2d_out_shape(xd, wd, s, ns, p, npd, d, nd, _grp(group), _enc(auto_pad), out)
    if rc:
        raise ZantError(rc)
    return tuple(out)


def conv_lean(x, w, y, bias, stride, pads=None, dilations=None, group=None, auto_pad=None, fuse_act=None):
    """OnnxConvLean (op_convolution.zig:42)."""
    if x.dim() != 4 or w.dim() != 4:
        raise ZantError(-1)
    ctx = context()
    xd, _ = dims(x.shape); wd, _ = dims(w.shape); yd, _ = dims(y.shape)
    s, ns = dims(stride); p, npd = dims(pads); d, nd = dims(dilations)
    ctx.check(lib.zant_hip_conv2d_f32(ctx.handle, _p(x), xd, _p(w), wd, _p(bias), _p(y), yd, s, ns, p, npd, d, nd,
                                      _grp(group), _enc(auto_pad), ACT[fuse_act]))
    return y


def conv_lean_static(x, w, y, bias, stride, pads=None, dilations=None, group=None, auto_pad=None, fuse_act=None):
    """conv_lean through the entry point that allocates nothing (scratch in a static device array)."""
    if x.dim() != 4 or w.dim() != 4:
        raise ZantError(-1)
    ctx = context()
    xd, _ = dims(x.shape); wd, _ = dims(w.shape); yd, _ = dims(y.shape)
    s, ns = dims(stride); p, npd = dims(pads); d, nd = dims(dilations)
    ctx.check(lib.zant_hip_conv2d_f32_static(ctx.handle, _p(x), xd, _p(w), wd, _p(bias), _p(y), yd, s, ns, p, npd, d,
                                             nd, _grp(group), _enc(auto_pad), ACT[fuse_act]))
    return y


class ConvPlan:
    """Prepared weights for conv_lean (zant_hip_conv2d_f32_prepack): shapes, attributes and the weight tensors are fixed
    once; the first call packs the weights into memory the plan owns, later calls launch the convolution only."""

    def __init__(self, xshape, w, bias, yshape, stride, pads=None, dilations=None, group=None, auto_pad=None, fuse_act=None,
                 fuse_pool=False):
        """fuse_pool: Conv (-> ReLU) -> MaxPool 2x2 / stride 2 in one kernel; yshape is then the pooled shape."""
        self.ctx = context()
        self.w, self.bias, self.yshape = w, bias, tuple(yshape)  # the plan borrows the device tensors: keep them alive
        xd, _ = dims(xshape); wd, _ = dims(w.shape); yd, _ = dims(yshape)
        s, ns = dims(stride); p, npd = dims(pads); d, nd = dims(dilations)
        h = C.c_void_p()
        self.ctx.check(lib.zant_hip_conv2d_f32_prepack(self.ctx.handle, xd, _p(w), wd, _p(bias), yd, s, ns, p, npd, d, nd,
                                                       _grp(group), _enc(auto_pad), ACT[fuse_act], int(bool(fuse_pool)),
                                                       C.byref(h)))
        self.handle = h

    def __call__(self, x, y):
        self.ctx.check(lib.zant_hip_conv2d_f32_packed(self.ctx.handle, self.handle, _p(x), _p(y)))
        return y

    def close(self):
        if self.handle and self.ctx.handle:
            lib.zant_hip_conv2d_plan_destroy(self.ctx.handle, self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def Conv(x, w, bias, stride, pads=None, dilations=None, group=None, auto_pad=None):
    """OnnxConv (op_convolution.zig:647): allocate the expected shape (zero filled), then conv_lean."""
    if x.dim() != 4 or w.dim() != 4:
        raise ZantError(-1)
    shape = get_convolution_output_shape(x.shape, w.shape, stride, pads, dilations, auto_pad, group)
    y = torch.zeros(shape, dtype=torch.float32, device=x.device)
    return conv_lean(x, w, y, bias, stride, pads, dilations, group, auto_pad)


# ------------------------------------------------------------------------------------------ MatMul / Gemm

def mat_mul_lean(a, b, y):
    ctx = context()
    ad, ar = dims(a.shape); bd, br = dims(b.shape)
    ctx.check(lib.zant_hip_matmul_f32(ctx.handle, _p(a), ad, ar, _p(b), bd, br, _p(y)))
    return y


def mat_mul(a, b):
    ad, ar = dims(a.shape); bd, br = dims(b.shape)
    rc = lib.zant_hip_matmul_check(ad, ar, bd, br)
    if rc:
        raise ZantError(rc)
    y = torch.zeros(tuple(a.shape[:-2]) + (a.shape[-2], b.shape[-1]), dtype=torch.float32, device=a.device)
    return mat_mul_lean(a, b, y)


def gemm_lean(a, b, c, alpha, beta, trans_a, trans_b, y, fuse_act=None):
    ctx = context()
    ad, _ = dims(a.shape); bd, _ = dims(b.shape); yd, _ = dims(y.shape)
    cd, cr = dims(None if c is None else c.shape)
    ctx.check(lib.zant_hip_gemm_f32(ctx.handle, _p(a), ad, _p(b), bd, _p(c), cd, cr, alpha, beta, int(trans_a),
                                    int(trans_b), _p(y), yd, ACT[fuse_act]))
    return y


def gemm(a, b, c, alpha, beta, trans_a, trans_b):
    ad, ar = dims(a.shape); bd, br = dims(b.shape)
    cd, cr = dims(None if c is None else c.shape)
    out = (C.c_int64 * 4)()
    rc = lib.zant_hip_gemm_check(ad, ar, bd, br, cd, cr, int(c is not None), int(trans_a), int(trans_b), out)
    if rc:
        raise ZantError(rc)
    y = torch.zeros(tuple(out), dtype=torch.float32, device=a.device)
    return gemm_lean(a, b, c, alpha, beta, trans_a, trans_b, y)


# ------------------------------------------------------------------------------------------ MaxPool

def get_onnx_maxpool_output_shape(xshape, kernel, strides, dilations, pads, auto_pad="NOTSET", ceil_mode=False):
    if len(xshape) != 4:
        raise ZantError(-1)
    xd, _ = dims(xshape); k, _ = dims(kernel); s, _ = dims(strides); d, _ = dims(dilations); p, _ = dims(pads)
    out = (C.c_int64 * 4)()
    rc = lib.zant_hip_maxpool2d_out_shape(xd, k, s, d, p, PAD[auto_pad], int(ceil_mode), out)
    if rc:
        raise ZantError(rc)
    return tuple(out)


def onnx_maxpool_lean(x, y, kernel, strides, dilations, pads, auto_pad="NOTSET"):
    ctx = context()
    xd, _ = dims(x.shape); yd, _ = dims(y.shape)
    k, _ = dims(kernel); s, _ = dims(strides); d, _ = dims(dilations); p, npd = dims(pads)
    fn = lib.zant_hip_maxpool2d_u8 if x.dtype == torch.uint8 else lib.zant_hip_maxpool2d_f32
    ctx.check(fn(ctx.handle, _p(x), xd, _p(y), yd, k, s, d, p, npd, PAD[auto_pad]))
    return y


def onnx_maxpool(x, kernel, strides, dilations, pads, auto_pad="NOTSET", ceil_mode=False):
    shape = get_onnx_maxpool_output_shape(x.shape, kernel, strides, dilations, pads, auto_pad, ceil_mode)
    y = torch.zeros(shape, dtype=x.dtype, device=x.device)
    return onnx_maxpool_lean(x, y, kernel, strides, dilations, pads, auto_pad)


def get_avgpool_output_shape(xshape, kernel, strides, pads=None, ceil_mode=False):
    xd, _ = dims(xshape); k, _ = dims(kernel); s, _ = dims(strides); p, _ = dims(pads)
    out = (C.c_int64 * 4)()
    rc = lib.zant_hip_avgpool2d_out_shape(xd, k, s, p, int(ceil_mode), out)
    if rc:
        raise ZantError(rc)
    return tuple(out)


def avgpool_lean(x, y, kernel, strides, pads=None, count_include_pad=False):
    """pool_forward with PoolingType.Avg (op_pooling.zig:223-260, 373-408) into a pre-shaped output."""
    if x.dim() != 4:
        raise ZantError(-5)
    ctx = context()
    xd, _ = dims(x.shape); yd, _ = dims(y.shape); k, _ = dims(kernel); s, _ = dims(strides); p, _ = dims(pads)
    ctx.check(lib.zant_hip_avgpool2d_f32(ctx.handle, _p(x), xd, _p(y), yd, k, s, p, int(count_include_pad)))
    return y


def avgpool(x, kernel, strides, pads=None, ceil_mode=False, count_include_pad=False):
    if x.dim() != 4:
        raise ZantError(-5)
    y = torch.zeros(get_avgpool_output_shape(x.shape, kernel, strides, pads, ceil_mode), dtype=torch.float32, device=x.device)
    return avgpool_lean(x, y, kernel, strides, pads, count_include_pad)


def batchnorm(x, gamma, beta, mean, var, epsilon=1e-5, out=None):
    """BatchNormLayer.forward, inference branch (batchNormLayer.zig:130-148), features on axis 1."""
    if x.dim() < 2:
        raise ZantError(-1)
    if not (gamma.numel() == beta.numel() == mean.numel() == var.numel() == x.shape[1]):
        raise ZantError(-5)
    ctx = context()
    xd, xr = dims(x.shape)
    y = torch.zeros_like(x) if out is None else out
    ctx.check(lib.zant_hip_batchnorm_f32(ctx.handle, _p(x), xd, xr, _p(gamma), _p(beta), _p(mean), _p(var), epsilon, _p(y)))
    return y


# ------------------------------------------------------------------------------------------ activations, add, reshape

def ReLU_lean(x, y):
    ctx = context()
    ctx.check(lib.zant_hip_relu_f32(ctx.handle, _p(x), _p(y), x.numel()))
    return y


def ReLU(x):
    if x.numel() == 0:
        raise ZantError(-9)
    return ReLU_lean(x, torch.zeros_like(x))


def leakyReLU_lean(x, slope, y):
    ctx = context()
    ctx.check(lib.zant_hip_leaky_relu_f32(ctx.handle, _p(x), slope, _p(y), x.numel()))
    return y


def leakyReLU(x, slope):
    if x.numel() == 0:
        raise ZantError(-9)
    return leakyReLU_lean(x, slope, torch.zeros_like(x))


def softmax_lean(x, y):
    ctx = context()
    ctx.check(lib.zant_hip_softmax_f32(ctx.handle, _p(x), _p(y), x.shape[0], x.shape[1]))
    return y


def softmax(x):
    if x.numel() == 0:
        raise ZantError(-9)
    return softmax_lean(x, torch.zeros_like(x))


def sigmoid_lean(x, y):
    """sigmoid_lean (lib_activation_function_math.zig:107)."""
    ctx = context()
    ctx.check(lib.zant_hip_sigmoid_f32(ctx.handle, _p(x), _p(y), x.numel()))
    return y


def sigmoid(x):
    if x.numel() == 0:
        raise ZantError(-9)
    return sigmoid_lean(x, torch.zeros_like(x))


def get_reduce_mean_output_shape(xshape, axes=None, keepdims=True, noop_with_empty_axes=False):
    xd, xr = dims(xshape); ad, na = dims(axes)
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    rc = lib.zant_hip_reduce_mean_f32(None, None, xd, xr, ad, na, int(keepdims), int(noop_with_empty_axes), None, yd, C.byref(yr))
    if rc:
        raise ZantError(rc)
    return tuple(yd)[:yr.value]


def reduce_mean_lean(x, y, axes=None, keepdims=True, noop_with_empty_axes=False):
    """lean_reduce_mean (lib_reduction_math.zig:87): y is pre-shaped by the caller."""
    ctx = context()
    xd, xr = dims(x.shape); ad, na = dims(axes)
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    ctx.check(lib.zant_hip_reduce_mean_f32(ctx.handle, _p(x), xd, xr, ad, na, int(keepdims), int(noop_with_empty_axes), _p(y),
                                           yd, C.byref(yr)))
    return y


def reduce_mean(x, axes=None, keepdims=True, noop_with_empty_axes=False):
    """reduce_mean (lib_reduction_math.zig:30)."""
    shape = get_reduce_mean_output_shape(x.shape, axes, keepdims, noop_with_empty_axes)
    return reduce_mean_lean(x, torch.zeros(shape, dtype=torch.float32, device=x.device), axes, keepdims, noop_with_empty_axes)


def _tensor_list(tensors, shapes):
    n = len(shapes)
    keep = [dims(s) for s in shapes]
    ptrs = (C.c_void_p * max(n, 1))(*[t.data_ptr() if t is not None else None for t in tensors])
    dd = (C.POINTER(C.c_int64) * max(n, 1))(*[C.cast(d, C.POINTER(C.c_int64)) for d, _ in keep])
    rr = (C.c_int * max(n, 1))(*[r for _, r in keep])
    return ptrs, dd, rr, keep


def get_concatenate_output_shape(shapes, axis):
    ptrs, dd, rr, keep = _tensor_list([None] * len(shapes), shapes)
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    rc = lib.zant_hip_concatenate(None, ptrs, dd, rr, len(shapes), axis, 4, None, yd, C.byref(yr))
    if rc:
        raise ZantError(rc)
    return tuple(yd)[:yr.value]


def lean_concatenate(tensors, axis, y):
    """lean_concatenate (lib_shape_math.zig:307): any element type; all inputs and y of one dtype."""
    ctx = context()
    for t in tensors:
        _p(t)
    ptrs, dd, rr, keep = _tensor_list(tensors, [t.shape for t in tensors])
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    ctx.check(lib.zant_hip_concatenate(ctx.handle, ptrs, dd, rr, len(tensors), axis, y.element_size(), _p(y), yd, C.byref(yr)))
    return y


def concatenate(tensors, axis):
    """concatenate (lib_shape_math.zig:463)."""
    shape = get_concatenate_output_shape([t.shape for t in tensors], axis)
    return lean_concatenate(tensors, axis, torch.zeros(shape, dtype=tensors[0].dtype, device=tensors[0].device))


COORD = {"half_pixel": 0, "align_corners": 1, "asymmetric": 2}


def get_resize_output_shape(xshape, scales, sizes):
    xd, xr = dims(xshape)
    sc = (C.c_float * max(len(scales), 1))(*scales) if scales is not None else None
    sd, _ = dims(sizes)
    n = len(scales) if scales is not None else (len(sizes) if sizes is not None else 0)
    yd = (C.c_int64 * 8)()
    rc = lib.zant_hip_resize_nearest(None, None, xd, xr, 4, sc, sd, n, 0, None, yd)
    if rc:
        raise ZantError(rc)
    return tuple(yd)[:xr]


def resize(x, mode, scales, sizes, coordinate_transformation_mode="half_pixel", out=None):
    """resize (lib_shape_math.zig:22) in its "nearest" mode; "linear" and "cubic" are not provided, any other mode
    string is UnsupportedMode as in the reference.  Unknown coordinate modes mean "asymmetric" (the reference's else)."""
    shape = get_resize_output_shape(x.shape, scales, sizes)  # InvalidInput comes before the mode is looked at (:23-28)
    if mode in ("linear", "cubic"):
        raise NotImplementedError(f"resize mode {mode}")
    if mode != "nearest":
        raise ZantError(-19)
    ctx = context()
    y = out if out is not None else torch.zeros(shape, dtype=x.dtype, device=x.device)
    xd, xr = dims(x.shape)
    sc = (C.c_float * max(len(scales), 1))(*scales) if scales is not None else None
    sd, _ = dims(sizes)
    n = len(scales) if scales is not None else len(sizes)
    yd = (C.c_int64 * 8)()
    ctx.check(lib.zant_hip_resize_nearest(ctx.handle, _p(x), xd, xr, x.element_size(), sc, sd, n,
                                          COORD.get(coordinate_transformation_mode, 2), _p(y), yd))
    return y


def sum_tensors_lean(a, b, y=None):
    ctx = context()
    ad, ar = dims(a.shape); bd, br = dims(b.shape)
    yd = (C.c_int64 * 8)(); yr = C.c_int()
    if y is None:
        # shape-only call (no launch on empty pointers is needed: compute the shape on the host side of the ABI)
        if a.numel() == b.numel():
            shape = tuple(a.shape)
        else:
            r = max(a.dim(), b.dim())
            s1 = (1,) * (r - a.dim()) + tuple(a.shape); s2 = (1,) * (r - b.dim()) + tuple(b.shape)
            for u, v in zip(s1, s2):
                if u != v and u != 1 and v != 1:
                    raise ZantError(-6)
            shape = tuple(max(u, v) for u, v in zip(s1, s2))
        y = torch.zeros(shape, dtype=torch.float32, device=a.device)
    ctx.check(lib.zant_hip_add_f32(ctx.handle, _p(a), ad, ar, _p(b), bd, br, _p(y), yd, C.byref(yr)))
    return y


def sum_tensors(a, b):
    if a.numel() != b.numel():
        raise ZantError(-7)  # lib_elementWise_math.zig:54
    return sum_tensors_lean(a, b)


def add_bias(t, bias):
    ctx = context()
    td, tr = dims(t.shape); bd, br = dims(bias.shape)
    ctx.check(lib.zant_hip_add_bias_f32(ctx.handle, _p(t), td, tr, _p(bias), bd, br))
    return t


def reshape_lean(x, new_shape, y=None):
    """reshape_lean (lib_shape_math.zig:1139).  With y=None the result is a view of x (no copy)."""
    ctx = context()
    xd, xr = dims(x.shape); nd, nr = dims(new_shape)
    out = (C.c_int64 * max(nr, 1))()
    dst = x if y is None else y
    ctx.check(lib.zant_hip_reshape(ctx.handle, _p(x), xd, xr, x.element_size(), nd, nr, _p(dst), out))
    return dst.view(tuple(out)[:nr])


# ------------------------------------------------------------------------------------------ int8 family

def _scalar_tensor(v, dtype, device):
    return torch.as_tensor(v, dtype=dtype, device=device).reshape(-1).contiguous()


def quantize_linear(x, y_scale, y_zp=None, axis=1, signed=False, out=None):
    """signed (or an int8 zero point tensor): int8 codes saturating to [-128, 127]; otherwise uint8."""
    ctx = context()
    signed = signed or (torch.is_tensor(y_zp) and y_zp.dtype == torch.int8)
    dt = torch.int8 if signed else torch.uint8
    s = _scalar_tensor(y_scale, torch.float32, x.device)
    zp = None if y_zp is None else _scalar_tensor(y_zp, dt, x.device)
    y = out if out is not None else torch.zeros(x.shape, dtype=dt, device=x.device)
    xd, r = dims(x.shape)
    fn = lib.zant_hip_quantize_linear_f32_i8 if signed else lib.zant_hip_quantize_linear_f32_u8
    ctx.check(fn(ctx.handle, _p(x), xd, r, _p(s), _p(zp), s.numel(), axis, _p(y)))
    return y


def dequantize_linear(x, x_scale, x_zp=None, axis=1, out=None):
    """x: uint8, int8 or int32 codes (the zero point has x's type)."""
    ctx = context()
    s = _scalar_tensor(x_scale, torch.float32, x.device)
    zp = None if x_zp is None else _scalar_tensor(x_zp, x.dtype, x.device)
    y = out if out is not None else torch.zeros(x.shape, dtype=torch.float32, device=x.device)
    xd, r = dims(x.shape)
    fn = {torch.uint8: lib.zant_hip_dequantize_linear_u8_f32, torch.int8: lib.zant_hip_dequantize_linear_i8_f32,
          torch.int32: lib.zant_hip_dequantize_linear_i32_f32}[x.dtype]
    ctx.check(fn(ctx.handle, _p(x), xd, r, _p(s), _p(zp), s.numel(), axis, _p(y)))
    return y


def qconv_out_shape(xshape, wshape, stride, pads, dilations):
    dkh, dkw = (wshape[2] - 1) * dilations[0] + 1, (wshape[3] - 1) * dilations[1] + 1
    oh = (xshape[2] + pads[0] + pads[2] - dkh) // stride[0] + 1
    ow = (xshape[3] + pads[1] + pads[3] - dkw) // stride[1] + 1
    return (xshape[0], wshape[0], oh, ow)


def qlinearconv_lean(x, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp, bias, y, stride, pads, dilations, group=1,
                     act=None, act_alpha=0.0, act_scale=1.0, act_zp=0):
    ctx = context()
    xd, _ = dims(x.shape); wd, _ = dims(w.shape); yd, _ = dims(y.shape)
    s, _ = dims(stride); p, _ = dims(pads); d, _ = dims(dilations)
    ctx.check(lib.zant_hip_qlinearconv_u8i8(ctx.handle, _p(x), xd, x_scale, x_zp, _p(w), wd, _p(w_scale),
                                            w_scale.numel(), _p(w_zp), y_scale, y_zp, _p(bias), _p(y), yd, s, p, d,
                                            group, ACT[act], act_alpha, act_scale, act_zp))
    return y


def qlinearconv(x, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp, bias, stride, pads, dilations, group=1,
                act=None, act_alpha=0.0, act_scale=1.0, act_zp=0):
    y = torch.zeros(qconv_out_shape(x.shape, w.shape, stride, pads, dilations), dtype=torch.uint8, device=x.device)
    return qlinearconv_lean(x, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp, bias, y, stride, pads, dilations, group,
                            act, act_alpha, act_scale, act_zp)


NCHW, BLOCKED16 = 0, 1  # enum zant_layout


def blocked16_bytes(shape):
    d, _ = dims(shape)
    return int(lib.zant_hip_blocked16_bytes(d))


def to_blocked16(x):
    """NCHW u8 -> the channel-blocked layout of the int8 matrix-core kernels (a flat byte tensor)."""
    ctx = context()
    d, _ = dims(x.shape)
    xb = torch.empty(blocked16_bytes(x.shape), dtype=torch.uint8, device=x.device)
    ctx.check(lib.zant_hip_to_blocked16_u8(ctx.handle, _p(x), d, _p(xb)))
    return xb


def from_blocked16(xb, shape):
    ctx = context()
    d, _ = dims(shape)
    y = torch.empty(tuple(shape), dtype=torch.uint8, device=xb.device)
    ctx.check(lib.zant_hip_from_blocked16_u8(ctx.handle, _p(xb), d, _p(y)))
    return y


class QConvPlan:
    """Prepared weights for qlinearconv_lean (zant_hip_qlinearconv_prepack).  x_layout / y_layout: NCHW or BLOCKED16."""

    def __init__(self, xshape, x_scale, x_zp, w, w_scale, w_zp, y_scale, y_zp, bias, stride, pads, dilations, group=1,
                 act=None, act_alpha=0.0, act_scale=1.0, act_zp=0, x_layout=NCHW, y_layout=NCHW):
        self.ctx = context()
        self.keep = (w, w_scale, w_zp, bias)  # the plan borrows the device tensors: keep them alive
        self.yshape = qconv_out_shape(xshape, w.shape, stride, pads, dilations)
        xd, _ = dims(xshape); wd, _ = dims(w.shape); yd, _ = dims(self.yshape)
        s, _ = dims(stride); p, _ = dims(pads); d, _ = dims(dilations)
        h = C.c_void_p()
        self.ctx.check(lib.zant_hip_qlinearconv_prepack(self.ctx.handle, xd, x_scale, x_zp, _p(w), wd, _p(w_scale),
                                                        w_scale.numel(), _p(w_zp), y_scale, y_zp, _p(bias), yd, s, p, d,
                                                        group, ACT[act], act_alpha, act_scale, act_zp, x_layout, y_layout,
                                                        C.byref(h)))
        self.handle = h
        self.y_layout = y_layout

    def __call__(self, x, y=None):
        if y is None:
            y = (torch.empty(blocked16_bytes(self.yshape), dtype=torch.uint8, device=x.device) if self.y_layout == BLOCKED16
                 else torch.zeros(self.yshape, dtype=torch.uint8, device=x.device))
        self.ctx.check(lib.zant_hip_qlinearconv_u8i8_packed(self.ctx.handle, self.handle, _p(x), _p(y)))
        return y

    def close(self):
        if self.handle and self.ctx.handle:
            lib.zant_hip_qlinearconv_plan_destroy(self.ctx.handle, self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def qlinear_act(x, x_scale, x_zp, act, alpha, y_scale, y_zp, out=None):
    ctx = context()
    y = out if out is not None else torch.zeros_like(x)
    ctx.check(lib.zant_hip_qlinear_act_u8(ctx.handle, _p(x), x.numel(), x_scale, x_zp, ACT[act], alpha, y_scale, y_zp,
                                          _p(y)))
    return y


def qlinear_add(a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp, out=None):
    if a.shape != b.shape:
        raise ZantError(-7)
    ctx = context()
    y = out if out is not None else torch.zeros_like(a)
    ctx.check(lib.zant_hip_qlinear_add_u8(ctx.handle, _p(a), a_scale, a_zp, _p(b), b_scale, b_zp, y_scale, y_zp, _p(y),
                                          a.numel()))
    return y


def qlinear_global_avgpool(x, x_scale, x_zp, y_scale, y_zp, out=None):
    ctx = context()
    y = out if out is not None else torch.zeros((x.shape[0], x.shape[1], 1, 1), dtype=torch.uint8, device=x.device)
    xd, _ = dims(x.shape)
    ctx.check(lib.zant_hip_qlinear_global_avgpool_u8(ctx.handle, _p(x), xd, x_scale, x_zp, y_scale, y_zp, _p(y)))
    return y
