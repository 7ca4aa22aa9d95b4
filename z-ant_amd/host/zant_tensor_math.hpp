// Host-side C++ mirror of the reference's operator interface over the C ABI of libzant_hip.so.
//
// The reference is Zig: `Tensor(T)` (src/Core/Tensor/tensor.zig:25-31) and the `tensMath` facade
// (src/Core/Tensor/TensorMath/tensor_math_standard.zig:43-149) whose operators come in a lean form
// (caller supplies a pre-shaped output, returns an error union) and a standard form (validates,
// allocates the output, calls the lean form).  This header keeps those names, argument order and
// error behaviour; a Zig error becomes a thrown zant::Error whose code() is the zant_status.
// Tensor data lives on the GPU; optional arguments are pointers / std::optional (null = Zig null).
#pragma once
#include <cstdint>
#include <optional>
#include <stdexcept>
#include <string>
#include <vector>

#include "zant_hip.h"

namespace zant {

class Error : public std::runtime_error {
  public:
    explicit Error(int code) : std::runtime_error(zant_hip_status_name(code)), code_(code) {}
    int code() const { return code_; }

  private:
    int code_;
};

inline void check(int rc) {
    if (rc != ZANT_OK) throw Error(rc);
}

// One context per thread, like one generated library instance.
inline zant_ctx *&default_ctx() {
    static zant_ctx *ctx = nullptr;
    if (!ctx) check(zant_hip_ctx_create(&ctx, 0, nullptr));
    return ctx;
}

// Tensor(T): data (device), size, shape, owns_memory -- tensor.zig:25-31.
template <typename T>
struct Tensor {
    T *data = nullptr;
    size_t size = 0;
    std::vector<int64_t> shape;
    bool owns_memory = false;

    Tensor() = default;
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;
    Tensor(Tensor &&o) noexcept { *this = std::move(o); }
    Tensor &operator=(Tensor &&o) noexcept {
        deinit();
        data = o.data; size = o.size; shape = std::move(o.shape); owns_memory = o.owns_memory;
        o.data = nullptr; o.size = 0; o.owns_memory = false;
        return *this;
    }
    ~Tensor() { deinit(); }

    // fromShape: zero filled (tensor.zig:116-130)
    static Tensor fromShape(const std::vector<int64_t> &shape) {
        Tensor t;
        t.shape = shape;
        t.size = 1;
        for (int64_t d : shape) t.size *= size_t(d);
        void *p = nullptr;
        check(zant_hip_malloc(default_ctx(), &p, t.size * sizeof(T)));
        t.data = static_cast<T *>(p);
        t.owns_memory = true;
        check(zant_hip_memset(default_ctx(), t.data, 0, t.size * sizeof(T)));
        return t;
    }
    // fromArray: copies host data (tensor.zig:63-100)
    static Tensor fromArray(const T *host, const std::vector<int64_t> &shape) {
        Tensor t = fromShape(shape);
        check(zant_hip_upload(default_ctx(), t.data, host, t.size * sizeof(T)));
        return t;
    }
    // fromConstBuffer: borrows device memory, e.g. a slice of the arena (tensor.zig:142-150)
    static Tensor fromConstBuffer(T *device_data, const std::vector<int64_t> &shape) {
        Tensor t;
        t.shape = shape;
        t.size = 1;
        for (int64_t d : shape) t.size *= size_t(d);
        t.data = device_data;
        t.owns_memory = false;
        return t;
    }
    std::vector<T> toHost() const {
        std::vector<T> h(size);
        check(zant_hip_download(default_ctx(), h.data(), data, size * sizeof(T)));
        return h;
    }
    void deinit() {
        if (owns_memory && data) (void)zant_hip_free(default_ctx(), data);
        data = nullptr;
        owns_memory = false;
    }
};

enum class AutoPadType { NOTSET = 0, SAME_UPPER = 1, SAME_LOWER = 2, VALID = 3 };  // op_pooling.zig:9-14

namespace tensMath {

using Dims = std::vector<int64_t>;

// conv_lean = OnnxConvLean (op_convolution.zig:42)
inline void conv_lean(Tensor<float> *input, Tensor<float> *kernel, Tensor<float> *output, const Tensor<float> *bias,
                      const Dims &stride, const Dims *pads, const Dims *dilations, std::optional<int64_t> group,
                      const char *auto_pad) {
    if (input->shape.size() != 4 || kernel->shape.size() != 4) throw Error(ZANT_InvalidDimensions);
    check(zant_hip_conv2d_f32(default_ctx(), input->data, input->shape.data(), kernel->data, kernel->shape.data(),
                              bias ? bias->data : nullptr, output->data, output->shape.data(), stride.data(),
                              int(stride.size()), pads ? pads->data() : nullptr, pads ? int(pads->size()) : 0,
                              dilations ? dilations->data() : nullptr, dilations ? int(dilations->size()) : 0,
                              group ? *group : -1, auto_pad, ZANT_ACT_NONE));
}

// Conv = OnnxConv (op_convolution.zig:647)
inline Tensor<float> Conv(Tensor<float> *input, Tensor<float> *kernel, const Tensor<float> *bias, const Dims &stride,
                          const Dims *pads, const Dims *dilations, std::optional<int64_t> group, const char *auto_pad) {
    if (input->shape.size() != 4 || kernel->shape.size() != 4) throw Error(ZANT_InvalidDimensions);
    int64_t ydim[4];
    check(zant_hip_conv2d_out_shape(input->shape.data(), kernel->shape.data(), stride.data(), int(stride.size()),
                                    pads ? pads->data() : nullptr, pads ? int(pads->size()) : 0,
                                    dilations ? dilations->data() : nullptr, dilations ? int(dilations->size()) : 0,
                                    group ? *group : -1, auto_pad, ydim));
    Tensor<float> out = Tensor<float>::fromShape({ydim[0], ydim[1], ydim[2], ydim[3]});
    conv_lean(input, kernel, &out, bias, stride, pads, dilations, group, auto_pad);
    return out;
}

// mat_mul_lean / mat_mul (op_mat_mul.zig:92, :22)
inline void mat_mul_lean(const Tensor<float> *A, const Tensor<float> *B, Tensor<float> *Y) {
    check(zant_hip_matmul_f32(default_ctx(), A->data, A->shape.data(), int(A->shape.size()), B->data, B->shape.data(),
                              int(B->shape.size()), Y->data));
}
inline Tensor<float> mat_mul(const Tensor<float> *A, const Tensor<float> *B) {
    check(zant_hip_matmul_check(A->shape.data(), int(A->shape.size()), B->shape.data(), int(B->shape.size())));
    Dims out = A->shape;
    out[out.size() - 1] = B->shape.back();
    Tensor<float> Y = Tensor<float>::fromShape(out);
    mat_mul_lean(A, B, &Y);
    return Y;
}

// gemm_lean / gemm (op_gemm.zig:91, :15)
inline void gemm_lean(Tensor<float> *A, Tensor<float> *B, Tensor<float> *C, float alpha, float beta, bool transA,
                      bool transB, Tensor<float> *result) {
    check(zant_hip_gemm_f32(default_ctx(), A->data, A->shape.data(), B->data, B->shape.data(), C ? C->data : nullptr,
                            C ? C->shape.data() : nullptr, C ? int(C->shape.size()) : 0, alpha, beta, transA, transB,
                            result->data, result->shape.data(), ZANT_ACT_NONE));
}
inline Tensor<float> gemm(Tensor<float> *A, Tensor<float> *B, Tensor<float> *C, float alpha, float beta, bool transA,
                          bool transB) {
    int64_t ydim[4];
    check(zant_hip_gemm_check(A->shape.data(), int(A->shape.size()), B->shape.data(), int(B->shape.size()),
                              C ? C->shape.data() : nullptr, C ? int(C->shape.size()) : 0, C != nullptr, transA, transB,
                              ydim));
    Tensor<float> Y = Tensor<float>::fromShape({ydim[0], ydim[1], ydim[2], ydim[3]});
    gemm_lean(A, B, C, alpha, beta, transA, transB, &Y);
    return Y;
}

// onnx_maxpool_lean / onnx_maxpool (op_pooling.zig:570, :663)
template <typename T>
inline void onnx_maxpool_lean(Tensor<T> *input, Tensor<T> *output, const Dims &kernel_shape, const Dims &strides,
                              const Dims &dilations, const Dims &pads, AutoPadType auto_pad);
template <>
inline void onnx_maxpool_lean<float>(Tensor<float> *input, Tensor<float> *output, const Dims &k, const Dims &s,
                                     const Dims &d, const Dims &p, AutoPadType ap) {
    check(zant_hip_maxpool2d_f32(default_ctx(), input->data, input->shape.data(), output->data, output->shape.data(),
                                 k.data(), s.data(), d.data(), p.data(), int(p.size()), int(ap)));
}
template <>
inline void onnx_maxpool_lean<uint8_t>(Tensor<uint8_t> *input, Tensor<uint8_t> *output, const Dims &k, const Dims &s,
                                       const Dims &d, const Dims &p, AutoPadType ap) {
    check(zant_hip_maxpool2d_u8(default_ctx(), input->data, input->shape.data(), output->data, output->shape.data(),
                                k.data(), s.data(), d.data(), p.data(), int(p.size()), int(ap)));
}
template <typename T>
inline Tensor<T> onnx_maxpool(Tensor<T> *input, const Dims &k, const Dims &s, const Dims &d, const Dims &p,
                              AutoPadType ap, bool ceil_mode) {
    if (input->shape.size() != 4) throw Error(ZANT_InvalidDimensions);
    int64_t ydim[4];
    check(zant_hip_maxpool2d_out_shape(input->shape.data(), k.data(), s.data(), d.data(), p.data(), int(ap), ceil_mode,
                                       ydim));
    Tensor<T> out = Tensor<T>::fromShape({ydim[0], ydim[1], ydim[2], ydim[3]});
    onnx_maxpool_lean<T>(input, &out, k, s, d, p, ap);
    return out;
}

// ReLU_lean / ReLU, leakyReLU_lean / leakyReLU, softmax_lean / softmax (lib_activation_function_math.zig)
inline void ReLU_lean(Tensor<float> *in, Tensor<float> *out) {
    check(zant_hip_relu_f32(default_ctx(), in->data, out->data, int64_t(in->size)));
}
inline Tensor<float> ReLU(Tensor<float> *in) {
    if (in->size == 0) throw Error(ZANT_ZeroSizeTensor);
    Tensor<float> out = Tensor<float>::fromShape(in->shape);
    ReLU_lean(in, &out);
    return out;
}
inline void leakyReLU_lean(Tensor<float> *in, float slope, Tensor<float> *out) {
    check(zant_hip_leaky_relu_f32(default_ctx(), in->data, slope, out->data, int64_t(in->size)));
}
inline Tensor<float> leakyReLU(Tensor<float> *in, float slope) {
    if (in->size == 0) throw Error(ZANT_ZeroSizeTensor);
    Tensor<float> out = Tensor<float>::fromShape(in->shape);
    leakyReLU_lean(in, slope, &out);
    return out;
}
inline void softmax_lean(Tensor<float> *in, Tensor<float> *out) {
    check(zant_hip_softmax_f32(default_ctx(), in->data, out->data, in->shape[0], in->shape[1]));
}
inline Tensor<float> softmax(Tensor<float> *in) {
    if (in->size == 0) throw Error(ZANT_ZeroSizeTensor);
    Tensor<float> out = Tensor<float>::fromShape(in->shape);
    softmax_lean(in, &out);
    return out;
}

// sigmoid_lean / sigmoid (lib_activation_function_math.zig:107, :95)
inline void sigmoid_lean(Tensor<float> *in, Tensor<float> *out) {
    check(zant_hip_sigmoid_f32(default_ctx(), in->data, out->data, int64_t(in->size)));
}
inline Tensor<float> sigmoid(Tensor<float> *in) {
    if (in->size == 0) throw Error(ZANT_ZeroSizeTensor);
    Tensor<float> out = Tensor<float>::fromShape(in->shape);
    sigmoid_lean(in, &out);
    return out;
}

// lean_reduce_mean / reduce_mean (lib_reduction_math.zig:87, :30); axes == nullptr is Zig's null
inline void reduce_mean_lean(Tensor<float> *in, Tensor<float> *out, const Dims *axes, bool keepdims, bool noop_with_empty_axes) {
    int64_t ydim[8];
    int yr = 0;
    check(zant_hip_reduce_mean_f32(default_ctx(), in->data, in->shape.data(), int(in->shape.size()), axes ? axes->data() : nullptr,
                                   axes ? int(axes->size()) : 0, keepdims, noop_with_empty_axes, out->data, ydim, &yr));
}
inline Tensor<float> reduce_mean(Tensor<float> *in, const Dims *axes, bool keepdims, bool noop_with_empty_axes) {
    int64_t ydim[8];
    int yr = 0;
    check(zant_hip_reduce_mean_f32(nullptr, nullptr, in->shape.data(), int(in->shape.size()), axes ? axes->data() : nullptr,
                                   axes ? int(axes->size()) : 0, keepdims, noop_with_empty_axes, nullptr, ydim, &yr));
    Tensor<float> out = Tensor<float>::fromShape(Dims(ydim, ydim + yr));
    reduce_mean_lean(in, &out, axes, keepdims, noop_with_empty_axes);
    return out;
}

// get_concatenate_output_shape / lean_concatenate / concatenate (lib_shape_math.zig:582, :307, :463)
template <typename T>
inline Dims concatenate_impl(const std::vector<Tensor<T> *> &tensors, int64_t axis, T *out) {
    std::vector<const void *> ptrs;
    std::vector<const int64_t *> shapes;
    std::vector<int> ranks;
    for (Tensor<T> *t : tensors) {
        ptrs.push_back(t->data);
        shapes.push_back(t->shape.data());
        ranks.push_back(int(t->shape.size()));
    }
    int64_t ydim[8];
    int yr = 0;
    check(zant_hip_concatenate(out ? default_ctx() : nullptr, ptrs.data(), shapes.data(), ranks.data(), int(tensors.size()), axis,
                               sizeof(T), out, ydim, &yr));
    return Dims(ydim, ydim + yr);
}
template <typename T>
inline void lean_concatenate(const std::vector<Tensor<T> *> &tensors, int64_t axis, Tensor<T> *out) {
    out->shape = concatenate_impl<T>(tensors, axis, out->data);
}
template <typename T>
inline Tensor<T> concatenate(const std::vector<Tensor<T> *> &tensors, int64_t axis) {
    Tensor<T> out = Tensor<T>::fromShape(concatenate_impl<T>(tensors, axis, nullptr));
    lean_concatenate<T>(tensors, axis, &out);
    return out;
}

// resize in "nearest" mode (lib_shape_math.zig:22); scales / sizes == nullptr is Zig's null
template <typename T>
inline Tensor<T> resize(Tensor<T> *t, const std::string &mode, const std::vector<float> *scales, const Dims *sizes,
                        const std::string &coordinate_transformation_mode) {
    int64_t ydim[8];
    const int n = scales ? int(scales->size()) : sizes ? int(sizes->size()) : 0;
    const int cm = coordinate_transformation_mode == "half_pixel" ? 0 : coordinate_transformation_mode == "align_corners" ? 1 : 2;
    check(zant_hip_resize_nearest(nullptr, nullptr, t->shape.data(), int(t->shape.size()), sizeof(T), scales ? scales->data() : nullptr,
                                  sizes ? sizes->data() : nullptr, n, cm, nullptr, ydim));
    if (mode != "nearest") throw Error(ZANT_UnsupportedMode);  // "linear" / "cubic" are not provided either
    Tensor<T> out = Tensor<T>::fromShape(Dims(ydim, ydim + t->shape.size()));
    check(zant_hip_resize_nearest(default_ctx(), t->data, t->shape.data(), int(t->shape.size()), sizeof(T),
                                  scales ? scales->data() : nullptr, sizes ? sizes->data() : nullptr, n, cm, out.data, ydim));
    return out;
}

// sum_tensors_lean / sum_tensors, add_bias (lib_elementWise_math.zig:70, :52, :22)
inline void sum_tensors_lean(Tensor<float> *t1, Tensor<float> *t2, Tensor<float> *out) {
    int64_t ydim[8];
    int yr = 0;
    check(zant_hip_add_f32(default_ctx(), t1->data, t1->shape.data(), int(t1->shape.size()), t2->data, t2->shape.data(),
                           int(t2->shape.size()), out->data, ydim, &yr));
    out->shape.assign(ydim, ydim + yr);  // the lean op rewrites the output shape (:157)
}
inline Tensor<float> sum_tensors(Tensor<float> *t1, Tensor<float> *t2) {
    if (t1->size != t2->size) throw Error(ZANT_InputTensorDifferentSize);
    Tensor<float> out = Tensor<float>::fromShape(t2->shape);
    sum_tensors_lean(t1, t2, &out);
    return out;
}
inline void add_bias(Tensor<float> *tensor, Tensor<float> *bias) {
    check(zant_hip_add_bias_f32(default_ctx(), tensor->data, tensor->shape.data(), int(tensor->shape.size()), bias->data,
                                bias->shape.data(), int(bias->shape.size())));
}

// reshape_lean (lib_shape_math.zig:1139); -1 stands for the maxInt(usize) sentinel
template <typename T>
inline void reshape_lean(Tensor<T> *in, const Dims &newShape, std::optional<bool> /*allowZero*/, Tensor<T> *out) {
    Dims resolved(newShape.size());
    check(zant_hip_reshape(default_ctx(), in->data, in->shape.data(), int(in->shape.size()), sizeof(T), newShape.data(),
                           int(newShape.size()), out->data, resolved.data()));
    out->shape = resolved;
    out->size = in->size;
}

// ---- the quantised family: ONNX QuantizeLinear / DequantizeLinear / QLinearConv ---------------------------
// The reference has no such operators (src/Core/Quantization/quantization.zig is empty); these keep its two forms
// (lean: pre-shaped output; standard: allocates) and the ONNX input order.  Scale and zero-point tensors live on the
// device and hold one element (per tensor) or shape[axis] elements (per axis).

// quantize_linear_lean: y = saturate(round_half_even(x / y_scale) + y_zero_point); T_out: uint8_t or int8_t
template <typename T_out>
inline void quantize_linear_lean(Tensor<float> *x, Tensor<float> *y_scale, Tensor<T_out> *y_zero_point, int64_t axis,
                                 Tensor<T_out> *y);
template <>
inline void quantize_linear_lean<uint8_t>(Tensor<float> *x, Tensor<float> *y_scale, Tensor<uint8_t> *y_zero_point,
                                          int64_t axis, Tensor<uint8_t> *y) {
    if (axis < 0) axis += int64_t(x->shape.size());
    check(zant_hip_quantize_linear_f32_u8(default_ctx(), x->data, x->shape.data(), int(x->shape.size()), y_scale->data,
                                          y_zero_point ? y_zero_point->data : nullptr, int64_t(y_scale->size), int(axis), y->data));
}
template <>
inline void quantize_linear_lean<int8_t>(Tensor<float> *x, Tensor<float> *y_scale, Tensor<int8_t> *y_zero_point,
                                         int64_t axis, Tensor<int8_t> *y) {
    if (axis < 0) axis += int64_t(x->shape.size());
    check(zant_hip_quantize_linear_f32_i8(default_ctx(), x->data, x->shape.data(), int(x->shape.size()), y_scale->data,
                                          y_zero_point ? y_zero_point->data : nullptr, int64_t(y_scale->size), int(axis), y->data));
}
template <typename T_out>
inline Tensor<T_out> quantize_linear(Tensor<float> *x, Tensor<float> *y_scale, Tensor<T_out> *y_zero_point, int64_t axis) {
    Tensor<T_out> y = Tensor<T_out>::fromShape(x->shape);
    quantize_linear_lean<T_out>(x, y_scale, y_zero_point, axis, &y);
    return y;
}

// dequantize_linear_lean: y = (x - x_zero_point) * x_scale; T_in: uint8_t, int8_t or int32_t
template <typename T_in>
inline void dequantize_linear_lean(Tensor<T_in> *x, Tensor<float> *x_scale, Tensor<T_in> *x_zero_point, int64_t axis,
                                   Tensor<float> *y);
#define ZANT_DEQUANT_LEAN(T_in, fn)                                                                                       \
    template <>                                                                                                           \
    inline void dequantize_linear_lean<T_in>(Tensor<T_in> * x, Tensor<float> * x_scale, Tensor<T_in> * x_zero_point,      \
                                             int64_t axis, Tensor<float> *y) {                                            \
        if (axis < 0) axis += int64_t(x->shape.size());                                                                   \
        check(fn(default_ctx(), x->data, x->shape.data(), int(x->shape.size()), x_scale->data,                            \
                 x_zero_point ? x_zero_point->data : nullptr, int64_t(x_scale->size), int(axis), y->data));               \
    }
ZANT_DEQUANT_LEAN(uint8_t, zant_hip_dequantize_linear_u8_f32)
ZANT_DEQUANT_LEAN(int8_t, zant_hip_dequantize_linear_i8_f32)
ZANT_DEQUANT_LEAN(int32_t, zant_hip_dequantize_linear_i32_f32)
#undef ZANT_DEQUANT_LEAN
template <typename T_in>
inline Tensor<float> dequantize_linear(Tensor<T_in> *x, Tensor<float> *x_scale, Tensor<T_in> *x_zero_point, int64_t axis) {
    Tensor<float> y = Tensor<float>::fromShape(x->shape);
    dequantize_linear_lean<T_in>(x, x_scale, x_zero_point, axis, &y);
    return y;
}

namespace detail {
inline void qconv_attrs(const Dims &stride, const Dims *pads, const Dims *dilations, int64_t s[2], int64_t p[4], int64_t d[2]) {
    if (stride.empty()) throw Error(ZANT_WrongStride);
    s[0] = stride[0]; s[1] = stride.size() > 1 ? stride[1] : stride[0];  // as conv_lean, op_convolution.zig:68-69
    for (int i = 0; i < 4; ++i) p[i] = 0;
    if (pads) {
        if (pads->size() < 4) throw Error(ZANT_InvalidPadding);
        for (int i = 0; i < 4; ++i) p[i] = (*pads)[size_t(i)];
    }
    d[0] = d[1] = 1;
    if (dilations && !dilations->empty()) { d[0] = (*dilations)[0]; d[1] = dilations->size() > 1 ? (*dilations)[1] : d[0]; }
}
}  // namespace detail

// qlinearconv_lean: ONNX input order (x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, B), then
// conv_lean's attributes.  The activation scales / zero points are per-tensor scalars (host values); w_scale holds one
// element or one per output channel; pads are [top, left, bottom, right]; group == channels is a depthwise convolution.
inline void qlinearconv_lean(Tensor<uint8_t> *x, float x_scale, uint8_t x_zero_point, Tensor<int8_t> *w,
                             Tensor<float> *w_scale, Tensor<int8_t> *w_zero_point, float y_scale, uint8_t y_zero_point,
                             const Tensor<int32_t> *bias, Tensor<uint8_t> *y, const Dims &stride, const Dims *pads,
                             const Dims *dilations, std::optional<int64_t> group) {
    if (x->shape.size() != 4 || w->shape.size() != 4 || y->shape.size() != 4) throw Error(ZANT_InvalidDimensions);
    int64_t s[2], p[4], d[2];
    detail::qconv_attrs(stride, pads, dilations, s, p, d);
    check(zant_hip_qlinearconv_u8i8(default_ctx(), x->data, x->shape.data(), x_scale, x_zero_point, w->data, w->shape.data(),
                                    w_scale->data, int64_t(w_scale->size), w_zero_point ? w_zero_point->data : nullptr, y_scale,
                                    y_zero_point, bias ? bias->data : nullptr, y->data, y->shape.data(), s, p, d,
                                    group ? *group : 1, ZANT_ACT_NONE, 0.0f, 1.0f, 0));
}
inline Tensor<uint8_t> qlinearconv(Tensor<uint8_t> *x, float x_scale, uint8_t x_zero_point, Tensor<int8_t> *w,
                                   Tensor<float> *w_scale, Tensor<int8_t> *w_zero_point, float y_scale, uint8_t y_zero_point,
                                   const Tensor<int32_t> *bias, const Dims &stride, const Dims *pads, const Dims *dilations,
                                   std::optional<int64_t> group) {
    if (x->shape.size() != 4 || w->shape.size() != 4) throw Error(ZANT_InvalidDimensions);
    int64_t s[2], p[4], d[2];
    detail::qconv_attrs(stride, pads, dilations, s, p, d);
    if (s[0] <= 0 || s[1] <= 0) throw Error(ZANT_WrongStride);
    const int64_t dkh = (w->shape[2] - 1) * d[0] + 1, dkw = (w->shape[3] - 1) * d[1] + 1;
    Tensor<uint8_t> y = Tensor<uint8_t>::fromShape({x->shape[0], w->shape[0], (x->shape[2] + p[0] + p[2] - dkh) / s[0] + 1,
                                                    (x->shape[3] + p[1] + p[3] - dkw) / s[1] + 1});
    qlinearconv_lean(x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, bias, &y, stride, pads, dilations, group);
    return y;
}

// Prepared weights for qlinearconv_lean (zant_hip_qlinearconv_prepack): everything weight-dependent is derived at the
// first run and kept; activations are NCHW or, between two prepared convolutions, channel-blocked.
class QLinearConvPlan {
  public:
    QLinearConvPlan(const Dims &xshape, float x_scale, uint8_t x_zero_point, Tensor<int8_t> *w, Tensor<float> *w_scale,
                    Tensor<int8_t> *w_zero_point, float y_scale, uint8_t y_zero_point, const Tensor<int32_t> *bias,
                    const Dims &yshape, const Dims &stride, const Dims *pads, const Dims *dilations, std::optional<int64_t> group,
                    int x_layout = ZANT_LAYOUT_NCHW, int y_layout = ZANT_LAYOUT_NCHW) {
        if (xshape.size() != 4 || w->shape.size() != 4 || yshape.size() != 4) throw Error(ZANT_InvalidDimensions);
        int64_t s[2], p[4], d[2];
        detail::qconv_attrs(stride, pads, dilations, s, p, d);
        check(zant_hip_qlinearconv_prepack(default_ctx(), xshape.data(), x_scale, x_zero_point, w->data, w->shape.data(),
                                           w_scale->data, int64_t(w_scale->size), w_zero_point ? w_zero_point->data : nullptr,
                                           y_scale, y_zero_point, bias ? bias->data : nullptr, yshape.data(), s, p, d,
                                           group ? *group : 1, ZANT_ACT_NONE, 0.0f, 1.0f, 0, x_layout, y_layout, &plan_));
    }
    QLinearConvPlan(const QLinearConvPlan &) = delete;
    QLinearConvPlan &operator=(const QLinearConvPlan &) = delete;
    ~QLinearConvPlan() { zant_hip_qlinearconv_plan_destroy(default_ctx(), plan_); }
    void run(const uint8_t *x, uint8_t *y) { check(zant_hip_qlinearconv_u8i8_packed(default_ctx(), plan_, x, y)); }

  private:
    zant_qconv_plan *plan_ = nullptr;
};

// Prepared weights for conv_lean (zant_hip_conv2d_f32_prepack), same attributes; fuse_act / fuse_pool: ReLU and a
// 2 x 2 / stride 2 max pool in the same kernel (yshape is then the pooled shape).
class ConvPlan {
  public:
    ConvPlan(const Dims &xshape, Tensor<float> *kernel, const Tensor<float> *bias, const Dims &yshape, const Dims &stride,
             const Dims *pads, const Dims *dilations, std::optional<int64_t> group, const char *auto_pad,
             int fuse_act = ZANT_ACT_NONE, bool fuse_pool = false) {
        if (xshape.size() != 4 || kernel->shape.size() != 4 || yshape.size() != 4) throw Error(ZANT_InvalidDimensions);
        check(zant_hip_conv2d_f32_prepack(default_ctx(), xshape.data(), kernel->data, kernel->shape.data(),
                                          bias ? bias->data : nullptr, yshape.data(), stride.data(), int(stride.size()),
                                          pads ? pads->data() : nullptr, pads ? int(pads->size()) : 0,
                                          dilations ? dilations->data() : nullptr, dilations ? int(dilations->size()) : 0,
                                          group ? *group : -1, auto_pad, fuse_act, fuse_pool ? 1 : 0, &plan_));
    }
    ConvPlan(const ConvPlan &) = delete;
    ConvPlan &operator=(const ConvPlan &) = delete;
    ~ConvPlan() { zant_hip_conv2d_plan_destroy(default_ctx(), plan_); }
    void run(const float *x, float *y) { check(zant_hip_conv2d_f32_packed(default_ctx(), plan_, x, y)); }

  private:
    zant_conv_plan *plan_ = nullptr;
};

}  // namespace tensMath
}  // namespace zant
