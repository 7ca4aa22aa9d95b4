/*
 * zant_oracle.h -- CPU restatement of Z-Ant's tensor-math hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP backend is
 * compared against; it is never linked into, imported by, or used as a
 * fallback for the product library.  Only tests, the smoke check and the
 * benchmark's CPU-baseline leg may load it.
 *
 * Every f32 function restates, loop for loop, the algorithm of the reference
 * Zig source it cites (paths relative to the reference tree).  The int8
 * family (QuantizeLinear / DequantizeLinear / QLinearConv and the fused
 * activation / add / pooling forms) has NO counterpart in the reference
 * (src/Core/Quantization/quantization.zig is empty; grouped conv is rejected
 * at op_convolution.zig:59-65): those functions restate the ONNX operator
 * definitions in exact integer arithmetic plus one fixed f32 requantisation
 * sequence, and their parity is "unpinned by the reference" -- they are
 * pinned by closed forms, brute force and library routines in the tests.
 *
 * Build: `make -C oracle` -> oracle/libzant_oracle.so (gcc -O2
 * -ffp-contract=off so that a*b+c is never fused: Zig's default float mode
 * is strict, so the reference rounds the product and the sum separately).
 */
#ifndef ZANT_ORACLE_H
#define ZANT_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes: one per Zig error the hot path can return
 * (src/Utils/errorHandler.zig:36-84).  0 = success. */
enum {
    ZO_OK = 0,
    ZO_InvalidDimensions = -1,
    ZO_InvalidPadding = -2,
    ZO_InputTensorsWrongShape = -3,
    ZO_InputTensorDifferentShape = -4,
    ZO_InputTensorDimensionMismatch = -5,
    ZO_IncompatibleBroadcastShapes = -6,
    ZO_InputTensorDifferentSize = -7,
    ZO_EmptyTensor = -8,
    ZO_ZeroSizeTensor = -9,
    ZO_InvalidInput = -10,
    ZO_InputArrayWrongSize = -11,
    ZO_WrongStride = -12,
    ZO_MemError = -13,
    ZO_InvalidAxes = -14,       /* TensorMathError.InvalidAxes */
    ZO_AxisOutOfBounds = -15,   /* TensorError.AxisOutOfBounds */
    ZO_MismatchedShape = -16,   /* TensorError.MismatchedShape */
    ZO_MismatchedRank = -17,    /* TensorError.MismatchedRank */
    ZO_EmptyTensorList = -18,   /* TensorMathError.EmptyTensorList */
    ZO_UnsupportedMode = -19    /* TensorError.UnsupportedMode */
};

/* AutoPadType, op_pooling.zig:9-14 (same numbering). */
enum { ZO_PAD_NOTSET = 0, ZO_PAD_SAME_UPPER = 1, ZO_PAD_SAME_LOWER = 2, ZO_PAD_VALID = 3 };

/* ---- f32 path (restates the reference) ---------------------------------- */

/* OnnxConvLean, op_convolution.zig:42-219.  `auto_pad` is the string the
 * reference compares against ("NOTSET", "VALID", "SAME_UPPER", "SAME_LOWER")
 * or NULL; pads are honoured only when auto_pad == "NOTSET" (:86-129).
 * n_stride / n_dil / n_pads are the slice lengths; dil / pads may be NULL.
 * group < 0 stands for Zig's `null`. */
int zo_conv_lean_f32(const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                     const float *bias, float *y, const int64_t ydim[4],
                     const int64_t *stride, int n_stride, const int64_t *pads, int n_pads,
                     const int64_t *dil, int n_dil, int64_t group, const char *auto_pad);

/* Output shape of the allocating OnnxConv wrapper, op_convolution.zig:647-745. */
int zo_conv_out_shape(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride, int n_stride,
                      const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                      const char *auto_pad, int64_t ydim[4]);

/* convolve_tensor_with_bias, op_convolution.zig:228-331 (input already padded). */
int zo_convolve_with_bias_f32(const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                              const float *bias, const int64_t stride[2], const int64_t dil[2],
                              float *y, int64_t ydim_out[4]);

/* mat_mul checks (op_mat_mul.zig:22-55) then lean_mat_mul (:92-172). */
int zo_mat_mul_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank);
int zo_mat_mul_lean_f32(const float *a, const int64_t *adim, int a_rank, const float *b, const int64_t *bdim,
                        int b_rank, float *y);

/* gemm checks (op_gemm.zig:15-61, writes the result dims) and lean_gemm (:91-185). */
int zo_gemm_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank, const int64_t *cdim,
                  int c_rank, int has_c, int trans_a, int trans_b, int64_t ydim[4]);
int zo_gemm_lean_f32(const float *a, const int64_t adim[4], const float *b, const int64_t bdim[4],
                     const float *c, const int64_t *cdim, int c_rank, float alpha, float beta, int trans_a,
                     int trans_b, float *y, const int64_t ydim[4]);

/* get_onnx_maxpool_output_shape (op_pooling.zig:477-567) and lean_onnx_maxpool (:570-659). */
int zo_maxpool_out_shape(const int64_t xdim[4], const int64_t kernel[2], const int64_t strides[2],
                         const int64_t dil[2], const int64_t pads[4], int auto_pad, int ceil_mode,
                         int64_t ydim[4]);
int zo_maxpool_lean_f32(const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4],
                        const int64_t kernel[2], const int64_t strides[2], const int64_t dil[2],
                        const int64_t *pads, int n_pads, int auto_pad);

/* lean_ReLU (lib_activation_function_math.zig:22-28): writes only where x > 0;
 * the caller's output keeps its previous content elsewhere. */
/* pool_forward, .Avg (op_pooling.zig:223-260, 373-408), extended with ONNX AveragePool's pads / count_include_pad. */
int zo_avgpool_f32(const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4], const int64_t kernel[2],
                   const int64_t strides[2], const int64_t pads[4], int count_include_pad);
/* BatchNormLayer.forward, inference branch (batchNormLayer.zig:130-148), features on axis 1. */
int zo_batchnorm_f32(const float *x, int64_t outer, int64_t features, int64_t inner, const float *gamma,
                     const float *beta, const float *mean, const float *var, float epsilon, float *y);
int zo_relu_lean_f32(const float *x, float *y, int64_t n);
/* lean_leakyReLU (:68-77). */
int zo_leaky_relu_lean_f32(const float *x, float slope, float *y, int64_t n);
/* lean_softmax (:154-187): rows = shape[0], cols = shape[1]. */
int zo_softmax_lean_f32(const float *x, float *y, int64_t rows, int64_t cols);
/* sigmoid_lean (lib_activation_function_math.zig:107-122): 1 / (1 + exp(-x)). */
int zo_sigmoid_lean_f32(const float *x, float *y, int64_t n);
/* reduce_mean + lean_reduce_mean (lib_reduction_math.zig:30-268).  axes NULL or
 * n_axes 0: identity when noop_with_empty_axes, else the mean of everything
 * (shape all ones with keepdims, else [1]).  Negative axes count from the end;
 * an axis outside the rank is InvalidAxes.  A repeated axis is InvalidAxes here
 * (the reference would square the reduced extent and read out of bounds).
 * y NULL: shape only. */
int zo_reduce_mean_f32(const float *x, const int64_t *xdim, int rank, const int64_t *axes, int n_axes, int keepdims,
                       int noop_with_empty_axes, float *y, int64_t *ydim_out, int *y_rank_out);
/* concatenate / lean_concatenate + get_concatenate_output_shape
 * (lib_shape_math.zig:307-461, 463-580, 582-630), any element width.  Lower-rank
 * inputs are padded with leading ones as lean_concatenate does (:335-358); the
 * output rank is the largest input rank.  y NULL: shape only. */
int zo_concatenate(const void *const *xs, const int64_t *const *dims, const int *ranks, int n, int64_t axis,
                   size_t elem_size, void *y, int64_t *ydim_out, int *y_rank_out);
/* resize in "nearest" mode + get_resize_output_shape (lib_shape_math.zig:22-160):
 * exactly one of scales / sizes (each of length rank); coordinate modes
 * 0 half_pixel, 1 align_corners, 2 asymmetric (anything else in the reference);
 * index = clamp(round-half-away(pos)), all in f32 as the reference computes it.
 * y NULL: shape only. */
int zo_resize_nearest(const void *x, const int64_t *xdim, int rank, size_t elem_size, const float *scales,
                      const int64_t *sizes, int n_param, int coord_mode, void *y, int64_t *ydim_out);
/* lean_sum_tensors (lib_elementWise_math.zig:70-210): same-size add, else
 * right-aligned NumPy broadcast up to rank 4.  The reference derives the
 * operand strides from the OUTPUT strides (:160-169), which indexes past the
 * end of an operand whose broadcast axis is followed by a larger axis
 * (e.g. {1,8,28,28}+{8,1,1}); the intent (ONNX Add) is restated here. */
int zo_sum_tensors_lean_f32(const float *a, const int64_t *adim, int a_rank, const float *b,
                            const int64_t *bdim, int b_rank, float *y, int64_t *ydim_out, int *y_rank_out);
/* add_bias (lib_elementWise_math.zig:22-45), in place. */
int zo_add_bias_f32(float *t, const int64_t *tdim, int t_rank, const float *bias, const int64_t *bdim, int b_rank);
/* reshape_lean (lib_shape_math.zig:1139-1209): dim 0 copies the input dim,
 * dim -1 (passed as -1 here, maxInt(usize) there) is inferred. */
int zo_reshape_lean(const void *x, const int64_t *xdim, int x_rank, size_t elem_size, const int64_t *new_shape,
                    int new_rank, void *y, int64_t *ydim_out);

/* Independent check used only to pin the restatement: 7-loop direct
 * correlation with double accumulation, explicit pads, any group. */
int zo_conv_direct_f64acc(const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                          const float *bias, float *y, const int64_t ydim[4], const int64_t stride[2],
                          const int64_t pads[4], const int64_t dil[2], int64_t group);

/* ---- int8 family (ONNX definitions; no reference counterpart) ------------ */

/* Activation applied in dequantised space between two quantised tensors. */
enum { ZO_ACT_NONE = 0, ZO_ACT_RELU = 1, ZO_ACT_LEAKY = 2, ZO_ACT_RELU6 = 3 };

/* y = sat_u8(rne(x / y_scale[c]) + y_zp[c]); per-tensor when n_scale == 1,
 * else per-axis over `axis` (ONNX QuantizeLinear). */
int zo_quantize_linear_f32_u8(const float *x, const int64_t *xdim, int rank, const float *y_scale,
                              const uint8_t *y_zp, int64_t n_scale, int axis, uint8_t *y);
/* y = (float)((int)x - x_zp[c]) * x_scale[c] (ONNX DequantizeLinear). */
int zo_dequantize_linear_u8_f32(const uint8_t *x, const int64_t *xdim, int rank, const float *x_scale,
                                const uint8_t *x_zp, int64_t n_scale, int axis, float *y);

/* ONNX QLinearConv, u8 activations x i8 weights -> i32 -> u8.
 * acc = sum (x - x_zp) * (w - w_zp[k]) + B[k] (padding contributes 0);
 * y = sat_u8(rne((float)acc * M[k]) + y_zp), M[k] = (x_scale * w_scale[k]) / y_scale in f32.
 * w_scale has n_wscale entries (1 = per tensor, K = per channel); w_zp may be NULL (= 0).
 * Explicit pads [top,left,bottom,right]; any group dividing C and K.
 * act/act_*: optional fused DequantizeLinear -> activation -> QuantizeLinear
 * applied to the u8 result: q2 = sat_u8(rne(f((q - y_zp) * y_scale) / act_scale) + act_zp). */
int zo_qlinearconv_u8i8(const uint8_t *x, const int64_t xdim[4], float x_scale, uint8_t x_zp,
                        const int8_t *w, const int64_t wdim[4], const float *w_scale, int64_t n_wscale,
                        const int8_t *w_zp, float y_scale, uint8_t y_zp, const int32_t *bias, uint8_t *y,
                        const int64_t ydim[4], const int64_t stride[2], const int64_t pads[4],
                        const int64_t dil[2], int64_t group, int act, float act_alpha, float act_scale,
                        uint8_t act_zp);
/* The int32 accumulator alone (before requantisation). */
int zo_qconv_acc_i32(const uint8_t *x, const int64_t xdim[4], uint8_t x_zp, const int8_t *w,
                     const int64_t wdim[4], const int8_t *w_zp, const int32_t *bias, int32_t *acc,
                     const int64_t ydim[4], const int64_t stride[2], const int64_t pads[4],
                     const int64_t dil[2], int64_t group);

/* DequantizeLinear -> {none,ReLU,LeakyReLU(alpha),ReLU6} -> QuantizeLinear, elementwise. */
int zo_qlinear_act_u8(const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act, float alpha,
                      float y_scale, uint8_t y_zp, uint8_t *y);
/* DequantizeLinear(a) + DequantizeLinear(b) -> QuantizeLinear (same shape). */
int zo_qlinear_add_u8(const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b, float b_scale,
                      uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n);
/* MaxPool on quantised values (order preserving => exact); windows with no
 * in-bounds tap yield 0, the minimum of the type. */
int zo_maxpool_lean_u8(const uint8_t *x, const int64_t xdim[4], uint8_t *y, const int64_t ydim[4],
                       const int64_t kernel[2], const int64_t strides[2], const int64_t dil[2],
                       const int64_t *pads, int n_pads, int auto_pad);
/* Global average pool of a quantised NCHW tensor -> [N,C,1,1]:
 * s = sum(q - x_zp) exact in i32; y = sat_u8(rne((((float)s * x_scale) / (float)(H*W)) / y_scale) + y_zp). */
int zo_qlinear_global_avgpool_u8(const uint8_t *x, const int64_t xdim[4], float x_scale, uint8_t x_zp,
                                 float y_scale, uint8_t y_zp, uint8_t *y);

const char *zo_error_name(int code);

#ifdef __cplusplus
}
#endif
#endif
