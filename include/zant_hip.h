/*
 * zant_hip.h -- C ABI of the MI355X (gfx950) backend for Z-Ant's tensor-math hot path.
 *
 * One shared library (libzant_hip.so), plain pointers and sizes only.  Every
 * operator entry point mirrors one `*_lean` function of the reference
 * (src/Core/Tensor/TensorMath/tensor_math_standard.zig:43-149): the caller owns
 * and pre-shapes the output, the call validates, enqueues hand-written HIP
 * kernels on the context's stream and returns a status.  Tensor arguments are
 * DEVICE pointers (row-major, contiguous, NCHW for rank 4); shape / attribute
 * arrays are HOST pointers.  A Zig `Tensor(T)` is not `extern` (tensor.zig:25-31),
 * so the Zig wrapper passes `t.data.ptr` and a copy of `t.shape`.
 *
 * Status codes: 0 = ok; negative values name the Zig error the reference would
 * return (src/Utils/errorHandler.zig:36-84) so the wrapper can map them back and
 * the generated `predict()` keeps its `catch return` behaviour
 * (src/codeGen/math_handler.zig:107).  The library never aborts.
 *
 * Threading: one zant_ctx = one HIP stream; use one context per host thread.
 * Calls are asynchronous; zant_hip_sync() waits for the stream.
 */
#ifndef ZANT_HIP_H
#define ZANT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct zant_ctx zant_ctx;
typedef struct zant_model zant_model;

enum zant_status {
    ZANT_OK = 0,
    ZANT_InvalidDimensions = -1,            /* TensorMathError.InvalidDimensions */
    ZANT_InvalidPadding = -2,               /* TensorMathError.InvalidPadding */
    ZANT_InputTensorsWrongShape = -3,       /* TensorMathError.InputTensorsWrongShape */
    ZANT_InputTensorDifferentShape = -4,    /* TensorMathError.InputTensorDifferentShape */
    ZANT_InputTensorDimensionMismatch = -5, /* TensorMathError.InputTensorDimensionMismatch */
    ZANT_IncompatibleBroadcastShapes = -6,  /* TensorMathError.IncompatibleBroadcastShapes */
    ZANT_InputTensorDifferentSize = -7,     /* TensorMathError.InputTensorDifferentSize */
    ZANT_EmptyTensor = -8,                  /* TensorError.EmptyTensor */
    ZANT_ZeroSizeTensor = -9,               /* TensorError.ZeroSizeTensor */
    ZANT_InvalidInput = -10,                /* TensorError.InvalidInput */
    ZANT_InputArrayWrongSize = -11,         /* TensorError.InputArrayWrongSize */
    ZANT_WrongStride = -12,                 /* TensorMathError.WrongStride */
    ZANT_MemError = -13,                    /* TensorMathError.MemError (host or device allocation) */
    ZANT_InvalidAxes = -14,                 /* TensorMathError.InvalidAxes */
    ZANT_AxisOutOfBounds = -15,             /* TensorError.AxisOutOfBounds */
    ZANT_MismatchedShape = -16,             /* TensorError.MismatchedShape */
    ZANT_MismatchedRank = -17,              /* TensorError.MismatchedRank */
    ZANT_EmptyTensorList = -18,             /* TensorMathError.EmptyTensorList */
    ZANT_UnsupportedMode = -19,             /* TensorError.UnsupportedMode */
    ZANT_HipError = -100,                   /* a HIP runtime call failed; see zant_hip_last_error() */
    ZANT_NullPointer = -101,
    ZANT_ArenaOverflow = -102,
    ZANT_NotFinalized = -103
};

/* AutoPadType of MaxPool, src/Core/Tensor/TensorMath/op_pooling.zig:9-14. */
enum zant_auto_pad { ZANT_PAD_NOTSET = 0, ZANT_PAD_SAME_UPPER = 1, ZANT_PAD_SAME_LOWER = 2, ZANT_PAD_VALID = 3 };

/* Activation fused into a producing kernel, or applied in dequantised space
 * between two quantised tensors. */
enum zant_act { ZANT_ACT_NONE = 0, ZANT_ACT_RELU = 1, ZANT_ACT_LEAKY = 2, ZANT_ACT_RELU6 = 3,
                ZANT_ACT_SOFTMAX = 4 /* zant_hip_gemm_f32 only: lean_softmax over every output row */ };

/* ---- context, memory, timing ------------------------------------------------ */

/* Creates a context on `device`.  `stream` is a hipStream_t to enqueue on, or
 * NULL to let the context create (and own) a stream at default priority. */
int zant_hip_ctx_create(zant_ctx **out, int device, void *stream);
void zant_hip_ctx_destroy(zant_ctx *ctx);
int zant_hip_sync(zant_ctx *ctx);
const char *zant_hip_status_name(int status);
const char *zant_hip_last_error(zant_ctx *ctx); /* ctx == NULL: the calling thread's last failed zant_hip_ctx_create */
const char *zant_hip_version(void);

/* Replaces setLogFunctionC (src/Core/Tensor/TensorMath/op_convolution.zig:37-41)
 * and the generated library's setLogFunction (src/codeGen/skeleton.zig:93-97). */
void setLogFunctionC(void (*func)(char *));
#ifndef ZANT_HIP_NO_PREDICT_DECL
void setLogFunction(void (*func)(char *));
#endif

/* The activation arena: ONE device allocation that model-level forward passes
 * carve their tensors from (the reference keeps one static array per node
 * output, src/codeGen/predict.zig:265-272).  Reserving again grows it. */
int zant_hip_arena_reserve(zant_ctx *ctx, size_t bytes);
void *zant_hip_arena_ptr(zant_ctx *ctx, size_t offset);
size_t zant_hip_arena_size(zant_ctx *ctx);

int zant_hip_malloc(zant_ctx *ctx, void **dev_ptr, size_t bytes);
int zant_hip_free(zant_ctx *ctx, void *dev_ptr);
int zant_hip_upload(zant_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int zant_hip_download(zant_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
int zant_hip_memset(zant_ctx *ctx, void *dst_dev, int byte_value, size_t bytes);

/* HIP-event stopwatch on the context's stream (what the benchmark times kernels with). */
int zant_hip_timer_start(zant_ctx *ctx);
int zant_hip_timer_stop(zant_ctx *ctx, float *elapsed_ms);
/* Per-kernel timing: while enabled, every operator brackets its MAIN kernel launch (not its small
 * weight-packing helpers) with HIP events on the context's stream; zant_hip_kernel_ms() waits for
 * the most recent one and returns its duration.  Off by default (two event records per call). */
int zant_hip_kernel_timing(zant_ctx *ctx, int enable);
int zant_hip_kernel_ms(zant_ctx *ctx, float *elapsed_ms);
/* The device function of the most recent operator's main kernel as a profiler's kernel trace names it, with its
 * template arguments (e.g. "conv_f32_mfma_kernel<4,2,2,4,9,true,true>"); "" where the launch site does not say.  The
 * string lives in the context and changes with the next operator call. */
const char *zant_hip_kernel_name(zant_ctx *ctx);

/* ---- f32 operators ------------------------------------------------------------ */

/* conv_lean = OnnxConvLean (op_convolution.zig:42-219).  stride/pads/dil are the
 * Zig slices (pointer + length; pads/dil may be NULL = Zig null); group < 0 = null;
 * auto_pad is the string the reference compares ("NOTSET", "VALID", "SAME_UPPER",
 * "SAME_LOWER") or NULL.  As in the reference, pads are honoured only under
 * "NOTSET" and group must be 1 or null.  fuse_act: ZANT_ACT_NONE, or
 * ZANT_ACT_RELU to apply ReLU_lean to the result in the same kernel. */
int zant_hip_conv2d_f32(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w,
                        const int64_t wdim[4], const float *bias, float *y, const int64_t ydim[4],
                        const int64_t *stride, int n_stride, const int64_t *pads, int n_pads,
                        const int64_t *dil, int n_dil, int64_t group, const char *auto_pad, int fuse_act);
/* Shape the allocating wrapper OnnxConv expects (op_convolution.zig:647-732). Host only. */
int zant_hip_conv2d_out_shape(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride, int n_stride,
                              const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                              const char *auto_pad, int64_t ydim[4]);

/* zant_hip_conv2d_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, checks
 * and results; the tiled kernel's scratch (packed weights and two tile counters, which zant_hip_conv2d_f32
 * keeps in a context workspace it grows with hipMalloc) lives in a static device array of
 * ZANT_HIP_STATIC_SCRATCH_BYTES that every device the library runs on holds until the process ends.  The call
 * performs no hipMalloc / hipFree.  A convolution whose packed weights (K and C rounded up to the tile, x KH x KW
 * x 4 bytes, + 256) exceed the array returns ZANT_ArenaOverflow and launches nothing; zant_hip_last_error()
 * gives both sizes.  Every call on a device shares that device's array: calls on one stream may follow each
 * other freely (each re-packs the weights and re-arms the counters in stream order), calls that overlap on one
 * device (several contexts or streams) race. */
#define ZANT_HIP_STATIC_SCRATCH_BYTES (8u << 20)
int zant_hip_conv2d_f32_static(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w,
                               const int64_t wdim[4], const float *bias, float *y, const int64_t ydim[4],
                               const int64_t *stride, int n_stride, const int64_t *pads, int n_pads,
                               const int64_t *dil, int n_dil, int64_t group, const char *auto_pad, int fuse_act);

/* Prepared weights for zant_hip_conv2d_f32.  The reference's conv_lean takes the weights on every call
 * (op_convolution.zig:42), so zant_hip_conv2d_f32 has to assume they changed and re-packs them for the
 * matrix-core kernel each time.  A plan fixes shapes, attributes (same meaning and checks as zant_hip_conv2d_f32,
 * made here) and the weight / bias tensors once: the first zant_hip_conv2d_f32_packed packs into memory the plan
 * owns, later calls launch the convolution kernel only.  w and bias are DEVICE pointers that must stay valid and
 * unchanged while the plan lives.  Destroy the plan before its context.
 * fuse_pool != 0: the plan is Conv (-> ReLU with fuse_act) -> onnx_maxpool_lean with a 2 x 2 kernel, stride 2, no padding,
 * floor mode (op_pooling.zig:570-659) in ONE kernel -- what a code generator that peephole-fuses the chain emits
 * (hardcoded_mnist8.zig:186-268 is such a chain); ydim is then the pooled shape.  Taken for stride 1, dilation 1 and
 * the shapes whose convolution kernel has the pooled epilogue (8 or more input channels, or a 1- / 3-channel 3x3 or a
 * 1-channel 5x5 first layer); other shapes return ZANT_InvalidInput and the caller issues the two operators. */
typedef struct zant_conv_plan zant_conv_plan;
int zant_hip_conv2d_f32_prepack(zant_ctx *ctx, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                                const float *bias, const int64_t ydim[4], const int64_t *stride, int n_stride,
                                const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                                const char *auto_pad, int fuse_act, int fuse_pool, zant_conv_plan **out);
int zant_hip_conv2d_f32_packed(zant_ctx *ctx, zant_conv_plan *plan, const float *x, float *y);
void zant_hip_conv2d_plan_destroy(zant_ctx *ctx, zant_conv_plan *plan);

/* mat_mul_lean = lean_mat_mul (op_mat_mul.zig:92-172): last two dims only. */
int zant_hip_matmul_f32(zant_ctx *ctx, const float *a, const int64_t *adim, int a_rank, const float *b,
                        const int64_t *bdim, int b_rank, float *y);
/* The checks of the allocating mat_mul (op_mat_mul.zig:22-55). Host only. */
int zant_hip_matmul_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank);

/* gemm_lean = lean_gemm (op_gemm.zig:91-185): Y = alpha*op(A)*op(B) + beta*C on
 * {1,1,R,C} tensors, C broadcast over rows and/or columns.  Transposes are folded
 * into the loads.  fuse_act as for conv; ZANT_ACT_SOFTMAX (the classifier head Gemm -> Softmax in one kernel,
 * lean_softmax, lib_activation_function_math.zig:154-187, on the [rows, cols] result) is accepted for cols <= 16 without trans_a
 * and returns InvalidInput otherwise. */
int zant_hip_gemm_f32(zant_ctx *ctx, const float *a, const int64_t adim[4], const float *b, const int64_t bdim[4],
                      const float *c, const int64_t *cdim, int c_rank, float alpha, float beta, int trans_a,
                      int trans_b, float *y, const int64_t ydim[4], int fuse_act);
/* The checks of the allocating gemm (op_gemm.zig:15-61); writes the result dims. Host only. */
int zant_hip_gemm_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank, const int64_t *cdim,
                        int c_rank, int has_c, int trans_a, int trans_b, int64_t ydim[4]);

/* onnx_maxpool_lean = lean_onnx_maxpool (op_pooling.zig:570-659) and its shape
 * function get_onnx_maxpool_output_shape (:477-567, host only). */
int zant_hip_maxpool2d_f32(zant_ctx *ctx, const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4],
                           const int64_t kernel[2], const int64_t strides[2], const int64_t dil[2],
                           const int64_t *pads, int n_pads, int auto_pad);
int zant_hip_maxpool2d_out_shape(const int64_t xdim[4], const int64_t kernel[2], const int64_t strides[2],
                                 const int64_t dil[2], const int64_t pads[4], int auto_pad, int ceil_mode,
                                 int64_t ydim[4]);

/* Average pooling: pool_forward with PoolingType.Avg (op_pooling.zig:223-260, 373-408): per window the sum of
 * the taps inside the input, in (row, column) order, divided by their count.  The reference takes no padding;
 * pads [top, left, bottom, right] (NULL = none, each smaller than the kernel) and count_include_pad extend it to
 * ONNX AveragePool: with count_include_pad the divisor is the number of taps inside the PADDED input.  The
 * shape function gives pool_forward's (H - k) / s + 1 over the padded input, with ONNX's ceil_mode (host only). */
int zant_hip_avgpool2d_f32(zant_ctx *ctx, const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4],
                           const int64_t kernel[2], const int64_t strides[2], const int64_t pads[4],
                           int count_include_pad);
int zant_hip_avgpool2d_out_shape(const int64_t xdim[4], const int64_t kernel[2], const int64_t strides[2],
                                 const int64_t pads[4], int ceil_mode, int64_t ydim[4]);
/* BatchNormalization, inference form: BatchNormLayer.forward with is_training false
 * (src/Model/Layers/batchNormLayer.zig:130-148): y = (x - mean[f]) / sqrt(var[f] + epsilon) * gamma[f] + beta[f]
 * in that order of operations, f the index on axis 1 (the reference's layer takes [batch, features]; any rank
 * 2..8 here, as ONNX BatchNormalization on NCHW needs).  gamma, beta, mean, var: device arrays of xdim[1]. */
int zant_hip_batchnorm_f32(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank, const float *gamma,
                           const float *beta, const float *mean, const float *var, float epsilon, float *y);

/* ReLU_lean (lib_activation_function_math.zig:22-28).  The reference writes only
 * where x > 0 and relies on a zeroed output; this writes x > 0 ? x : 0 everywhere,
 * which is the same result on the zeroed outputs the reference always passes. */
int zant_hip_relu_f32(zant_ctx *ctx, const float *x, float *y, int64_t n);
/* leakyReLU_lean (:68-77): x <= 0 ? slope*x : x. */
int zant_hip_leaky_relu_f32(zant_ctx *ctx, const float *x, float slope, float *y, int64_t n);
/* sigmoid_lean (:107-122): 1 / (1 + exp(-x)). */
int zant_hip_sigmoid_f32(zant_ctx *ctx, const float *x, float *y, int64_t n);
/* softmax_lean (:154-187): rows = shape[0], cols = shape[1]. */
int zant_hip_softmax_f32(zant_ctx *ctx, const float *x, float *y, int64_t rows, int64_t cols);
/* sum_tensors_lean (lib_elementWise_math.zig:70-210): same-size add, else
 * right-aligned NumPy broadcast (rank <= 8).  Writes the output shape when
 * ydim_out is not NULL. */
int zant_hip_add_f32(zant_ctx *ctx, const float *a, const int64_t *adim, int a_rank, const float *b,
                     const int64_t *bdim, int b_rank, float *y, int64_t *ydim_out, int *y_rank_out);
/* add_bias (lib_elementWise_math.zig:22-45), in place over the last axis. */
int zant_hip_add_bias_f32(zant_ctx *ctx, float *t, const int64_t *tdim, int t_rank, const float *bias,
                          const int64_t *bdim, int b_rank);
/* reduce_mean / lean_reduce_mean (lib_reduction_math.zig:30-268).  axes NULL or
 * n_axes 0: a copy when noop_with_empty_axes, else the mean of everything (shape
 * all ones with keepdims, else [1]).  Negative axes count from the end; an axis
 * outside the rank, or named twice, is ZANT_InvalidAxes.  The output shape goes
 * to ydim_out / y_rank_out (room for 8); y == NULL asks for the shape only.
 * Sums run in f32 like the reference's, in a different order (tree / lanes). */
int zant_hip_reduce_mean_f32(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank, const int64_t *axes,
                             int n_axes, int keepdims, int noop_with_empty_axes, float *y, int64_t *ydim_out,
                             int *y_rank_out);
/* concatenate / lean_concatenate and get_concatenate_output_shape
 * (lib_shape_math.zig:307-461, 463-580, 582-630) for elements of 1, 2, 4 or 8
 * bytes, up to 16 inputs.  Lower-rank inputs get leading ones as in
 * lean_concatenate (:335-358).  y == NULL asks for the shape only. */
int zant_hip_concatenate(zant_ctx *ctx, const void *const *xs, const int64_t *const *dims, const int *ranks, int n,
                         int64_t axis, size_t elem_size, void *y, int64_t *ydim_out, int *y_rank_out);
/* resize(mode "nearest") and get_resize_output_shape (lib_shape_math.zig:22-160):
 * exactly one of scales / sizes, each of length rank (else ZANT_InvalidInput);
 * coord_mode 0 half_pixel, 1 align_corners, anything else asymmetric, as the
 * reference's string comparison falls through; indices computed in f32 and
 * rounded half away from zero, as there.  Elements of 1, 2, 4 or 8 bytes.
 * The "linear" and "cubic" modes are not provided.  y == NULL: shape only. */
int zant_hip_resize_nearest(zant_ctx *ctx, const void *x, const int64_t *xdim, int rank, size_t elem_size,
                            const float *scales, const int64_t *sizes, int n_param, int coord_mode, void *y,
                            int64_t *ydim_out);
/* reshape_lean (lib_shape_math.zig:1139-1209): resolves 0 / -1 entries into
 * ydim_out and copies the data unless y == x (a view). */
int zant_hip_reshape(zant_ctx *ctx, const void *x, const int64_t *xdim, int x_rank, size_t elem_size,
                     const int64_t *new_shape, int new_rank, void *y, int64_t *ydim_out);

/* ---- int8 operators (ONNX definitions; the reference has none) ----------------- */

/* QuantizeLinear: y = sat_u8(rne(x / y_scale[c]) + y_zp[c]); n_scale == 1 per tensor,
 * else per `axis`.  y_scale / y_zp are device pointers (y_zp may be NULL = 0). */
int zant_hip_quantize_linear_f32_u8(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank,
                                    const float *y_scale, const uint8_t *y_zp, int64_t n_scale, int axis,
                                    uint8_t *y);
/* DequantizeLinear: y = (x - x_zp[c]) * x_scale[c]. */
int zant_hip_dequantize_linear_u8_f32(zant_ctx *ctx, const uint8_t *x, const int64_t *xdim, int rank,
                                      const float *x_scale, const uint8_t *x_zp, int64_t n_scale, int axis,
                                      float *y);
/* The same operators for the other code types ONNX defines: int8 codes (saturating to [-128, 127]) and
 * DequantizeLinear of int32 (accumulators, biases).  The zero point has the code type. */
int zant_hip_quantize_linear_f32_i8(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank,
                                    const float *y_scale, const int8_t *y_zp, int64_t n_scale, int axis,
                                    int8_t *y);
int zant_hip_dequantize_linear_i8_f32(zant_ctx *ctx, const int8_t *x, const int64_t *xdim, int rank,
                                      const float *x_scale, const int8_t *x_zp, int64_t n_scale, int axis,
                                      float *y);
int zant_hip_dequantize_linear_i32_f32(zant_ctx *ctx, const int32_t *x, const int64_t *xdim, int rank,
                                       const float *x_scale, const int32_t *x_zp, int64_t n_scale, int axis,
                                       float *y);
/* QLinearConv (u8 x i8 -> i32 -> u8), explicit pads [top,left,bottom,right], any
 * group dividing C and K (group == C: depthwise).  w_scale (n_wscale = 1 or K),
 * w_zp (NULL = 0) and bias (NULL = 0) are device pointers; activation scales and
 * zero points are host scalars.  Requantisation:
 *   y = sat_u8(rne((float)acc * ((x_scale * w_scale[k]) / y_scale)) + y_zp)
 * then, when act != ZANT_ACT_NONE, the fused DequantizeLinear -> act -> QuantizeLinear:
 *   y = sat_u8(rne(act((y - y_zp) * y_scale) / act_scale) + act_zp). */
int zant_hip_qlinearconv_u8i8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale,
                              uint8_t x_zp, const int8_t *w, const int64_t wdim[4], const float *w_scale,
                              int64_t n_wscale, const int8_t *w_zp, float y_scale, uint8_t y_zp,
                              const int32_t *bias, uint8_t *y, const int64_t ydim[4], const int64_t stride[2],
                              const int64_t pads[4], const int64_t dil[2], int64_t group, int act,
                              float act_alpha, float act_scale, uint8_t act_zp);
/* Layouts of a u8 activation tensor [N, C, H, W].  ZANT_LAYOUT_NCHW is the reference's row-major layout, the only one
 * the lean operators above take.  ZANT_LAYOUT_BLOCKED16 is what the int8 matrix-core kernels read and write natively:
 * [N][ceil(C/16)][H][W][16] bytes, each holding value ^ 0x80 (zant_hip_blocked16_bytes() bytes in all; bytes of
 * channels >= C are unspecified).  A caller that chains prepared convolutions keeps its activations blocked and
 * converts only at the ends. */
enum zant_layout { ZANT_LAYOUT_NCHW = 0, ZANT_LAYOUT_BLOCKED16 = 1 };
size_t zant_hip_blocked16_bytes(const int64_t dim[4]);
int zant_hip_to_blocked16_u8(zant_ctx *ctx, const uint8_t *x, const int64_t dim[4], uint8_t *x_blocked);
int zant_hip_from_blocked16_u8(zant_ctx *ctx, const uint8_t *x_blocked, const int64_t dim[4], uint8_t *y);
/* Prepared weights for zant_hip_qlinearconv_u8i8 (no counterpart in the reference, whose operators take the weights on
 * every call).  Arguments, checks and results are those of zant_hip_qlinearconv_u8i8, made once here; x_layout /
 * y_layout say how the activations handed to zant_hip_qlinearconv_u8i8_packed are laid out.  The first packed call
 * derives everything weight-dependent (packed weights, requantisation multipliers and corrections) into memory the
 * plan owns; later calls launch the convolution kernel only, and with blocked activations no layout conversion
 * either.  w, w_scale, w_zp and bias are DEVICE pointers that must stay valid and unchanged while the plan lives.
 * Destroy the plan before its context. */
typedef struct zant_qconv_plan zant_qconv_plan;
int zant_hip_qlinearconv_prepack(zant_ctx *ctx, const int64_t xdim[4], float x_scale, uint8_t x_zp, const int8_t *w,
                                 const int64_t wdim[4], const float *w_scale, int64_t n_wscale, const int8_t *w_zp,
                                 float y_scale, uint8_t y_zp, const int32_t *bias, const int64_t ydim[4],
                                 const int64_t stride[2], const int64_t pads[4], const int64_t dil[2], int64_t group,
                                 int act, float act_alpha, float act_scale, uint8_t act_zp, int x_layout, int y_layout,
                                 zant_qconv_plan **out);
int zant_hip_qlinearconv_u8i8_packed(zant_ctx *ctx, zant_qconv_plan *plan, const uint8_t *x, uint8_t *y);
void zant_hip_qlinearconv_plan_destroy(zant_ctx *ctx, zant_qconv_plan *plan);
/* DequantizeLinear -> {none, ReLU, LeakyReLU(alpha), ReLU6} -> QuantizeLinear. */
int zant_hip_qlinear_act_u8(zant_ctx *ctx, const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act,
                            float alpha, float y_scale, uint8_t y_zp, uint8_t *y);
/* DequantizeLinear(a) + DequantizeLinear(b) -> QuantizeLinear, same shape. */
int zant_hip_qlinear_add_u8(zant_ctx *ctx, const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b,
                            float b_scale, uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n);
/* MaxPool on quantised values (same window rules as zant_hip_maxpool2d_f32). */
int zant_hip_maxpool2d_u8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], uint8_t *y,
                          const int64_t ydim[4], const int64_t kernel[2], const int64_t strides[2],
                          const int64_t dil[2], const int64_t *pads, int n_pads, int auto_pad);
/* Global average pool of a quantised NCHW tensor -> [N,C,1,1]. */
int zant_hip_qlinear_global_avgpool_u8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale,
                                       uint8_t x_zp, float y_scale, uint8_t y_zp, uint8_t *y);

/* ---- generated-library level: a whole network in one preallocated arena -------- */

/* The reference's code generator emits one static array per node output, a
 * straight-line predict() that calls one *_lean operator per ONNX node, and a
 * compiled-in input shape (src/codeGen/predict.zig:23-70, 265-377).  A zant_model
 * is the GPU form of such a generated library: nodes are appended in ready order
 * (src/codeGen/utils.zig:114-135), parameters are copied to the device once, and
 * zant_model_finalize() fuses activations into their producers, turns Reshape
 * into a view and assigns every activation an offset in ONE arena allocation by
 * liveness, so that zant_model_run() performs no device allocation at all.
 * Tensor handles are small non-negative ints; a negative return is a zant_status. */
enum zant_dtype { ZANT_F32 = 0, ZANT_U8 = 1 };

/* ctx == NULL creates a dry-run model: nodes are validated and shapes can be queried (zant_model_tensor_dims,
 * zant_model_output_dims) without touching a GPU, as a code generator needs; zant_model_finalize refuses it. */
int zant_model_create(zant_ctx *ctx, zant_model **out);
void zant_model_destroy(zant_model *m);
/* The network input (batch compiled in, like the reference).  scale / zp describe a u8 input. */
int zant_model_input(zant_model *m, int dtype, const int64_t *dims, int rank, float scale, int zp);
/* f32 nodes; w / bias / b / c are HOST pointers copied at finalize. */
int zant_model_conv(zant_model *m, int x, const float *w, const int64_t wdim[4], const float *bias,
                    const int64_t *stride, int n_stride, const int64_t *pads, int n_pads, const int64_t *dil,
                    int n_dil, int64_t group, const char *auto_pad);
int zant_model_relu(zant_model *m, int x);
int zant_model_leaky_relu(zant_model *m, int x, float slope);
int zant_model_maxpool(zant_model *m, int x, const int64_t kernel[2], const int64_t strides[2],
                       const int64_t dil[2], const int64_t pads[4], int auto_pad, int ceil_mode);
/* AveragePool (zant_hip_avgpool2d_f32); pads may be NULL. */
int zant_model_avgpool(zant_model *m, int x, const int64_t kernel[2], const int64_t strides[2], const int64_t pads[4],
                       int ceil_mode, int count_include_pad);
/* BatchNormalization, inference form (zant_hip_batchnorm_f32); gamma / beta / mean / var are HOST arrays of
 * `features` = dims[1] floats.  Behind a convolution that nothing else reads, finalize folds it into the
 * convolution's weights and bias (w * s, (b - mean) * s + beta with s = gamma / sqrt(var + epsilon)). */
int zant_model_batchnorm(zant_model *m, int x, const float *gamma, const float *beta, const float *mean,
                         const float *var, int64_t features, float epsilon);
int zant_model_reshape(zant_model *m, int x, const int64_t *new_shape, int rank);
int zant_model_gemm(zant_model *m, int a, const float *b, const int64_t bdim[4], const float *c,
                    const int64_t *cdim, int c_rank, float alpha, float beta, int trans_a, int trans_b);
int zant_model_matmul(zant_model *m, int a, const float *b, const int64_t *bdim, int b_rank);
int zant_model_add_const(zant_model *m, int x, const float *c, const int64_t *cdim, int c_rank);
int zant_model_add(zant_model *m, int a, int b);
int zant_model_softmax(zant_model *m, int x);
int zant_model_sigmoid(zant_model *m, int x);
/* ReduceMean over the given axes (GlobalAveragePool is axes {2, 3} with keepdims). */
int zant_model_reduce_mean(zant_model *m, int x, const int64_t *axes, int n_axes, int keepdims);
/* Concat of up to 16 tensors of one element type; quantised inputs must share scale and zero point. */
int zant_model_concat(zant_model *m, const int *xs, int n, int64_t axis);
/* Resize, "nearest" mode: exactly one of scales / sizes (length = rank), coord_mode as zant_hip_resize_nearest. */
int zant_model_resize_nearest(zant_model *m, int x, const float *scales, const int64_t *sizes, int n_param,
                              int coord_mode);
/* int8 nodes; activation scales / zero points are tracked per tensor. */
int zant_model_quantize(zant_model *m, int x, float y_scale, int y_zp);
int zant_model_dequantize(zant_model *m, int x);
int zant_model_qlinearconv(zant_model *m, int x, const int8_t *w, const int64_t wdim[4], const float *w_scale,
                           int64_t n_wscale, const int32_t *bias, float y_scale, int y_zp,
                           const int64_t stride[2], const int64_t pads[4], const int64_t dil[2], int64_t group);
int zant_model_qlinear_act(zant_model *m, int x, int act, float alpha, float y_scale, int y_zp);
int zant_model_qlinear_add(zant_model *m, int a, int b, float y_scale, int y_zp);
int zant_model_qlinear_global_avgpool(zant_model *m, int x, float y_scale, int y_zp);
/* Fuses, plans the arena (reserved on the context), uploads parameters.  The last node's output is
 * the network output. */
int zant_model_finalize(zant_model *m);
int zant_model_output_dims(zant_model *m, int64_t *dims, int *rank, int *dtype);
/* Shape (room for 8 dims) and element type of any tensor id handed out by the builder calls. */
int zant_model_tensor_dims(zant_model *m, int tensor, int64_t *dims, int *rank, int *dtype);
size_t zant_model_arena_bytes(zant_model *m);   /* planned arena size */
size_t zant_model_unfused_bytes(zant_model *m); /* sum of all node outputs, the reference's static arrays */
int zant_model_num_launches(zant_model *m);     /* operator calls per run after fusion */
/* One forward pass, device in / device out, asynchronous, no allocation.  input_dev == NULL means the
 * caller already wrote the input at zant_model_input_ptr(); output_dev == NULL leaves the result at
 * zant_model_output_ptr() (both inside the arena, valid after finalize).  A pass does not write to the
 * input's storage: an input placed at zant_model_input_ptr() once serves any number of passes. */
int zant_model_run(zant_model *m, const void *input_dev, void *output_dev);
void *zant_model_input_ptr(zant_model *m);
void *zant_model_output_ptr(zant_model *m);
/* Host in / host out: upload, run, download (synchronous). */
int zant_model_predict_host(zant_model *m, const void *input_host, void *output_host);
/* One pass with per-kernel timing: fills, for each kernel-launching node in execution order, the
 * duration of its main kernel (ms), its algorithmic work (flops or integer ops; 0 for data movement)
 * and its algorithmic bytes (inputs + parameters + output, each once).  Returns the number of entries
 * written (at most `capacity`) or a negative status.  zant_model_launch_name() names entry i, e.g.
 * "Conv+Relu+MaxPool". */
int zant_model_profile(zant_model *m, float *ms, double *ops, double *bytes, int capacity);
const char *zant_model_launch_name(zant_model *m, int i);
/* The device function behind entry i of the last zant_model_profile (see zant_hip_kernel_name); "" before it. */
const char *zant_model_launch_kernel(zant_model *m, int i);
/* Debug: copies tensor `id` to the host: replays the last pass up to the node that produces it (its storage may have
 * been planned under a later tensor), reads it from the arena, then replays the rest of the pass, so that afterwards
 * the arena -- zant_model_output_ptr() included -- holds the last pass's result again.  It costs a whole pass and, like
 * a pass, overwrites the per-kernel figures of an earlier zant_model_profile.  Tensors that a fusion removed (the
 * output of a convolution whose pool, or of a residual block's inner layers, run in the same kernel) are never
 * materialised: ZANT_InvalidInput. */
int zant_model_read_tensor(zant_model *m, int id, void *dst_host, size_t bytes);

/* The reference's exported entry point (src/codeGen/predict.zig:34-39), served by the bound model:
 * silent return when shape_len is 0, differs from the model's rank, or a dimension differs
 * (predict.zig:317-335); otherwise *result points at library-owned host storage that stays valid
 * until the next call. */
int zant_model_bind_predict(zant_model *m);
/* A generated library defines predict / setLogFunction itself, typed by its network's element types (the reference's
 * comptime T); it defines ZANT_HIP_NO_PREDICT_DECL before including this file. */
#ifndef ZANT_HIP_NO_PREDICT_DECL
void predict(float *input, uint32_t *input_shape, uint32_t shape_len, float **result);
#endif
/* predict() for callers that only know the batch: `n` must equal the leading dimension the bound model was built
 * with (the reference compiles the batch into predict's shape check, predict.zig:328-334); otherwise it returns
 * silently with *result untouched, as predict does.  No counterpart in the reference: it exists for the batched
 * measurements (batch 4096 / 512 / 1024). */
void predict_batched(float *input, uint32_t n, float **result);

#ifdef __cplusplus
}
#endif
#endif /* ZANT_HIP_H */
