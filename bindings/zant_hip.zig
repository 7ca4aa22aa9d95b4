//! tensor_math_hip.zig -- Zig binding of libzant_hip.so (include/zant_hip.h) for Z-Ant.
//!
//! Dropped into src/Core/Tensor/TensorMath/ next to tensor_math_standard.zig and selected in
//! src/Core/Tensor/tensor.zig:6 by a build option, it serves the `*_lean` names the generated code calls
//! (tensor_math_standard.zig:43-149) with the signatures of the reference, and forwards them to the C ABI.
//! `Tensor(T).data` of every tensor handed to these functions points at DEVICE memory (zant_hip_malloc, or a
//! slice of the context's arena wrapped with Tensor.fromConstBuffer, tensor.zig:142-150); `shape` stays on the
//! host.  Part one is the `extern fn` block, one declaration per function of the header in the header's
//! order; part two is the wrappers.  Written for Zig 0.13 like the reference.

const std = @import("std");
const zant = @import("../../../zant.zig");
const Tensor = zant.core.tensor.Tensor;
const TensorMathError = zant.utils.error_handler.TensorMathError;
const TensorError = zant.utils.error_handler.TensorError;
pub const AutoPadType = @import("op_pooling.zig").AutoPadType; // NOTSET, SAME_UPPER, SAME_LOWER, VALID = 0..3 on both sides

// ---------------------------------------------------------------------------------------------------------
// Part one: include/zant_hip.h
// ---------------------------------------------------------------------------------------------------------

pub const zant_ctx = opaque {};
pub const zant_model = opaque {};
pub const zant_conv_plan = opaque {};
pub const zant_qconv_plan = opaque {};
pub const LogFn = ?*const fn ([*c]u8) callconv(.C) void;

pub const ZANT_OK: c_int = 0;
pub const ZANT_HipError: c_int = -100;
pub const ZANT_NullPointer: c_int = -101;
pub const ZANT_ArenaOverflow: c_int = -102;
pub const ZANT_NotFinalized: c_int = -103;

pub const ZANT_ACT_NONE: c_int = 0;
pub const ZANT_ACT_RELU: c_int = 1;
pub const ZANT_ACT_LEAKY: c_int = 2;
pub const ZANT_ACT_RELU6: c_int = 3;
pub const ZANT_ACT_SOFTMAX: c_int = 4;

pub const ZANT_LAYOUT_NCHW: c_int = 0;
pub const ZANT_LAYOUT_BLOCKED16: c_int = 1;

pub const ZANT_F32: c_int = 0;
pub const ZANT_U8: c_int = 1;

pub const ZANT_HIP_STATIC_SCRATCH_BYTES: usize = 8 << 20;

// context, memory, timing
pub extern fn zant_hip_ctx_create(out: *?*zant_ctx, device: c_int, stream: ?*anyopaque) c_int;
pub extern fn zant_hip_ctx_destroy(ctx: ?*zant_ctx) void;
pub extern fn zant_hip_sync(ctx: ?*zant_ctx) c_int;
pub extern fn zant_hip_status_name(status: c_int) [*:0]const u8;
pub extern fn zant_hip_last_error(ctx: ?*zant_ctx) [*:0]const u8;
pub extern fn zant_hip_version() [*:0]const u8;
pub extern fn setLogFunctionC(func: LogFn) void;
pub extern fn setLogFunction(func: LogFn) void;
pub extern fn zant_hip_arena_reserve(ctx: ?*zant_ctx, bytes: usize) c_int;
pub extern fn zant_hip_arena_ptr(ctx: ?*zant_ctx, offset: usize) ?*anyopaque;
pub extern fn zant_hip_arena_size(ctx: ?*zant_ctx) usize;
pub extern fn zant_hip_malloc(ctx: ?*zant_ctx, dev_ptr: *?*anyopaque, bytes: usize) c_int;
pub extern fn zant_hip_free(ctx: ?*zant_ctx, dev_ptr: ?*anyopaque) c_int;
pub extern fn zant_hip_upload(ctx: ?*zant_ctx, dst_dev: ?*anyopaque, src_host: ?*const anyopaque, bytes: usize) c_int;
pub extern fn zant_hip_download(ctx: ?*zant_ctx, dst_host: ?*anyopaque, src_dev: ?*const anyopaque, bytes: usize) c_int;
pub extern fn zant_hip_memset(ctx: ?*zant_ctx, dst_dev: ?*anyopaque, byte_value: c_int, bytes: usize) c_int;
pub extern fn zant_hip_timer_start(ctx: ?*zant_ctx) c_int;
pub extern fn zant_hip_timer_stop(ctx: ?*zant_ctx, elapsed_ms: *f32) c_int;
pub extern fn zant_hip_kernel_timing(ctx: ?*zant_ctx, enable: c_int) c_int;
pub extern fn zant_hip_kernel_ms(ctx: ?*zant_ctx, elapsed_ms: *f32) c_int;
pub extern fn zant_hip_kernel_name(ctx: ?*zant_ctx) [*:0]const u8;

// f32 operators
pub extern fn zant_hip_conv2d_f32(ctx: ?*zant_ctx, x: [*]const f32, xdim: *const [4]i64, w: [*]const f32, wdim: *const [4]i64, bias: ?[*]const f32, y: [*]f32, ydim: *const [4]i64, stride: [*]const i64, n_stride: c_int, pads: ?[*]const i64, n_pads: c_int, dil: ?[*]const i64, n_dil: c_int, group: i64, auto_pad: ?[*:0]const u8, fuse_act: c_int) c_int;
pub extern fn zant_hip_conv2d_out_shape(xdim: *const [4]i64, wdim: *const [4]i64, stride: [*]const i64, n_stride: c_int, pads: ?[*]const i64, n_pads: c_int, dil: ?[*]const i64, n_dil: c_int, group: i64, auto_pad: ?[*:0]const u8, ydim: *[4]i64) c_int;
pub extern fn zant_hip_conv2d_f32_static(ctx: ?*zant_ctx, x: [*]const f32, xdim: *const [4]i64, w: [*]const f32, wdim: *const [4]i64, bias: ?[*]const f32, y: [*]f32, ydim: *const [4]i64, stride: [*]const i64, n_stride: c_int, pads: ?[*]const i64, n_pads: c_int, dil: ?[*]const i64, n_dil: c_int, group: i64, auto_pad: ?[*:0]const u8, fuse_act: c_int) c_int;
pub extern fn zant_hip_conv2d_f32_prepack(ctx: ?*zant_ctx, xdim: *const [4]i64, w: [*]const f32, wdim: *const [4]i64, bias: ?[*]const f32, ydim: *const [4]i64, stride: [*]const i64, n_stride: c_int, pads: ?[*]const i64, n_pads: c_int, dil: ?[*]const i64, n_dil: c_int, group: i64, auto_pad: ?[*:0]const u8, fuse_act: c_int, fuse_pool: c_int, out: *?*zant_conv_plan) c_int;
pub extern fn zant_hip_conv2d_f32_packed(ctx: ?*zant_ctx, plan: ?*zant_conv_plan, x: [*]const f32, y: [*]f32) c_int;
pub extern fn zant_hip_conv2d_plan_destroy(ctx: ?*zant_ctx, plan: ?*zant_conv_plan) void;
pub extern fn zant_hip_matmul_f32(ctx: ?*zant_ctx, a: [*]const f32, adim: [*]const i64, a_rank: c_int, b: [*]const f32, bdim: [*]const i64, b_rank: c_int, y: [*]f32) c_int;
pub extern fn zant_hip_matmul_check(adim: [*]const i64, a_rank: c_int, bdim: [*]const i64, b_rank: c_int) c_int;
pub extern fn zant_hip_gemm_f32(ctx: ?*zant_ctx, a: [*]const f32, adim: *const [4]i64, b: [*]const f32, bdim: *const [4]i64, c: ?[*]const f32, cdim: ?[*]const i64, c_rank: c_int, alpha: f32, beta: f32, trans_a: c_int, trans_b: c_int, y: [*]f32, ydim: *const [4]i64, fuse_act: c_int) c_int;
pub extern fn zant_hip_gemm_check(adim: [*]const i64, a_rank: c_int, bdim: [*]const i64, b_rank: c_int, cdim: ?[*]const i64, c_rank: c_int, has_c: c_int, trans_a: c_int, trans_b: c_int, ydim: *[4]i64) c_int;
pub extern fn zant_hip_maxpool2d_f32(ctx: ?*zant_ctx, x: [*]const f32, xdim: *const [4]i64, y: [*]f32, ydim: *const [4]i64, kernel: *const [2]i64, strides: *const [2]i64, dil: *const [2]i64, pads: ?[*]const i64, n_pads: c_int, auto_pad: c_int) c_int;
pub extern fn zant_hip_maxpool2d_out_shape(xdim: *const [4]i64, kernel: *const [2]i64, strides: *const [2]i64, dil: *const [2]i64, pads: *const [4]i64, auto_pad: c_int, ceil_mode: c_int, ydim: *[4]i64) c_int;
pub extern fn zant_hip_avgpool2d_f32(ctx: ?*zant_ctx, x: [*]const f32, xdim: *const [4]i64, y: [*]f32, ydim: *const [4]i64, kernel: *const [2]i64, strides: *const [2]i64, pads: ?*const [4]i64, count_include_pad: c_int) c_int;
pub extern fn zant_hip_avgpool2d_out_shape(xdim: *const [4]i64, kernel: *const [2]i64, strides: *const [2]i64, pads: ?*const [4]i64, ceil_mode: c_int, ydim: *[4]i64) c_int;
pub extern fn zant_hip_batchnorm_f32(ctx: ?*zant_ctx, x: [*]const f32, xdim: [*]const i64, rank: c_int, gamma: [*]const f32, beta: [*]const f32, mean: [*]const f32, variance: [*]const f32, epsilon: f32, y: [*]f32) c_int;
pub extern fn zant_hip_relu_f32(ctx: ?*zant_ctx, x: [*]const f32, y: [*]f32, n: i64) c_int;
pub extern fn zant_hip_leaky_relu_f32(ctx: ?*zant_ctx, x: [*]const f32, slope: f32, y: [*]f32, n: i64) c_int;
pub extern fn zant_hip_sigmoid_f32(ctx: ?*zant_ctx, x: [*]const f32, y: [*]f32, n: i64) c_int;
pub extern fn zant_hip_softmax_f32(ctx: ?*zant_ctx, x: [*]const f32, y: [*]f32, rows: i64, cols: i64) c_int;
pub extern fn zant_hip_add_f32(ctx: ?*zant_ctx, a: [*]const f32, adim: [*]const i64, a_rank: c_int, b: [*]const f32, bdim: [*]const i64, b_rank: c_int, y: [*]f32, ydim_out: ?[*]i64, y_rank_out: ?*c_int) c_int;
pub extern fn zant_hip_add_bias_f32(ctx: ?*zant_ctx, t: [*]f32, tdim: [*]const i64, t_rank: c_int, bias: [*]const f32, bdim: [*]const i64, b_rank: c_int) c_int;
pub extern fn zant_hip_reduce_mean_f32(ctx: ?*zant_ctx, x: ?[*]const f32, xdim: [*]const i64, rank: c_int, axes: ?[*]const i64, n_axes: c_int, keepdims: c_int, noop_with_empty_axes: c_int, y: ?[*]f32, ydim_out: [*]i64, y_rank_out: *c_int) c_int;
pub extern fn zant_hip_concatenate(ctx: ?*zant_ctx, xs: ?[*]const ?*const anyopaque, dims: [*]const [*]const i64, ranks: [*]const c_int, n: c_int, axis: i64, elem_size: usize, y: ?*anyopaque, ydim_out: [*]i64, y_rank_out: *c_int) c_int;
pub extern fn zant_hip_resize_nearest(ctx: ?*zant_ctx, x: ?*const anyopaque, xdim: [*]const i64, rank: c_int, elem_size: usize, scales: ?[*]const f32, sizes: ?[*]const i64, n_param: c_int, coord_mode: c_int, y: ?*anyopaque, ydim_out: [*]i64) c_int;
pub extern fn zant_hip_reshape(ctx: ?*zant_ctx, x: ?*const anyopaque, xdim: [*]const i64, x_rank: c_int, elem_size: usize, new_shape: [*]const i64, new_rank: c_int, y: ?*anyopaque, ydim_out: [*]i64) c_int;

// int8 operators
pub extern fn zant_hip_quantize_linear_f32_u8(ctx: ?*zant_ctx, x: [*]const f32, xdim: [*]const i64, rank: c_int, y_scale: [*]const f32, y_zp: ?[*]const u8, n_scale: i64, axis: c_int, y: [*]u8) c_int;
pub extern fn zant_hip_dequantize_linear_u8_f32(ctx: ?*zant_ctx, x: [*]const u8, xdim: [*]const i64, rank: c_int, x_scale: [*]const f32, x_zp: ?[*]const u8, n_scale: i64, axis: c_int, y: [*]f32) c_int;
pub extern fn zant_hip_quantize_linear_f32_i8(ctx: ?*zant_ctx, x: [*]const f32, xdim: [*]const i64, rank: c_int, y_scale: [*]const f32, y_zp: ?[*]const i8, n_scale: i64, axis: c_int, y: [*]i8) c_int;
pub extern fn zant_hip_dequantize_linear_i8_f32(ctx: ?*zant_ctx, x: [*]const i8, xdim: [*]const i64, rank: c_int, x_scale: [*]const f32, x_zp: ?[*]const i8, n_scale: i64, axis: c_int, y: [*]f32) c_int;
pub extern fn zant_hip_dequantize_linear_i32_f32(ctx: ?*zant_ctx, x: [*]const i32, xdim: [*]const i64, rank: c_int, x_scale: [*]const f32, x_zp: ?[*]const i32, n_scale: i64, axis: c_int, y: [*]f32) c_int;
pub extern fn zant_hip_qlinearconv_u8i8(ctx: ?*zant_ctx, x: [*]const u8, xdim: *const [4]i64, x_scale: f32, x_zp: u8, w: [*]const i8, wdim: *const [4]i64, w_scale: [*]const f32, n_wscale: i64, w_zp: ?[*]const i8, y_scale: f32, y_zp: u8, bias: ?[*]const i32, y: [*]u8, ydim: *const [4]i64, stride: *const [2]i64, pads: *const [4]i64, dil: *const [2]i64, group: i64, act: c_int, act_alpha: f32, act_scale: f32, act_zp: u8) c_int;
pub extern fn zant_hip_blocked16_bytes(dim: *const [4]i64) usize;
pub extern fn zant_hip_to_blocked16_u8(ctx: ?*zant_ctx, x: [*]const u8, dim: *const [4]i64, x_blocked: [*]u8) c_int;
pub extern fn zant_hip_from_blocked16_u8(ctx: ?*zant_ctx, x_blocked: [*]const u8, dim: *const [4]i64, y: [*]u8) c_int;
pub extern fn zant_hip_qlinearconv_prepack(ctx: ?*zant_ctx, xdim: *const [4]i64, x_scale: f32, x_zp: u8, w: [*]const i8, wdim: *const [4]i64, w_scale: [*]const f32, n_wscale: i64, w_zp: ?[*]const i8, y_scale: f32, y_zp: u8, bias: ?[*]const i32, ydim: *const [4]i64, stride: *const [2]i64, pads: *const [4]i64, dil: *const [2]i64, group: i64, act: c_int, act_alpha: f32, act_scale: f32, act_zp: u8, x_layout: c_int, y_layout: c_int, out: *?*zant_qconv_plan) c_int;
pub extern fn zant_hip_qlinearconv_u8i8_packed(ctx: ?*zant_ctx, plan: ?*zant_qconv_plan, x: [*]const u8, y: [*]u8) c_int;
pub extern fn zant_hip_qlinearconv_plan_destroy(ctx: ?*zant_ctx, plan: ?*zant_qconv_plan) void;
pub extern fn zant_hip_qlinear_act_u8(ctx: ?*zant_ctx, x: [*]const u8, n: i64, x_scale: f32, x_zp: u8, act: c_int, alpha: f32, y_scale: f32, y_zp: u8, y: [*]u8) c_int;
pub extern fn zant_hip_qlinear_add_u8(ctx: ?*zant_ctx, a: [*]const u8, a_scale: f32, a_zp: u8, b: [*]const u8, b_scale: f32, b_zp: u8, y_scale: f32, y_zp: u8, y: [*]u8, n: i64) c_int;
pub extern fn zant_hip_maxpool2d_u8(ctx: ?*zant_ctx, x: [*]const u8, xdim: *const [4]i64, y: [*]u8, ydim: *const [4]i64, kernel: *const [2]i64, strides: *const [2]i64, dil: *const [2]i64, pads: ?[*]const i64, n_pads: c_int, auto_pad: c_int) c_int;
pub extern fn zant_hip_qlinear_global_avgpool_u8(ctx: ?*zant_ctx, x: [*]const u8, xdim: *const [4]i64, x_scale: f32, x_zp: u8, y_scale: f32, y_zp: u8, y: [*]u8) c_int;

// generated-library level
pub extern fn zant_model_create(ctx: ?*zant_ctx, out: *?*zant_model) c_int;
pub extern fn zant_model_destroy(m: ?*zant_model) void;
pub extern fn zant_model_input(m: ?*zant_model, dtype: c_int, dims: [*]const i64, rank: c_int, scale: f32, zp: c_int) c_int;
pub extern fn zant_model_conv(m: ?*zant_model, x: c_int, w: [*]const f32, wdim: *const [4]i64, bias: ?[*]const f32, stride: [*]const i64, n_stride: c_int, pads: ?[*]const i64, n_pads: c_int, dil: ?[*]const i64, n_dil: c_int, group: i64, auto_pad: ?[*:0]const u8) c_int;
pub extern fn zant_model_relu(m: ?*zant_model, x: c_int) c_int;
pub extern fn zant_model_leaky_relu(m: ?*zant_model, x: c_int, slope: f32) c_int;
pub extern fn zant_model_maxpool(m: ?*zant_model, x: c_int, kernel: *const [2]i64, strides: *const [2]i64, dil: *const [2]i64, pads: *const [4]i64, auto_pad: c_int, ceil_mode: c_int) c_int;
pub extern fn zant_model_avgpool(m: ?*zant_model, x: c_int, kernel: *const [2]i64, strides: *const [2]i64, pads: ?*const [4]i64, ceil_mode: c_int, count_include_pad: c_int) c_int;
pub extern fn zant_model_batchnorm(m: ?*zant_model, x: c_int, gamma: [*]const f32, beta: [*]const f32, mean: [*]const f32, variance: [*]const f32, features: i64, epsilon: f32) c_int;
pub extern fn zant_model_reshape(m: ?*zant_model, x: c_int, new_shape: [*]const i64, rank: c_int) c_int;
pub extern fn zant_model_gemm(m: ?*zant_model, a: c_int, b: [*]const f32, bdim: *const [4]i64, c: ?[*]const f32, cdim: ?[*]const i64, c_rank: c_int, alpha: f32, beta: f32, trans_a: c_int, trans_b: c_int) c_int;
pub extern fn zant_model_matmul(m: ?*zant_model, a: c_int, b: [*]const f32, bdim: [*]const i64, b_rank: c_int) c_int;
pub extern fn zant_model_add_const(m: ?*zant_model, x: c_int, c: [*]const f32, cdim: [*]const i64, c_rank: c_int) c_int;
pub extern fn zant_model_add(m: ?*zant_model, a: c_int, b: c_int) c_int;
pub extern fn zant_model_softmax(m: ?*zant_model, x: c_int) c_int;
pub extern fn zant_model_sigmoid(m: ?*zant_model, x: c_int) c_int;
pub extern fn zant_model_reduce_mean(m: ?*zant_model, x: c_int, axes: ?[*]const i64, n_axes: c_int, keepdims: c_int) c_int;
pub extern fn zant_model_concat(m: ?*zant_model, xs: [*]const c_int, n: c_int, axis: i64) c_int;
pub extern fn zant_model_resize_nearest(m: ?*zant_model, x: c_int, scales: ?[*]const f32, sizes: ?[*]const i64, n_param: c_int, coord_mode: c_int) c_int;
pub extern fn zant_model_quantize(m: ?*zant_model, x: c_int, y_scale: f32, y_zp: c_int) c_int;
pub extern fn zant_model_dequantize(m: ?*zant_model, x: c_int) c_int;
pub extern fn zant_model_qlinearconv(m: ?*zant_model, x: c_int, w: [*]const i8, wdim: *const [4]i64, w_scale: [*]const f32, n_wscale: i64, bias: ?[*]const i32, y_scale: f32, y_zp: c_int, stride: *const [2]i64, pads: *const [4]i64, dil: *const [2]i64, group: i64) c_int;
pub extern fn zant_model_qlinear_act(m: ?*zant_model, x: c_int, act: c_int, alpha: f32, y_scale: f32, y_zp: c_int) c_int;
pub extern fn zant_model_qlinear_add(m: ?*zant_model, a: c_int, b: c_int, y_scale: f32, y_zp: c_int) c_int;
pub extern fn zant_model_qlinear_global_avgpool(m: ?*zant_model, x: c_int, y_scale: f32, y_zp: c_int) c_int;
pub extern fn zant_model_finalize(m: ?*zant_model) c_int;
pub extern fn zant_model_output_dims(m: ?*zant_model, dims: [*]i64, rank: *c_int, dtype: *c_int) c_int;
pub extern fn zant_model_tensor_dims(m: ?*zant_model, tensor: c_int, dims: [*]i64, rank: *c_int, dtype: *c_int) c_int;
pub extern fn zant_model_arena_bytes(m: ?*zant_model) usize;
pub extern fn zant_model_unfused_bytes(m: ?*zant_model) usize;
pub extern fn zant_model_num_launches(m: ?*zant_model) c_int;
pub extern fn zant_model_run(m: ?*zant_model, input_dev: ?*const anyopaque, output_dev: ?*anyopaque) c_int;
pub extern fn zant_model_input_ptr(m: ?*zant_model) ?*anyopaque;
pub extern fn zant_model_output_ptr(m: ?*zant_model) ?*anyopaque;
pub extern fn zant_model_predict_host(m: ?*zant_model, input_host: ?*const anyopaque, output_host: ?*anyopaque) c_int;
pub extern fn zant_model_profile(m: ?*zant_model, ms: [*]f32, ops: [*]f64, bytes: [*]f64, capacity: c_int) c_int;
pub extern fn zant_model_launch_name(m: ?*zant_model, i: c_int) [*:0]const u8;
pub extern fn zant_model_launch_kernel(m: ?*zant_model, i: c_int) [*:0]const u8;
pub extern fn zant_model_read_tensor(m: ?*zant_model, id: c_int, dst_host: ?*anyopaque, bytes: usize) c_int;
pub extern fn zant_model_bind_predict(m: ?*zant_model) c_int;
pub extern fn predict(input: [*]f32, input_shape: [*]u32, shape_len: u32, result: *[*]f32) void;
pub extern fn predict_batched(input: [*]f32, n: u32, result: *[*]f32) void;

// ---------------------------------------------------------------------------------------------------------
// Part two: the lean façade
// ---------------------------------------------------------------------------------------------------------

/// One context (= one HIP stream) per generated library instance; `init` before the first operator call.
pub var ctx: ?*zant_ctx = null;

pub fn init(device: c_int) !void {
    if (ctx != null) return;
    try toErr(zant_hip_ctx_create(&ctx, device, null));
}

pub fn deinit() void {
    zant_hip_ctx_destroy(ctx);
    ctx = null;
}

/// Status code -> the Zig error the reference's operator returns (src/Utils/errorHandler.zig:36-84).
pub fn toErr(rc: c_int) !void {
    return switch (rc) {
        0 => {},
        -1 => TensorMathError.InvalidDimensions,
        -2 => TensorMathError.InvalidPadding,
        -3 => TensorMathError.InputTensorsWrongShape,
        -4 => TensorMathError.InputTensorDifferentShape,
        -5 => TensorMathError.InputTensorDimensionMismatch,
        -6 => TensorMathError.IncompatibleBroadcastShapes,
        -7 => TensorMathError.InputTensorDifferentSize,
        -8 => TensorError.EmptyTensor,
        -9 => TensorError.ZeroSizeTensor,
        -10 => TensorError.InvalidInput,
        -11 => TensorError.InputArrayWrongSize,
        -12 => TensorMathError.WrongStride,
        -14 => TensorMathError.InvalidAxes,
        -15 => TensorError.AxisOutOfBounds,
        -16 => TensorError.MismatchedShape,
        -17 => TensorError.MismatchedRank,
        -18 => TensorMathError.EmptyTensorList,
        -19 => TensorError.UnsupportedMode,
        else => TensorMathError.MemError, // -13 MemError, -100.. HIP failures (text: zant_hip_last_error)
    };
}

const MAX_RANK = 8;

fn dims4(shape: []const usize) ![4]i64 {
    if (shape.len != 4) return TensorMathError.InvalidDimensions;
    return .{ @intCast(shape[0]), @intCast(shape[1]), @intCast(shape[2]), @intCast(shape[3]) };
}

fn dimsN(shape: []const usize) ![MAX_RANK]i64 {
    if (shape.len > MAX_RANK) return TensorMathError.InvalidDimensions;
    var out = [_]i64{1} ** MAX_RANK;
    for (shape, 0..) |d, i| out[i] = @intCast(d);
    return out;
}

fn toI64(comptime n: usize, s: []const usize) [n]i64 {
    var out = [_]i64{0} ** n;
    for (0..@min(n, s.len)) |i| out[i] = @intCast(s[i]);
    return out;
}

fn onlyF32(comptime T: type) void {
    if (T != f32) @compileError("this lean operator of the HIP backend is f32 only; the quantised family is qlinearconv_lean / quantize_linear_lean / dequantize_linear_lean / onnx_maxpool_lean(u8)");
}

/// conv_lean = OnnxConvLean (op_convolution.zig:42).
pub fn conv_lean(comptime T: type, input: *Tensor(T), kernel: *Tensor(T), output: *Tensor(T), bias: ?*const Tensor(T), stride: []const usize, pads: ?[]const usize, dilations: ?[]const usize, group: ?usize, auto_pad: ?[]const u8) !void {
    comptime onlyF32(T);
    if (input.shape.len != 4 or kernel.shape.len != 4) return TensorMathError.InvalidDimensions;
    const xd = try dims4(input.shape);
    const wd = try dims4(kernel.shape);
    const yd = try dims4(output.shape);
    const s = toI64(2, stride);
    var p = [_]i64{0} ** 4;
    var d = [_]i64{1} ** 2;
    if (pads) |pp| p = toI64(4, pp);
    if (dilations) |dd| d = toI64(2, dd);
    var ap_buf: [16:0]u8 = undefined; // the C side takes a 0-terminated copy of the Zig slice
    const ap: ?[*:0]const u8 = if (auto_pad) |a| blk: {
        if (a.len > 15) return TensorMathError.InvalidPadding;
        @memcpy(ap_buf[0..a.len], a);
        ap_buf[a.len] = 0;
        break :blk &ap_buf;
    } else null;
    try toErr(zant_hip_conv2d_f32(ctx, input.data.ptr, &xd, kernel.data.ptr, &wd, if (bias) |b| b.data.ptr else null, output.data.ptr, &yd, &s, @intCast(stride.len), if (pads != null) &p else null, if (pads) |pp| @intCast(pp.len) else 0, if (dilations != null) &d else null, if (dilations) |dd| @intCast(dd.len) else 0, if (group) |g| @intCast(g) else -1, ap, ZANT_ACT_NONE));
}

/// gemm_lean = lean_gemm (op_gemm.zig:91).
pub fn gemm_lean(comptime T: anytype, A: *Tensor(T), B: *Tensor(T), C: ?*Tensor(T), alpha: T, beta: T, transA: bool, transB: bool, result: *Tensor(T)) !void {
    comptime onlyF32(T);
    const ad = try dims4(A.shape);
    const bd = try dims4(B.shape);
    const yd = try dims4(result.shape);
    var cd = [_]i64{1} ** MAX_RANK;
    if (C) |c| cd = try dimsN(c.shape);
    try toErr(zant_hip_gemm_f32(ctx, A.data.ptr, &ad, B.data.ptr, &bd, if (C) |c| c.data.ptr else null, if (C != null) &cd else null, if (C) |c| @intCast(c.shape.len) else 0, alpha, beta, @intFromBool(transA), @intFromBool(transB), result.data.ptr, &yd, ZANT_ACT_NONE));
}

/// mat_mul_lean = lean_mat_mul (op_mat_mul.zig:92): the last two dimensions only, as there.
pub fn mat_mul_lean(comptime T: anytype, A: *const Tensor(T), B: *const Tensor(T), Y: *Tensor(T)) !void {
    comptime onlyF32(T);
    const ad = try dimsN(A.shape);
    const bd = try dimsN(B.shape);
    try toErr(zant_hip_matmul_f32(ctx, A.data.ptr, &ad, @intCast(A.shape.len), B.data.ptr, &bd, @intCast(B.shape.len), Y.data.ptr));
}
pub const lean_matmul = mat_mul_lean; // both names exist in tensor_math_standard.zig (:47, :109)

/// onnx_maxpool_lean = lean_onnx_maxpool (op_pooling.zig:570-579).
pub fn onnx_maxpool_lean(comptime T: type, input: *Tensor(T), output: *Tensor(T), kernel_shape: []const usize, strides: []const usize, dilations: []const usize, pads: []const usize, auto_pad: AutoPadType) !void {
    if (T != f32 and T != u8) @compileError("onnx_maxpool_lean of the HIP backend takes f32 or u8 (quantised values: max-pooling commutes with the monotone quantisation)");
    const xd = try dims4(input.shape);
    const yd = try dims4(output.shape);
    const k = toI64(2, kernel_shape);
    const s = toI64(2, strides);
    const d = toI64(2, dilations);
    const p = toI64(4, pads);
    if (T == u8) {
        try toErr(zant_hip_maxpool2d_u8(ctx, input.data.ptr, &xd, output.data.ptr, &yd, &k, &s, &d, &p, @intCast(pads.len), @intFromEnum(auto_pad)));
    } else {
        try toErr(zant_hip_maxpool2d_f32(ctx, input.data.ptr, &xd, output.data.ptr, &yd, &k, &s, &d, &p, @intCast(pads.len), @intFromEnum(auto_pad)));
    }
}

/// get_onnx_maxpool_output_shape (op_pooling.zig:477-485); the caller frees the result, as there.
pub fn get_onnx_maxpool_output_shape(input_shape: []const usize, kernel_shape: []const usize, strides: []const usize, dilations: []const usize, pads: []const usize, auto_pad: AutoPadType, ceil_mode: bool) ![]usize {
    const xd = try dims4(input_shape);
    const k = toI64(2, kernel_shape);
    const s = toI64(2, strides);
    const d = toI64(2, dilations);
    const p = toI64(4, pads);
    var yd: [4]i64 = undefined;
    try toErr(zant_hip_maxpool2d_out_shape(&xd, &k, &s, &d, &p, @intFromEnum(auto_pad), @intFromBool(ceil_mode), &yd));
    const out = try zant.utils.allocator.allocator.alloc(usize, 4);
    for (yd, 0..) |v, i| out[i] = @intCast(v);
    return out;
}

/// get_convolution_output_shape (op_convolution.zig:333).
pub fn get_convolution_output_shape(input_shape: []const usize, kernel_shape: []const usize, stride: []const usize, pads: ?[]const usize, dilations: ?[]const usize, auto_pad: ?[]const u8) ![4]usize {
    const xd = try dims4(input_shape);
    const wd = try dims4(kernel_shape);
    const s = toI64(2, stride);
    var p = [_]i64{0} ** 4;
    var d = [_]i64{1} ** 2;
    if (pads) |pp| p = toI64(4, pp);
    if (dilations) |dd| d = toI64(2, dd);
    var ap_buf: [16:0]u8 = undefined;
    const ap: ?[*:0]const u8 = if (auto_pad) |a| blk: {
        if (a.len > 15) return TensorMathError.InvalidPadding;
        @memcpy(ap_buf[0..a.len], a);
        ap_buf[a.len] = 0;
        break :blk &ap_buf;
    } else null;
    var yd: [4]i64 = undefined;
    try toErr(zant_hip_conv2d_out_shape(&xd, &wd, &s, @intCast(stride.len), if (pads != null) &p else null, if (pads) |pp| @intCast(pp.len) else 0, if (dilations != null) &d else null, if (dilations) |dd| @intCast(dd.len) else 0, -1, ap, &yd));
    return .{ @intCast(yd[0]), @intCast(yd[1]), @intCast(yd[2]), @intCast(yd[3]) };
}

/// ReLU_lean = lean_ReLU (lib_activation_function_math.zig:22).
pub fn ReLU_lean(comptime T: anytype, input_tensor: *Tensor(T), output_tensor: *Tensor(T)) !void {
    comptime onlyF32(T);
    try toErr(zant_hip_relu_f32(ctx, input_tensor.data.ptr, output_tensor.data.ptr, @intCast(input_tensor.size)));
}

/// leakyReLU_lean = lean_leakyReLU (lib_activation_function_math.zig:68).
pub fn leakyReLU_lean(comptime T: anytype, input_tensor: *Tensor(T), slope: T, output_tensor: *Tensor(T)) !void {
    comptime onlyF32(T);
    try toErr(zant_hip_leaky_relu_f32(ctx, input_tensor.data.ptr, slope, output_tensor.data.ptr, @intCast(input_tensor.size)));
}

/// sigmoid_lean (lib_activation_function_math.zig:107).
pub fn sigmoid_lean(comptime T: anytype, input_tensor: *Tensor(T), output_tensor: *Tensor(T)) !void {
    comptime onlyF32(T);
    try toErr(zant_hip_sigmoid_f32(ctx, input_tensor.data.ptr, output_tensor.data.ptr, @intCast(input_tensor.size)));
}

/// softmax_lean = lean_softmax (lib_activation_function_math.zig:154): rows = shape[0], cols = shape[1].
pub fn softmax_lean(comptime T: anytype, input: *Tensor(T), output: *Tensor(T)) !void {
    comptime onlyF32(T);
    if (input.shape.len < 2) return TensorMathError.InvalidDimensions;
    try toErr(zant_hip_softmax_f32(ctx, input.data.ptr, output.data.ptr, @intCast(input.shape[0]), @intCast(input.shape[1])));
}

/// sum_tensors_lean = lean_sum_tensors (lib_elementWise_math.zig:70).
pub fn sum_tensors_lean(comptime inputType: anytype, comptime outputType: anytype, t1: *Tensor(inputType), t2: *Tensor(inputType), outputTensor: *Tensor(outputType)) !void {
    comptime onlyF32(inputType);
    comptime onlyF32(outputType);
    const ad = try dimsN(t1.shape);
    const bd = try dimsN(t2.shape);
    try toErr(zant_hip_add_f32(ctx, t1.data.ptr, &ad, @intCast(t1.shape.len), t2.data.ptr, &bd, @intCast(t2.shape.len), outputTensor.data.ptr, null, null));
}

/// add_bias (lib_elementWise_math.zig:22), in place.
pub fn add_bias(comptime T: anytype, tensor: *Tensor(T), bias: *Tensor(T)) !void {
    comptime onlyF32(T);
    const td = try dimsN(tensor.shape);
    const bd = try dimsN(bias.shape);
    try toErr(zant_hip_add_bias_f32(ctx, tensor.data.ptr, &td, @intCast(tensor.shape.len), bias.data.ptr, &bd, @intCast(bias.shape.len)));
}

/// reshape_lean (lib_shape_math.zig:1139): the output tensor's `shape` slice receives the resolved shape.
pub fn reshape_lean(comptime T: anytype, input: *Tensor(T), newShape: []const usize, allowZero: ?bool, output: *Tensor(T)) !void {
    _ = allowZero;
    if (newShape.len > MAX_RANK) return TensorMathError.InvalidDimensions;
    const xd = try dimsN(input.shape);
    var nd = [_]i64{1} ** MAX_RANK;
    for (newShape, 0..) |d, i| nd[i] = @intCast(d);
    var yd: [MAX_RANK]i64 = undefined;
    try toErr(zant_hip_reshape(ctx, input.data.ptr, &xd, @intCast(input.shape.len), @sizeOf(T), &nd, @intCast(newShape.len), output.data.ptr, &yd));
    if (output.shape.len == newShape.len) {
        for (0..newShape.len) |i| output.shape[i] = @intCast(yd[i]);
    }
}

/// reduce_mean_lean = lean_reduce_mean (lib_reduction_math.zig:87-94).  keepdims is unused there too: the
/// output is pre-shaped; it is derived here from the output's rank so the checks see the same request.
pub fn reduce_mean_lean(comptime T: anytype, input_tensor: *Tensor(T), output_tensor: *Tensor(T), axes: ?[]const i64, _: bool, noop_with_empty_axes: bool) !void {
    comptime onlyF32(T);
    const xd = try dimsN(input_tensor.shape);
    var yd: [MAX_RANK]i64 = undefined;
    var yr: c_int = 0;
    const keep = output_tensor.shape.len == input_tensor.shape.len;
    try toErr(zant_hip_reduce_mean_f32(ctx, input_tensor.data.ptr, &xd, @intCast(input_tensor.shape.len), if (axes) |a| a.ptr else null, if (axes) |a| @intCast(a.len) else 0, @intFromBool(keep), @intFromBool(noop_with_empty_axes), output_tensor.data.ptr, &yd, &yr));
}

/// get_reduce_mean_output_shape: the shape pass of reduce_mean (lib_reduction_math.zig:30-85), host only.
pub fn get_reduce_mean_output_shape(input_shape: []const usize, axes: ?[]const i64, keepdims: bool, noop_with_empty_axes: bool) ![]usize {
    const xd = try dimsN(input_shape);
    var yd: [MAX_RANK]i64 = undefined;
    var yr: c_int = 0;
    try toErr(zant_hip_reduce_mean_f32(null, null, &xd, @intCast(input_shape.len), if (axes) |a| a.ptr else null, if (axes) |a| @intCast(a.len) else 0, @intFromBool(keepdims), @intFromBool(noop_with_empty_axes), null, &yd, &yr));
    const out = try zant.utils.allocator.allocator.alloc(usize, @intCast(yr));
    for (out, 0..) |*v, i| v.* = @intCast(yd[i]);
    return out;
}

/// lean_concatenate (lib_shape_math.zig:307): up to 16 inputs.
pub fn lean_concatenate(comptime T: type, allocator: *const std.mem.Allocator, tensors: []const Tensor(T), axis: isize, output: *Tensor(T)) !void {
    _ = allocator; // the reference needs it for index scratch; nothing is allocated here
    if (tensors.len == 0) return TensorMathError.EmptyTensorList;
    if (tensors.len > 16) return TensorError.InvalidInput;
    var ptrs: [16]?*const anyopaque = undefined;
    var dims: [16][MAX_RANK]i64 = undefined;
    var dim_ptrs: [16][*]const i64 = undefined;
    var ranks: [16]c_int = undefined;
    for (tensors, 0..) |t, i| {
        ptrs[i] = t.data.ptr;
        dims[i] = try dimsN(t.shape);
        dim_ptrs[i] = &dims[i];
        ranks[i] = @intCast(t.shape.len);
    }
    var yd: [MAX_RANK]i64 = undefined;
    var yr: c_int = 0;
    try toErr(zant_hip_concatenate(ctx, &ptrs, &dim_ptrs, &ranks, @intCast(tensors.len), @intCast(axis), @sizeOf(T), output.data.ptr, &yd, &yr));
}

/// get_concatenate_output_shape (lib_shape_math.zig:582).
pub fn get_concatenate_output_shape(tensors: []const []const usize, axis: isize) ![]usize {
    if (tensors.len == 0) return TensorMathError.EmptyTensorList;
    if (tensors.len > 16) return TensorError.InvalidInput;
    var dims: [16][MAX_RANK]i64 = undefined;
    var dim_ptrs: [16][*]const i64 = undefined;
    var ranks: [16]c_int = undefined;
    for (tensors, 0..) |s, i| {
        dims[i] = try dimsN(s);
        dim_ptrs[i] = &dims[i];
        ranks[i] = @intCast(s.len);
    }
    var yd: [MAX_RANK]i64 = undefined;
    var yr: c_int = 0;
    try toErr(zant_hip_concatenate(null, null, &dim_ptrs, &ranks, @intCast(tensors.len), @intCast(axis), 4, null, &yd, &yr));
    const out = try zant.utils.allocator.allocator.alloc(usize, @intCast(yr));
    for (out, 0..) |*v, i| v.* = @intCast(yd[i]);
    return out;
}

fn coordMode(s: []const u8) c_int {
    if (std.mem.eql(u8, s, "half_pixel")) return 0;
    if (std.mem.eql(u8, s, "align_corners")) return 1;
    return 2; // the reference's comparison chain falls through to asymmetric (lib_shape_math.zig:120-135)
}

/// resize_lean: the "nearest" mode of resize (lib_shape_math.zig:22) into a pre-shaped device tensor.  The
/// reference's resize allocates its result; its generated code sizes the output from get_resize_output_shape
/// first, which is what this pair serves.  "linear" and "cubic": TensorError.UnsupportedMode.
pub fn resize_lean(comptime T: type, t: *Tensor(T), comptime mode: []const u8, scales: ?[]const f32, sizes: ?[]const usize, coordinate_transformation_mode: []const u8, output: *Tensor(T)) !void {
    if (comptime !std.mem.eql(u8, mode, "nearest")) return TensorError.UnsupportedMode;
    if (scales == null and sizes == null) return TensorError.InvalidInput;
    const xd = try dimsN(t.shape);
    var sz = [_]i64{0} ** MAX_RANK;
    if (sizes) |s| {
        if (s.len > MAX_RANK) return TensorError.InvalidInput;
        for (s, 0..) |v, i| sz[i] = @intCast(v);
    }
    var yd: [MAX_RANK]i64 = undefined;
    try toErr(zant_hip_resize_nearest(ctx, t.data.ptr, &xd, @intCast(t.shape.len), @sizeOf(T), if (scales) |s| s.ptr else null, if (sizes != null) &sz else null, @intCast(if (scales) |s| s.len else sizes.?.len), coordMode(coordinate_transformation_mode), output.data.ptr, &yd));
}

/// get_resize_output_shape (lib_shape_math.zig:78).
pub fn get_resize_output_shape(input_shape: []const usize, scales: ?[]const f32, sizes: ?[]const usize) ![]usize {
    if (scales == null and sizes == null) return TensorError.InvalidInput;
    const xd = try dimsN(input_shape);
    var sz = [_]i64{0} ** MAX_RANK;
    if (sizes) |s| {
        if (s.len > MAX_RANK) return TensorError.InvalidInput;
        for (s, 0..) |v, i| sz[i] = @intCast(v);
    }
    var yd: [MAX_RANK]i64 = undefined;
    try toErr(zant_hip_resize_nearest(null, null, &xd, @intCast(input_shape.len), 4, if (scales) |s| s.ptr else null, if (sizes != null) &sz else null, @intCast(if (scales) |s| s.len else sizes.?.len), 2, null, &yd));
    const out = try zant.utils.allocator.allocator.alloc(usize, input_shape.len);
    for (out, 0..) |*v, i| v.* = @intCast(yd[i]);
    return out;
}

/// Average pooling into a pre-shaped tensor: pool_forward with PoolingType.Avg (op_pooling.zig:223, 373-408),
/// extended with ONNX AveragePool's pads / count_include_pad.  The reference has no lean form of it.
pub fn avgpool_lean(comptime T: type, input: *Tensor(T), output: *Tensor(T), kernel: [2]usize, stride: [2]usize, pads: ?[4]usize, count_include_pad: bool) !void {
    comptime onlyF32(T);
    const xd = try dims4(input.shape);
    const yd = try dims4(output.shape);
    const k = toI64(2, &kernel);
    const s = toI64(2, &stride);
    var p = [_]i64{0} ** 4;
    if (pads) |pp| p = toI64(4, &pp);
    try toErr(zant_hip_avgpool2d_f32(ctx, input.data.ptr, &xd, output.data.ptr, &yd, &k, &s, if (pads != null) &p else null, @intFromBool(count_include_pad)));
}

/// get_pooling_output_shape (op_pooling.zig:16): (H - k) / s + 1, no padding, floor.
pub fn get_pooling_output_shape(input_shape: []const usize, kernel: [2]usize, stride: [2]usize) ![4]usize {
    const xd = try dims4(input_shape);
    const k = toI64(2, &kernel);
    const s = toI64(2, &stride);
    var yd: [4]i64 = undefined;
    try toErr(zant_hip_avgpool2d_out_shape(&xd, &k, &s, null, 0, &yd));
    return .{ @intCast(yd[0]), @intCast(yd[1]), @intCast(yd[2]), @intCast(yd[3]) };
}

/// BatchNormLayer.forward with is_training false (src/Model/Layers/batchNormLayer.zig:130-148) into a
/// pre-shaped tensor; gamma / beta / running_mean / running_var are device tensors of shape[1] values.
pub fn batchnorm_lean(comptime T: type, input: *Tensor(T), gamma: *Tensor(T), beta: *Tensor(T), running_mean: *Tensor(T), running_var: *Tensor(T), epsilon: T, output: *Tensor(T)) !void {
    comptime onlyF32(T);
    const xd = try dimsN(input.shape);
    try toErr(zant_hip_batchnorm_f32(ctx, input.data.ptr, &xd, @intCast(input.shape.len), gamma.data.ptr, beta.data.ptr, running_mean.data.ptr, running_var.data.ptr, epsilon, output.data.ptr));
}

// ---- the quantised family (ONNX QuantizeLinear / DequantizeLinear / QLinearConv) ---------------------------
// The reference has no such operators (src/Core/Quantization/quantization.zig is empty); these follow its house
// style -- comptime element types, pre-shaped output, `!void` -- and the ONNX input order.  Scales and zero points
// are tensors, as ONNX passes them: per tensor (one element) or per `axis`.

/// quantize_linear_lean: y = saturate(round_half_even(x / y_scale) + y_zero_point).  T_out: u8 or i8.
/// y_scale / y_zero_point hold one element, or input.shape[axis] elements (per-axis); they are DEVICE tensors.
pub fn quantize_linear_lean(comptime T_in: type, comptime T_out: type, x: *Tensor(T_in), y_scale: *Tensor(T_in), y_zero_point: ?*Tensor(T_out), axis: i64, y: *Tensor(T_out)) !void {
    comptime onlyF32(T_in);
    if (T_out != u8 and T_out != i8) @compileError("quantize_linear_lean: T_out is u8 or i8");
    const xd = try dimsN(x.shape);
    const rank: i64 = @intCast(x.shape.len);
    const ax: c_int = @intCast(if (axis < 0) axis + rank else axis);
    if (T_out == u8) {
        try toErr(zant_hip_quantize_linear_f32_u8(ctx, x.data.ptr, &xd, @intCast(x.shape.len), y_scale.data.ptr, if (y_zero_point) |z| z.data.ptr else null, @intCast(y_scale.size), ax, y.data.ptr));
    } else {
        try toErr(zant_hip_quantize_linear_f32_i8(ctx, x.data.ptr, &xd, @intCast(x.shape.len), y_scale.data.ptr, if (y_zero_point) |z| z.data.ptr else null, @intCast(y_scale.size), ax, y.data.ptr));
    }
}

/// dequantize_linear_lean: y = (x - x_zero_point) * x_scale.  T_in: u8, i8 or i32 (accumulators, biases).
pub fn dequantize_linear_lean(comptime T_in: type, comptime T_out: type, x: *Tensor(T_in), x_scale: *Tensor(T_out), x_zero_point: ?*Tensor(T_in), axis: i64, y: *Tensor(T_out)) !void {
    comptime onlyF32(T_out);
    if (T_in != u8 and T_in != i8 and T_in != i32) @compileError("dequantize_linear_lean: T_in is u8, i8 or i32");
    const xd = try dimsN(x.shape);
    const rank: i64 = @intCast(x.shape.len);
    const ax: c_int = @intCast(if (axis < 0) axis + rank else axis);
    const zp = if (x_zero_point) |z| z.data.ptr else null;
    const n: i64 = @intCast(x_scale.size);
    const r: c_int = @intCast(x.shape.len);
    switch (T_in) {
        u8 => try toErr(zant_hip_dequantize_linear_u8_f32(ctx, x.data.ptr, &xd, r, x_scale.data.ptr, zp, n, ax, y.data.ptr)),
        i8 => try toErr(zant_hip_dequantize_linear_i8_f32(ctx, x.data.ptr, &xd, r, x_scale.data.ptr, zp, n, ax, y.data.ptr)),
        else => try toErr(zant_hip_dequantize_linear_i32_f32(ctx, x.data.ptr, &xd, r, x_scale.data.ptr, zp, n, ax, y.data.ptr)),
    }
}

/// qlinearconv_lean: ONNX QLinearConv in the input order of the operator (x, x_scale, x_zero_point, w, w_scale,
/// w_zero_point, y_scale, y_zero_point, B) followed by conv_lean's attributes (op_convolution.zig:42).  x_scale,
/// x_zero_point, y_scale and y_zero_point are per-tensor HOST scalars (ONNX requires them to be scalars); w_scale
/// (one element or one per output channel), w_zero_point (null: 0) and bias are DEVICE tensors.  pads are
/// [top, left, bottom, right]; null pads / dilations mean 0 / 1; group null means 1 (group == channels: depthwise).
pub fn qlinearconv_lean(x: *Tensor(u8), x_scale: f32, x_zero_point: u8, w: *Tensor(i8), w_scale: *Tensor(f32), w_zero_point: ?*Tensor(i8), y_scale: f32, y_zero_point: u8, bias: ?*const Tensor(i32), y: *Tensor(u8), stride: []const usize, pads: ?[]const usize, dilations: ?[]const usize, group: ?usize) !void {
    const xd = try dims4(x.shape);
    const wd = try dims4(w.shape);
    const yd = try dims4(y.shape);
    if (stride.len < 1) return TensorMathError.WrongStride;
    var s = toI64(2, stride);
    if (stride.len == 1) s[1] = s[0]; // as conv_lean: stride[1] falls back to stride[0] (op_convolution.zig:68-69)
    var p = [_]i64{0} ** 4;
    var d = [_]i64{1} ** 2;
    if (pads) |pp| {
        if (pp.len < 4) return TensorMathError.InvalidPadding;
        p = toI64(4, pp);
    }
    if (dilations) |dd| {
        d = toI64(2, dd);
        if (dd.len == 1) d[1] = d[0];
    }
    try toErr(zant_hip_qlinearconv_u8i8(ctx, x.data.ptr, &xd, x_scale, x_zero_point, w.data.ptr, &wd, w_scale.data.ptr, @intCast(w_scale.size), if (w_zero_point) |z| z.data.ptr else null, y_scale, y_zero_point, if (bias) |b| b.data.ptr else null, y.data.ptr, &yd, &s, &p, &d, if (group) |g| @intCast(g) else 1, ZANT_ACT_NONE, 0.0, 1.0, 0));
}

/// Prepared weights for qlinearconv_lean: the weight-dependent tables are derived once, at the first `run`.
pub const QLinearConvPlan = struct {
    handle: ?*zant_qconv_plan = null,

    pub fn init(xshape: []const usize, x_scale: f32, x_zero_point: u8, w: *Tensor(i8), w_scale: *Tensor(f32), w_zero_point: ?*Tensor(i8), y_scale: f32, y_zero_point: u8, bias: ?*const Tensor(i32), yshape: []const usize, stride: [2]usize, pads: [4]usize, dilations: [2]usize, group: usize, x_layout: c_int, y_layout: c_int) !QLinearConvPlan {
        const xd = try dims4(xshape);
        const wd = try dims4(w.shape);
        const yd = try dims4(yshape);
        const s = toI64(2, &stride);
        const p = toI64(4, &pads);
        const d = toI64(2, &dilations);
        var self = QLinearConvPlan{};
        try toErr(zant_hip_qlinearconv_prepack(ctx, &xd, x_scale, x_zero_point, w.data.ptr, &wd, w_scale.data.ptr, @intCast(w_scale.size), if (w_zero_point) |z| z.data.ptr else null, y_scale, y_zero_point, if (bias) |b| b.data.ptr else null, &yd, &s, &p, &d, @intCast(group), ZANT_ACT_NONE, 0.0, 1.0, 0, x_layout, y_layout, &self.handle));
        return self;
    }

    pub fn run(self: *QLinearConvPlan, x: [*]const u8, y: [*]u8) !void {
        try toErr(zant_hip_qlinearconv_u8i8_packed(ctx, self.handle, x, y));
    }

    pub fn deinit(self: *QLinearConvPlan) void {
        zant_hip_qlinearconv_plan_destroy(ctx, self.handle);
        self.handle = null;
    }
};

/// Prepared weights for conv_lean (same attributes); `run` is conv_lean without the per-call weight packing.
/// fuse_pool: Conv (-> ReLU) -> onnx_maxpool_lean 2x2 / stride 2 in one kernel; yshape is then the pooled shape.
pub const ConvPlan = struct {
    handle: ?*zant_conv_plan = null,

    pub fn init(xshape: []const usize, kernel: *Tensor(f32), bias: ?*const Tensor(f32), yshape: []const usize, stride: []const usize, pads: ?[]const usize, dilations: ?[]const usize, group: ?usize, auto_pad: ?[]const u8, fuse_act: c_int, fuse_pool: bool) !ConvPlan {
        const xd = try dims4(xshape);
        const wd = try dims4(kernel.shape);
        const yd = try dims4(yshape);
        const s = toI64(2, stride);
        var p = [_]i64{0} ** 4;
        var d = [_]i64{1} ** 2;
        if (pads) |pp| p = toI64(4, pp);
        if (dilations) |dd| d = toI64(2, dd);
        var ap_buf: [16:0]u8 = undefined;
        const ap: ?[*:0]const u8 = if (auto_pad) |a| blk: {
            if (a.len > 15) return TensorMathError.InvalidPadding;
            @memcpy(ap_buf[0..a.len], a);
            ap_buf[a.len] = 0;
            break :blk &ap_buf;
        } else null;
        var self = ConvPlan{};
        try toErr(zant_hip_conv2d_f32_prepack(ctx, &xd, kernel.data.ptr, &wd, if (bias) |b| b.data.ptr else null, &yd, &s, @intCast(stride.len), if (pads != null) &p else null, if (pads) |pp| @intCast(pp.len) else 0, if (dilations != null) &d else null, if (dilations) |dd| @intCast(dd.len) else 0, if (group) |g| @intCast(g) else -1, ap, fuse_act, @intFromBool(fuse_pool), &self.handle));
        return self;
    }

    pub fn run(self: *ConvPlan, x: [*]const f32, y: [*]f32) !void {
        try toErr(zant_hip_conv2d_f32_packed(ctx, self.handle, x, y));
    }

    pub fn deinit(self: *ConvPlan) void {
        zant_hip_conv2d_plan_destroy(ctx, self.handle);
        self.handle = null;
    }
};

// ---- device tensors ---------------------------------------------------------------------------------------

/// A Tensor(T) whose `data` is device memory of the context: the shape is copied with `allocator`, the data is
/// allocated with zant_hip_malloc.  `owns_memory` is false so Tensor.deinit frees neither; release with
/// `freeDeviceTensor`.
pub fn deviceTensor(comptime T: type, allocator: *const std.mem.Allocator, shape: []const usize) !Tensor(T) {
    var n: usize = 1;
    for (shape) |d| n *= d;
    var p: ?*anyopaque = null;
    try toErr(zant_hip_malloc(ctx, &p, @max(n, 1) * @sizeOf(T)));
    const shp = try allocator.dupe(usize, shape);
    const base: [*]T = @ptrCast(@alignCast(p.?));
    return Tensor(T){ .data = base[0..n], .size = n, .shape = shp, .allocator = allocator, .owns_memory = false };
}

pub fn freeDeviceTensor(comptime T: type, t: *Tensor(T)) void {
    _ = zant_hip_free(ctx, @ptrCast(t.data.ptr));
    t.allocator.free(t.shape);
    t.data = &[_]T{};
    t.shape = &[_]usize{};
    t.size = 0;
}

pub fn upload(comptime T: type, dst: *Tensor(T), src: []const T) !void {
    if (src.len != dst.size) return TensorError.InputArrayWrongSize;
    try toErr(zant_hip_upload(ctx, @ptrCast(dst.data.ptr), @ptrCast(src.ptr), src.len * @sizeOf(T)));
}

pub fn download(comptime T: type, dst: []T, src: *const Tensor(T)) !void {
    if (dst.len != src.size) return TensorError.InputArrayWrongSize;
    try toErr(zant_hip_download(ctx, @ptrCast(dst.ptr), @ptrCast(src.data.ptr), dst.len * @sizeOf(T)));
}
