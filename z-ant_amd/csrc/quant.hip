// int8 elementwise family: QuantizeLinear, DequantizeLinear, the fused Dequantize -> activation ->
// Quantize, the quantised residual add and the quantised global average pool.  The reference holds no
// quantised operators; these follow the ONNX definitions with ONE fixed f32 sequence so that results
// are bit-identical with the CPU checker: IEEE divide, round-half-to-even, add zero point, saturate.
// All are HBM-bound byte streams: 16 bytes per lane per access on the contiguous axis.
#include "quant_common.h"

namespace {

constexpr int kThreads = 256;

inline unsigned grid_for(int64_t items, int per_block, int num_cus) {
    int64_t blocks = ceil_div64(items, per_block);
    const int64_t cap = int64_t(num_cus) * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return unsigned(blocks);
}

struct AxisGeom {
    int64_t n, inner, alen;  // element count, product of dims after the axis, axis length
    int per_axis;
};

__global__ void __launch_bounds__(kThreads) quantize_kernel(const float *__restrict__ x, const float *__restrict__ scale,
                                                           const uint8_t *__restrict__ zp, uint8_t *__restrict__ y,
                                                           AxisGeom g) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < g.n; i += step) {
        const int64_t c = g.per_axis ? (i / g.inner) % g.alen : 0;
        y[i] = sat_u8_rne(x[i] / scale[c], zp ? zp[c] : uint8_t(0));
    }
}

__global__ void __launch_bounds__(kThreads) dequantize_kernel(const uint8_t *__restrict__ x, const float *__restrict__ scale,
                                                             const uint8_t *__restrict__ zp, float *__restrict__ y,
                                                             AxisGeom g) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < g.n; i += step) {
        const int64_t c = g.per_axis ? (i / g.inner) % g.alen : 0;
        y[i] = float(int(x[i]) - int(zp ? zp[c] : uint8_t(0))) * scale[c];
    }
}

// u8 -> u8 through a 256-entry table held in LDS (the function of one byte is evaluated 256 times
// with the exact f32 sequence, then applied 16 bytes per lane).
__global__ void __launch_bounds__(kThreads) qlinear_act_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ y,
                                                              int64_t n, QAct qa, int vec) {
    __shared__ uint8_t lut[256];
    lut[threadIdx.x] = qact_apply(uint8_t(threadIdx.x), qa);
    __syncthreads();
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    const int64_t i0 = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    int64_t done = 0;
    if (vec) {
        const int64_t n16 = n >> 4;
        const uint4 *x16 = reinterpret_cast<const uint4 *>(x);
        uint4 *y16 = reinterpret_cast<uint4 *>(y);
        for (int64_t i = i0; i < n16; i += step) {
            uint4 v = x16[i];
            uint32_t *w = reinterpret_cast<uint32_t *>(&v);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t u = w[j];
                w[j] = uint32_t(lut[u & 255]) | (uint32_t(lut[(u >> 8) & 255]) << 8) |
                       (uint32_t(lut[(u >> 16) & 255]) << 16) | (uint32_t(lut[u >> 24]) << 24);
            }
            y16[i] = v;
        }
        done = n16 << 4;
    }
    for (int64_t i = done + i0; i < n; i += step) y[i] = lut[x[i]];
}

struct QAddArgs {
    float a_scale, b_scale, y_scale;
    int a_zp, b_zp;
    uint8_t y_zp;
};

__device__ __forceinline__ uint8_t qadd_one(uint8_t a, uint8_t b, const QAddArgs &q) {
    const float fa = float(int(a) - q.a_zp) * q.a_scale;
    const float fb = float(int(b) - q.b_zp) * q.b_scale;
    return sat_u8_rne((fa + fb) / q.y_scale, q.y_zp);
}

__global__ void __launch_bounds__(kThreads) qlinear_add_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                              uint8_t *__restrict__ y, int64_t n, QAddArgs q, int vec) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    const int64_t i0 = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    int64_t done = 0;
    if (vec) {
        const int64_t n16 = n >> 4;
        const uint4 *a16 = reinterpret_cast<const uint4 *>(a);
        const uint4 *b16 = reinterpret_cast<const uint4 *>(b);
        uint4 *y16 = reinterpret_cast<uint4 *>(y);
        for (int64_t i = i0; i < n16; i += step) {
            uint4 va = a16[i], vb = b16[i], vy;
            const uint32_t *wa = reinterpret_cast<const uint32_t *>(&va);
            const uint32_t *wb = reinterpret_cast<const uint32_t *>(&vb);
            uint32_t *wy = reinterpret_cast<uint32_t *>(&vy);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                uint32_t r = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    r |= uint32_t(qadd_one(uint8_t(wa[j] >> (8 * k)), uint8_t(wb[j] >> (8 * k)), q)) << (8 * k);
                wy[j] = r;
            }
            y16[i] = vy;
        }
        done = n16 << 4;
    }
    for (int64_t i = done + i0; i < n; i += step) y[i] = qadd_one(a[i], b[i], q);
}

// One wavefront per (n, c) plane: exact i32 sum, then the fixed f32 sequence.
__global__ void __launch_bounds__(kThreads) qgap_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ y, int64_t planes,
                                                       int hw, float x_scale, int x_zp, float y_scale, uint8_t y_zp) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = (int64_t(gridDim.x) * blockDim.x) >> 6;
    for (int64_t p = wave; p < planes; p += nwaves) {
        const uint8_t *src = x + p * hw;
        int s = 0;
        for (int j = lane; j < hw; j += 64) s += int(src[j]) - x_zp;
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if (lane == 0) {
            const float mean = (float(s) * x_scale) / float(hw);
            y[p] = sat_u8_rne(mean / y_scale, y_zp);
        }
    }
}

int axis_geom(const int64_t *dim, int rank, int64_t n_scale, int axis, AxisGeom *g) {
    if (!dim) return ZANT_NullPointer;
    if (rank < 0 || rank > 8 || n_scale < 1) return ZANT_InvalidDimensions;
    g->n = prod_dims(dim, rank);
    g->inner = 1; g->alen = 1; g->per_axis = 0;
    if (n_scale > 1) {
        if (axis < -rank || axis >= rank) return ZANT_InvalidDimensions;
        if (axis < 0) axis += rank;
        g->alen = dim[axis];
        for (int i = axis + 1; i < rank; ++i) g->inner *= dim[i];
        if (n_scale != g->alen) return ZANT_InputTensorDimensionMismatch;
        g->per_axis = 1;
    }
    return ZANT_OK;
}

}  // namespace

extern "C" int zant_hip_quantize_linear_f32_u8(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank,
                                               const float *y_scale, const uint8_t *y_zp, int64_t n_scale, int axis,
                                               uint8_t *y) {
    if (!ctx) return ZANT_NullPointer;
    AxisGeom g;
    int rc = axis_geom(xdim, rank, n_scale, axis, &g);
    if (rc) return rc;
    if (g.n == 0) return ZANT_OK;
    if (!x || !y || !y_scale) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(quantize_kernel, dim3(grid_for(g.n, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x,
                       y_scale, y_zp, y, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_dequantize_linear_u8_f32(zant_ctx *ctx, const uint8_t *x, const int64_t *xdim, int rank,
                                                 const float *x_scale, const uint8_t *x_zp, int64_t n_scale, int axis,
                                                 float *y) {
    if (!ctx) return ZANT_NullPointer;
    AxisGeom g;
    int rc = axis_geom(xdim, rank, n_scale, axis, &g);
    if (rc) return rc;
    if (g.n == 0) return ZANT_OK;
    if (!x || !y || !x_scale) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(dequantize_kernel, dim3(grid_for(g.n, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x,
                       x_scale, x_zp, y, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_qlinear_act_u8(zant_ctx *ctx, const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act,
                                       float alpha, float y_scale, uint8_t y_zp, uint8_t *y) {
    if (!ctx) return ZANT_NullPointer;
    if (act < ZANT_ACT_NONE || act > ZANT_ACT_RELU6) return ZANT_InvalidInput;
    if (n <= 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    QAct qa;
    qa.act = act; qa.alpha = alpha; qa.in_scale = x_scale; qa.in_zp = x_zp; qa.out_scale = y_scale; qa.out_zp = y_zp;
    const int vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qlinear_act_kernel, dim3(grid_for(n, kThreads * 16, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                       x, y, n, qa, vec);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_qlinear_add_u8(zant_ctx *ctx, const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b,
                                       float b_scale, uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n) {
    if (!ctx) return ZANT_NullPointer;
    if (n <= 0) return ZANT_OK;
    if (!a || !b || !y) return ZANT_NullPointer;
    QAddArgs q;
    q.a_scale = a_scale; q.b_scale = b_scale; q.y_scale = y_scale; q.a_zp = a_zp; q.b_zp = b_zp; q.y_zp = y_zp;
    const int vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qlinear_add_kernel, dim3(grid_for(n, kThreads * 16, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                       a, b, y, n, q, vec);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_qlinear_global_avgpool_u8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale,
                                                  uint8_t x_zp, float y_scale, uint8_t y_zp, uint8_t *y) {
    if (!ctx || !xdim) return ZANT_NullPointer;
    const int64_t planes = xdim[0] * xdim[1], hw = xdim[2] * xdim[3];
    if (planes < 0 || hw <= 0 || hw > (1 << 23)) return ZANT_InvalidDimensions;  // i32 sum cannot overflow
    if (planes == 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qgap_kernel, dim3(grid_for(planes, kThreads / 64, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x,
                       y, planes, int(hw), x_scale, int(x_zp), y_scale, y_zp);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
