// Memory-bound f32 operators: ReLU, LeakyReLU, Softmax, Add (same-size and broadcast), add_bias,
// Reshape and MaxPool (f32 and u8).  All are HBM-bound: 16-byte vector accesses on the contiguous
// axis, grid-stride loops sized to a few waves per CU.
#include "common.h"

namespace {

constexpr int kThreads = 256;

inline unsigned grid_for(int64_t work_items, int per_block, int num_cus) {
    int64_t blocks = ceil_div64(work_items, per_block);
    const int64_t cap = int64_t(num_cus) * 16;
    if (blocks > cap) blocks = cap;
    if (blocks < 1) blocks = 1;
    return unsigned(blocks);
}

// ---- unary f32 ---------------------------------------------------------------------------------

enum { UN_RELU = 0, UN_LEAKY = 1 };

template <int OP>
__device__ __forceinline__ float unary_op(float v, float slope) {
    if (OP == UN_RELU) return v > 0.0f ? v : 0.0f;  // NaN -> 0, like the reference's `if (x > 0)` on a zeroed output
    return v <= 0.0f ? slope * v : v;
}

template <int OP>
__global__ void __launch_bounds__(kThreads) unary_f32_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                            int64_t n, float slope) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int64_t n4 = n >> 2;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const f4 *x4 = reinterpret_cast<const f4 *>(x);
    f4 *y4 = reinterpret_cast<f4 *>(y);
    f4 v[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n4) v[u] = __builtin_nontemporal_load(x4 + j);
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n4) {
            f4 r;
            r.x = unary_op<OP>(v[u].x, slope);
            r.y = unary_op<OP>(v[u].y, slope);
            r.z = unary_op<OP>(v[u].z, slope);
            r.w = unary_op<OP>(v[u].w, slope);
            __builtin_nontemporal_store(r, y4 + j);
        }
    }
    if (blockIdx.x == 0) {  // the 0..3 elements behind the last full vector
        const int64_t j = (n4 << 2) + threadIdx.x;
        if (j < n) y[j] = unary_op<OP>(x[j], slope);
    }
}

template <int OP>
__global__ void __launch_bounds__(kThreads) unary_f32_unaligned_kernel(const float *__restrict__ x,
                                                                      float *__restrict__ y, int64_t n, float slope) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t j = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; j < n; j += step) y[j] = unary_op<OP>(x[j], slope);
}

template <int OP>
int launch_unary(zant_ctx *ctx, const float *x, float *y, int64_t n, float slope) {
    if (!ctx || (n && (!x || !y))) return ZANT_NullPointer;
    if (n <= 0) return ZANT_OK;
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    if (aligned) {
        KernelTimer kt(ctx);
        hipLaunchKernelGGL(unary_f32_kernel<OP>, dim3(zant_stream_grid(n >> 2)), dim3(kThreads), 0, ctx->stream, x, y, n,
                           slope);
    } else {
        KernelTimer kt(ctx);
        hipLaunchKernelGGL(unary_f32_unaligned_kernel<OP>, dim3(grid_for(n, kThreads, ctx->num_cus)), dim3(kThreads),
                           0, ctx->stream, x, y, n, slope);
    }
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// ---- softmax: one wavefront per row ------------------------------------------------------------

__device__ __forceinline__ float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__global__ void __launch_bounds__(kThreads) softmax_f32_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                              int64_t rows, int64_t cols) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = (int64_t(gridDim.x) * blockDim.x) >> 6;
    for (int64_t r = wave; r < rows; r += nwaves) {
        const float *xr = x + r * cols;
        float *yr = y + r * cols;
        float m = -INFINITY;
        for (int64_t j = lane; j < cols; j += 64) m = fmaxf(m, xr[j]);
        m = wave_max(m);
        float s = 0.0f;
        for (int64_t j = lane; j < cols; j += 64) {
            const float e = expf(xr[j] - m);
            yr[j] = e;
            s += e;
        }
        s = wave_sum(s);
        for (int64_t j = lane; j < cols; j += 64) yr[j] = yr[j] / s;
    }
}

// ---- add ----------------------------------------------------------------------------------------

__global__ void __launch_bounds__(kThreads) add_same_f32_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                               float *__restrict__ y, int64_t n, int vec) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    if (!vec) {  // unaligned operands: scalar, one element per thread of the same grid shape
        const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U * 4) + threadIdx.x;
        for (int u = 0; u < ZANT_STREAM_U * 4; ++u) {
            const int64_t j = base + u * kThreads;
            if (j < n) y[j] = a[j] + b[j];
        }
        return;
    }
    const int64_t n4 = n >> 2;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const f4 *a4 = reinterpret_cast<const f4 *>(a);
    const f4 *b4 = reinterpret_cast<const f4 *>(b);
    f4 *y4 = reinterpret_cast<f4 *>(y);
    f4 va[ZANT_STREAM_U], vb[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n4) { va[u] = __builtin_nontemporal_load(a4 + j); vb[u] = __builtin_nontemporal_load(b4 + j); }
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n4) __builtin_nontemporal_store(va[u] + vb[u], y4 + j);
    }
    if (blockIdx.x == 0) {
        const int64_t j = (n4 << 2) + threadIdx.x;
        if (j < n) y[j] = a[j] + b[j];
    }
}

struct BcastArgs {
    int rank;
    int64_t out_dim[8];
    int64_t sa[8];
    int64_t sb[8];
};

__global__ void __launch_bounds__(kThreads) add_bcast_f32_kernel(const float *__restrict__ a, const float *__restrict__ b,
                                                                float *__restrict__ y, int64_t n, BcastArgs g) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += step) {
        int64_t rem = i, ia = 0, ib = 0;
        for (int d = g.rank - 1; d >= 0; --d) {
            const int64_t pos = rem % g.out_dim[d];
            rem /= g.out_dim[d];
            ia += pos * g.sa[d];
            ib += pos * g.sb[d];
        }
        y[i] = a[ia] + b[ib];
    }
}

// y[i] += bias[i % len] over the last axis, in place.
__global__ void __launch_bounds__(kThreads) add_bias_f32_kernel(float *__restrict__ t, const float *__restrict__ bias,
                                                               int64_t n, int64_t len) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += step) t[i] += bias[i % len];
}

// ---- max pool -----------------------------------------------------------------------------------

struct PoolGeom {
    int64_t NC;
    int H, W, OH, OW, kh, kw, sh, sw, dh, dw, pt, pl;
};

template <typename T>
__device__ __forceinline__ T pool_lowest();
template <>
__device__ __forceinline__ float pool_lowest<float>() { return -INFINITY; }
template <>
__device__ __forceinline__ uint8_t pool_lowest<uint8_t>() { return 0; }
__device__ __forceinline__ float pool_max(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ uint8_t pool_max(uint8_t a, uint8_t b) { return a > b ? a : b; }

template <typename T>
__global__ void __launch_bounds__(kThreads) maxpool_generic_kernel(const T *__restrict__ x, T *__restrict__ y, PoolGeom g) {
    const int64_t total = g.NC * g.OH * g.OW;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int ow = int(i % g.OW);
        const int oh = int((i / g.OW) % g.OH);
        const int64_t nc = i / (int64_t(g.OW) * g.OH);
        const T *src = x + nc * g.H * g.W;
        T m = pool_lowest<T>();
        for (int kh = 0; kh < g.kh; ++kh) {
            const int ih = oh * g.sh - g.pt + kh * g.dh;
            if (ih < 0 || ih >= g.H) continue;
            for (int kw = 0; kw < g.kw; ++kw) {
                const int iw = ow * g.sw - g.pl + kw * g.dw;
                if (iw < 0 || iw >= g.W) continue;
                m = pool_max(m, src[ih * g.W + iw]);
            }
        }
        y[i] = m;
    }
}

// 2x2 / stride 2, no padding, no dilation: each thread produces PER outputs of one row from two
// contiguous input row segments (the common CNN case; fully coalesced loads and stores).
template <typename T, int PER>
__global__ void __launch_bounds__(kThreads) maxpool_2x2s2_kernel(const T *__restrict__ x, T *__restrict__ y, PoolGeom g) {
    const int ow_chunks = (g.OW + PER - 1) / PER;
    const int64_t total = g.NC * g.OH * ow_chunks;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int oc = int(i % ow_chunks);
        const int oh = int((i / ow_chunks) % g.OH);
        const int64_t nc = i / (int64_t(ow_chunks) * g.OH);
        const T *r0 = x + (nc * g.H + 2 * oh) * g.W + 2 * oc * PER;
        const T *r1 = r0 + g.W;
        T *dst = y + (nc * g.OH + oh) * g.OW + oc * PER;
        const int cnt = min(PER, g.OW - oc * PER);
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            if (j < cnt) {
                const T m0 = pool_max(r0[2 * j], r0[2 * j + 1]);
                const T m1 = pool_max(r1[2 * j], r1[2 * j + 1]);
                dst[j] = pool_max(m0, m1);
            }
        }
    }
}

int pool_geom(const int64_t xdim[4], const int64_t ydim[4], const int64_t kernel[2], const int64_t strides[2],
              const int64_t dil[2], const int64_t *pads, int n_pads, int auto_pad, PoolGeom *g) {
    if (!xdim || !ydim || !kernel || !strides || !dil) return ZANT_NullPointer;
    for (int i = 0; i < 4; ++i)
        if (xdim[i] < 0 || ydim[i] < 0 || xdim[i] > INT32_MAX || ydim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    if (kernel[0] <= 0 || kernel[1] <= 0 || strides[0] <= 0 || strides[1] <= 0 || dil[0] <= 0 || dil[1] <= 0)
        return ZANT_WrongStride;
    if (ydim[0] != xdim[0] || ydim[1] != xdim[1]) return ZANT_InvalidDimensions;
    int64_t top = 0, left = 0;
    // lean_onnx_maxpool's pad derivation (op_pooling.zig:593-618)
    if (auto_pad == ZANT_PAD_NOTSET) {
        if (pads && n_pads >= 4) { top = pads[0]; left = pads[1]; }
    } else if (auto_pad == ZANT_PAD_SAME_UPPER || auto_pad == ZANT_PAD_SAME_LOWER) {
        const int64_t th = (ydim[2] - 1) * strides[0] + kernel[0] - xdim[2];
        const int64_t tw = (ydim[3] - 1) * strides[1] + kernel[1] - xdim[3];
        if (auto_pad == ZANT_PAD_SAME_UPPER) { top = th / 2; left = tw / 2; }
        else { top = th - th / 2; left = tw - tw / 2; }
    } else if (auto_pad != ZANT_PAD_VALID) {
        return ZANT_InvalidPadding;
    }
    g->NC = xdim[0] * xdim[1];
    g->H = int(xdim[2]); g->W = int(xdim[3]); g->OH = int(ydim[2]); g->OW = int(ydim[3]);
    g->kh = int(kernel[0]); g->kw = int(kernel[1]); g->sh = int(strides[0]); g->sw = int(strides[1]);
    g->dh = int(dil[0]); g->dw = int(dil[1]); g->pt = int(top); g->pl = int(left);
    return ZANT_OK;
}

template <typename T>
int launch_maxpool(zant_ctx *ctx, const T *x, const int64_t xdim[4], T *y, const int64_t ydim[4],
                   const int64_t kernel[2], const int64_t strides[2], const int64_t dil[2], const int64_t *pads,
                   int n_pads, int auto_pad) {
    if (!ctx) return ZANT_NullPointer;
    PoolGeom g;
    int rc = pool_geom(xdim, ydim, kernel, strides, dil, pads, n_pads, auto_pad, &g);
    if (rc) return rc;
    const int64_t total = g.NC * g.OH * g.OW;
    if (total == 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    const bool fast = g.kh == 2 && g.kw == 2 && g.sh == 2 && g.sw == 2 && g.dh == 1 && g.dw == 1 && g.pt == 0 &&
                      g.pl == 0 && 2 * g.OH <= g.H && 2 * g.OW <= g.W;
    if (fast) {
        constexpr int PER = sizeof(T) == 1 ? 8 : 2;
        const int64_t items = g.NC * g.OH * ((g.OW + PER - 1) / PER);
        KernelTimer kt(ctx);
        hipLaunchKernelGGL((maxpool_2x2s2_kernel<T, PER>), dim3(grid_for(items, kThreads, ctx->num_cus)),
                           dim3(kThreads), 0, ctx->stream, x, y, g);
    } else {
        KernelTimer kt(ctx);
        hipLaunchKernelGGL(maxpool_generic_kernel<T>, dim3(grid_for(total, kThreads, ctx->num_cus)), dim3(kThreads), 0,
                           ctx->stream, x, y, g);
    }
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

}  // namespace

// -------------------------------------------------------------------------------------------------

extern "C" int zant_hip_relu_f32(zant_ctx *ctx, const float *x, float *y, int64_t n) {
    return launch_unary<UN_RELU>(ctx, x, y, n, 0.0f);
}

extern "C" int zant_hip_leaky_relu_f32(zant_ctx *ctx, const float *x, float slope, float *y, int64_t n) {
    return launch_unary<UN_LEAKY>(ctx, x, y, n, slope);
}

extern "C" int zant_hip_softmax_f32(zant_ctx *ctx, const float *x, float *y, int64_t rows, int64_t cols) {
    if (!ctx) return ZANT_NullPointer;
    if (rows < 0 || cols < 0) return ZANT_InvalidDimensions;
    if (rows == 0 || cols == 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(softmax_f32_kernel, dim3(grid_for(rows, kThreads / 64, ctx->num_cus)), dim3(kThreads), 0,
                       ctx->stream, x, y, rows, cols);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_add_f32(zant_ctx *ctx, const float *a, const int64_t *adim, int a_rank, const float *b,
                                const int64_t *bdim, int b_rank, float *y, int64_t *ydim_out, int *y_rank_out) {
    if (!ctx || !adim || !bdim) return ZANT_NullPointer;
    if (a_rank < 0 || b_rank < 0 || a_rank > 8 || b_rank > 8) return ZANT_InvalidDimensions;
    const int64_t asz = prod_dims(adim, a_rank), bsz = prod_dims(bdim, b_rank);
    if (asz == bsz) {  // lib_elementWise_math.zig:72-110
        if (y_rank_out) *y_rank_out = a_rank;
        if (ydim_out) for (int i = 0; i < a_rank; ++i) ydim_out[i] = adim[i];
        if (asz == 0) return ZANT_OK;
        if (!a || !b || !y) return ZANT_NullPointer;
        const int vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
        KernelTimer kt(ctx);
        hipLaunchKernelGGL(add_same_f32_kernel, dim3(zant_stream_grid((asz + 3) >> 2)), dim3(kThreads), 0, ctx->stream, a, b,
                           y, asz, vec);
        ZANT_LAUNCH_CHECK(ctx);
        return ZANT_OK;
    }
    BcastArgs g;
    g.rank = a_rank > b_rank ? a_rank : b_rank;
    int64_t s1[8], s2[8];
    for (int i = 0; i < g.rank; ++i) s1[i] = s2[i] = 1;
    for (int i = 0; i < a_rank; ++i) s1[g.rank - a_rank + i] = adim[i];  // :143-150
    for (int i = 0; i < b_rank; ++i) s2[g.rank - b_rank + i] = bdim[i];
    int64_t osz = 1;
    for (int i = 0; i < g.rank; ++i) {  // :153-158
        if (s1[i] != s2[i] && s1[i] != 1 && s2[i] != 1) return ZANT_IncompatibleBroadcastShapes;
        g.out_dim[i] = s1[i] > s2[i] ? s1[i] : s2[i];
        osz *= g.out_dim[i];
    }
    int64_t t1 = 1, t2 = 1;
    for (int i = g.rank - 1; i >= 0; --i) {
        g.sa[i] = s1[i] > 1 ? t1 : 0; t1 *= s1[i];
        g.sb[i] = s2[i] > 1 ? t2 : 0; t2 *= s2[i];
    }
    if (y_rank_out) *y_rank_out = g.rank;
    if (ydim_out) for (int i = 0; i < g.rank; ++i) ydim_out[i] = g.out_dim[i];
    if (osz == 0) return ZANT_OK;
    if (!a || !b || !y) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(add_bcast_f32_kernel, dim3(grid_for(osz, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                       a, b, y, osz, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_add_bias_f32(zant_ctx *ctx, float *t, const int64_t *tdim, int t_rank, const float *bias,
                                     const int64_t *bdim, int b_rank) {
    if (!ctx || !tdim || !bdim) return ZANT_NullPointer;
    const int64_t tsz = prod_dims(tdim, t_rank), bsz = prod_dims(bdim, b_rank);
    if (tsz == 0 || bsz == 0 || t_rank < 1) return ZANT_EmptyTensor;           // lib_elementWise_math.zig:24-29
    if (b_rank != 1) return ZANT_InputTensorsWrongShape;                       // :30-32
    if (bdim[0] != tdim[t_rank - 1]) return ZANT_InputTensorDimensionMismatch;  // :33-36
    if (!t || !bias) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(add_bias_f32_kernel, dim3(grid_for(tsz, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                       t, bias, tsz, bdim[0]);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_reshape(zant_ctx *ctx, const void *x, const int64_t *xdim, int x_rank, size_t elem_size,
                                const int64_t *new_shape, int new_rank, void *y, int64_t *ydim_out) {
    if (!ctx || !xdim || !new_shape || !ydim_out) return ZANT_NullPointer;
    const int64_t in_size = prod_dims(xdim, x_rank);
    int neg = -1;
    int64_t known = 1;
    for (int i = 0; i < new_rank; ++i) {  // lib_shape_math.zig:1153-1170
        if (new_shape[i] == 0) {
            if (i >= x_rank) return ZANT_InvalidInput;
            ydim_out[i] = xdim[i];
            known *= xdim[i];
        } else if (new_shape[i] < 0) {
            if (neg >= 0) return ZANT_InvalidInput;
            neg = i;
            ydim_out[i] = 1;
        } else {
            ydim_out[i] = new_shape[i];
            known *= new_shape[i];
        }
    }
    if (neg >= 0) {  // :1178-1188
        if (known == 0) return ZANT_InvalidInput;
        if (in_size % known != 0) return ZANT_InputArrayWrongSize;
        ydim_out[neg] = in_size / known;
    }
    if (prod_dims(ydim_out, new_rank) != in_size) return ZANT_InputArrayWrongSize;  // :1197-1199
    if (in_size == 0 || x == y) return ZANT_OK;  // a view inside the arena needs no copy
    if (!x || !y) return ZANT_NullPointer;
    ZANT_HIP_TRY(ctx, hipMemcpyAsync(y, x, size_t(in_size) * elem_size, hipMemcpyDeviceToDevice, ctx->stream));
    return ZANT_OK;
}

extern "C" int zant_hip_maxpool2d_f32(zant_ctx *ctx, const float *x, const int64_t xdim[4], float *y,
                                      const int64_t ydim[4], const int64_t kernel[2], const int64_t strides[2],
                                      const int64_t dil[2], const int64_t *pads, int n_pads, int auto_pad) {
    return launch_maxpool<float>(ctx, x, xdim, y, ydim, kernel, strides, dil, pads, n_pads, auto_pad);
}

extern "C" int zant_hip_maxpool2d_u8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], uint8_t *y,
                                     const int64_t ydim[4], const int64_t kernel[2], const int64_t strides[2],
                                     const int64_t dil[2], const int64_t *pads, int n_pads, int auto_pad) {
    return launch_maxpool<uint8_t>(ctx, x, xdim, y, ydim, kernel, strides, dil, pads, n_pads, auto_pad);
}

extern "C" int zant_hip_maxpool2d_out_shape(const int64_t xdim[4], const int64_t kernel[2], const int64_t strides[2],
                                            const int64_t dil[2], const int64_t pads[4], int auto_pad, int ceil_mode,
                                            int64_t ydim[4]) {
    if (!xdim || !kernel || !strides || !dil || !ydim) return ZANT_NullPointer;
    if (strides[0] <= 0 || strides[1] <= 0) return ZANT_WrongStride;
    const int64_t H = xdim[2], W = xdim[3];
    const int64_t ekh = (kernel[0] - 1) * dil[0] + 1, ekw = (kernel[1] - 1) * dil[1] + 1;  // op_pooling.zig:509-510
    int64_t ph = 0, pw = 0;
    switch (auto_pad) {
    case ZANT_PAD_NOTSET:
        if (!pads) return ZANT_NullPointer;
        ph = pads[0] + pads[2]; pw = pads[1] + pads[3];  // :513-520
        break;
    case ZANT_PAD_VALID: break;
    case ZANT_PAD_SAME_UPPER:
    case ZANT_PAD_SAME_LOWER: {
        const int64_t oh = (H + strides[0] - 1) / strides[0], ow = (W + strides[1] - 1) / strides[1];  // :531-532
        ph = (oh - 1) * strides[0] + ekh - H;  // :534-535
        pw = (ow - 1) * strides[1] + ekw - W;
        break;
    }
    default: return ZANT_InvalidPadding;
    }
    if (H + ph < ekh || W + pw < ekw) return ZANT_InvalidDimensions;
    if (ceil_mode) {  // :555-561
        ydim[2] = (H + ph - ekh + strides[0] - 1) / strides[0] + 1;
        ydim[3] = (W + pw - ekw + strides[1] - 1) / strides[1] + 1;
    } else {
        ydim[2] = (H + ph - ekh) / strides[0] + 1;
        ydim[3] = (W + pw - ekw) / strides[1] + 1;
    }
    ydim[0] = xdim[0]; ydim[1] = xdim[1];
    return ZANT_OK;
}
