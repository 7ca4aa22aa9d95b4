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

enum { UN_RELU = 0, UN_LEAKY = 1, UN_SIGMOID = 2 };

template <int OP>
__device__ __forceinline__ float unary_op(float v, float slope) {
    if (OP == UN_RELU) return v > 0.0f ? v : 0.0f;  // NaN -> 0, like the reference's `if (x > 0)` on a zeroed output
    if (OP == UN_SIGMOID) return 1.0f / (1.0f + expf(-v));  // lib_activation_function_math.zig:118
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

// p / d for 0 <= p < 2^20, d > 0, inv = 1.0f / d (the float quotient is off by at most one; the remainder corrects it).
__device__ __forceinline__ int small_div_host(int p, int d, float inv) {
    int q = int(float(p) * inv);
    const int r = p - q * d;
    q += r >= d ? 1 : 0;
    q -= r < 0 ? 1 : 0;
    return q;
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

// Rows of at most 16 values: one thread per row, the row in registers (a wavefront per row would leave most lanes
// idle).  A workgroup walks chunks of 256 rows; a chunk is one contiguous span that crosses HBM as whole 16-byte
// vectors into LDS and back, and each thread picks its row out of LDS.  The loop is software-pipelined: the loads of
// chunk i + 1 are in flight (in registers) while chunk i is computed and written out, and the two LDS buffers take
// turns, so a workgroup always has a chunk's bytes on their way -- one chunk per workgroup, load -> compute -> store in
// sequence, left the memory system idle for most of a workgroup's life.  Sequential max / sum over the row, in column
// order like the reference.
constexpr int kSoftmaxVecs = 4;  // 16-byte vectors per thread and chunk: 256 rows x 16 columns x 4 bytes / 256 threads / 16

__global__ void __launch_bounds__(kThreads) softmax_small_f32_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                    int64_t rows, int cols, int vec) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) float buf[2][kThreads * 16];
    const int64_t n_chunks = (rows + kThreads - 1) / kThreads;
    f4 pre[kSoftmaxVecs];
    // a chunk's vectors into registers (vec: spans start on 16-byte boundaries; otherwise the scalar path below)
    auto fetch = [&](int64_t chunk) {
        const int64_t row0 = chunk * kThreads;
        const int nel = int(min(int64_t(kThreads), rows - row0)) * cols, nvec = nel >> 2;
        const f4 *xb = reinterpret_cast<const f4 *>(x + row0 * cols);
#pragma unroll
        for (int u = 0; u < kSoftmaxVecs; ++u) {
            const int i = u * kThreads + int(threadIdx.x);
            if (i < nvec) pre[u] = __builtin_nontemporal_load(xb + i);
        }
    };
    int64_t chunk = blockIdx.x;
    if (vec && chunk < n_chunks) fetch(chunk);
    for (int par = 0; chunk < n_chunks; chunk += gridDim.x, par ^= 1) {
        float *b = buf[par];
        const int64_t row0 = chunk * kThreads;
        const int nrows = int(min(int64_t(kThreads), rows - row0)), nel = nrows * cols;
        const float *xb = x + row0 * cols;
        float *yb = y + row0 * cols;
        const int nvec = vec ? nel >> 2 : 0;
#pragma unroll
        for (int u = 0; u < kSoftmaxVecs; ++u) {
            const int i = u * kThreads + int(threadIdx.x);
            if (i < nvec) reinterpret_cast<f4 *>(b)[i] = pre[u];
        }
        for (int i = (nvec << 2) + threadIdx.x; i < nel; i += kThreads) b[i] = xb[i];
        __syncthreads();  // (also: everybody has left the previous chunk's write-out of the other buffer)
        if (vec && chunk + gridDim.x < n_chunks) fetch(chunk + gridDim.x);
        if (int(threadIdx.x) < nrows) {
            float *row = b + threadIdx.x * cols;
            float v[16];
            float m = -INFINITY;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                v[j] = j < cols ? row[j] : -INFINITY;
                m = fmaxf(m, v[j]);
            }
            // exp through the hardware's base-2 exponential (arguments are <= 0, results in (0, 1]: relative error a few
            // 1e-7, far inside the operator's tolerance) and one division per row: ten full-precision exponentials and
            // ten divisions per row were more vector work than the row's 80 bytes of traffic take to move
            float sum = 0.0f;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                v[j] = j < cols ? __builtin_amdgcn_exp2f((v[j] - m) * 1.44269504088896340736f) : 0.0f;
                sum += v[j];
            }
            const float inv = 1.0f / sum;
#pragma unroll
            for (int j = 0; j < 16; ++j)
                if (j < cols) row[j] = v[j] * inv;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kSoftmaxVecs; ++u) {
            const int i = u * kThreads + int(threadIdx.x);
            if (i < nvec) __builtin_nontemporal_store(reinterpret_cast<const f4 *>(b)[i], reinterpret_cast<f4 *>(yb) + i);
        }
        for (int i = (nvec << 2) + threadIdx.x; i < nel; i += kThreads) yb[i] = b[i];
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

// One operand has the output's shape, the other a single axis of length C and ones elsewhere (a per-channel term):
// y[i] = big[i] + small[(i / inner) % C].  With inner a multiple of 4 the four floats of a vector share a channel.
__global__ void __launch_bounds__(kThreads) add_channel_f32_kernel(const float *__restrict__ big, const float *__restrict__ small,
                                                                  float *__restrict__ y, uint32_t n4, uint32_t inner4, uint32_t C) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const uint32_t base = blockIdx.x * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const f4 *b4 = reinterpret_cast<const f4 *>(big);
    f4 *y4 = reinterpret_cast<f4 *>(y);
    f4 v[ZANT_STREAM_U];
    float c[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const uint32_t j = base + u * kThreads;
        if (j < n4) {
            v[u] = __builtin_nontemporal_load(b4 + j);
            c[u] = small[(j / inner4) % C];
        }
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const uint32_t j = base + u * kThreads;
        if (j < n4) __builtin_nontemporal_store(v[u] + c[u], y4 + j);
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

// 2x2 / stride 2 with even rows of inputs read as vectors: a thread turns two row segments of 2 * VEC inputs into VEC
// outputs (f32: VEC = 1, two 8-byte loads; u8: VEC = 8, two 16-byte loads, one 8-byte store).  A workgroup covers
// kThreads * ZANT_STREAM_U consecutive output vectors of the flattened [NC * OH, OW / VEC] grid and issues all its
// loads before its stores, nontemporal both ways (the streaming pattern of the elementwise kernels).  Needs W even
// (f32) or a multiple of 16 (u8), OW a multiple of VEC and aligned bases; the host checks.
template <typename T, int VEC>
__global__ void __launch_bounds__(kThreads) maxpool_2x2s2_stream_kernel(const T *__restrict__ x, T *__restrict__ y, PoolGeom g,
                                                                      int64_t total_vec, int ow_vec, float inv_ow_vec,
                                                                      float inv_oh) {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    constexpr bool F32 = sizeof(T) == 4;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    // flat row index of the first vector of this workgroup, then block-local arithmetic in 32 bits
    const int64_t row0 = (int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U)) / ow_vec;
    const int col0 = int((int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U)) - row0 * ow_vec);
    const int64_t nc0 = row0 / g.OH;
    const int oh0 = int(row0 - nc0 * g.OH);
    u4 r0[ZANT_STREAM_U], r1[ZANT_STREAM_U];
    int64_t dst[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int local = col0 + int(threadIdx.x) + u * kThreads;         // < ow_vec + kThreads * ZANT_STREAM_U
        const int drow = small_div_host(local, ow_vec, inv_ow_vec), oc = local - drow * ow_vec;
        const int ohl = oh0 + drow;                                       // rows past this plane roll over
        const int dnc = small_div_host(ohl, g.OH, inv_oh), oh = ohl - dnc * g.OH;
        const int64_t nc = nc0 + dnc;
        const T *p0 = x + (nc * g.H + 2 * oh) * int64_t(g.W) + int64_t(oc) * 2 * VEC;
        dst[u] = (nc * g.OH + oh) * int64_t(g.OW) + int64_t(oc) * VEC;
        if (base + u * kThreads < total_vec) {
            if (F32) {
                const f2 a = __builtin_nontemporal_load(reinterpret_cast<const f2 *>(p0));
                const f2 b = __builtin_nontemporal_load(reinterpret_cast<const f2 *>(p0 + g.W));
                r0[u][0] = __float_as_uint(a[0]); r0[u][1] = __float_as_uint(a[1]);
                r1[u][0] = __float_as_uint(b[0]); r1[u][1] = __float_as_uint(b[1]);
            } else {
                r0[u] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p0));
                r1[u] = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(p0 + g.W));
            }
        }
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        if (base + u * kThreads >= total_vec) continue;
        if (F32) {
            const float m = fmaxf(fmaxf(__uint_as_float(r0[u][0]), __uint_as_float(r0[u][1])),
                                  fmaxf(__uint_as_float(r1[u][0]), __uint_as_float(r1[u][1])));
            __builtin_nontemporal_store(m, reinterpret_cast<float *>(y) + dst[u]);
        } else {
            // bytes as 16-bit lanes (even bytes and odd bytes of a dword apart): the vertical maximum is one packed
            // 16-bit max per half, the horizontal one (bytes 0|1 and 2|3) the packed max of the two halves, and one byte
            // permute gathers the four window maxima of two input dwords
            typedef unsigned short us2 __attribute__((ext_vector_type(2)));
            auto pk = [](uint32_t v) { us2 r; r[0] = (unsigned short)(v & 0xffffu); r[1] = (unsigned short)(v >> 16); return r; };
            auto window_max = [&](uint32_t a, uint32_t b) -> uint32_t {  // -> max(bytes 0,1) | max(bytes 2,3) << 16
                const us2 e = __builtin_elementwise_max(pk(a & 0x00ff00ffu), pk(b & 0x00ff00ffu));
                const us2 od = __builtin_elementwise_max(pk((a >> 8) & 0x00ff00ffu), pk((b >> 8) & 0x00ff00ffu));
                const us2 h = __builtin_elementwise_max(e, od);
                return uint32_t(h[0]) | (uint32_t(h[1]) << 16);
            };
            u2 o;
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                const uint32_t lo = window_max(r0[u][d * 2], r1[u][d * 2]), hi = window_max(r0[u][d * 2 + 1], r1[u][d * 2 + 1]);
                o[d] = __builtin_amdgcn_perm(hi, lo, 0x06040200u);  // bytes 0, 2 of lo then bytes 0, 2 of hi
            }
            __builtin_nontemporal_store(o, reinterpret_cast<u2 *>(reinterpret_cast<uint8_t *>(y) + dst[u]));
        }
    }
}

// 2x2 / stride 2 on f32 planes that are not a whole number of vectors wide (26 x 26 -> 13 x 13 ...): a workgroup copies G
// whole consecutive planes to LDS -- a contiguous run of the input, read as 16-byte vectors whatever the row length --
// and writes their G * OH * OW results, also a contiguous run, as 16-byte vectors, four results per thread.  The rows of
// a window are two 8-byte LDS reads (W is even).  G is a multiple of 4, so both runs start on 16-byte boundaries.
constexpr int kPoolLdsFloats = 4 * 1024;  // 16 KB: eight workgroups (all 32 wave slots) share a CU
template <bool AVG>  // AVG: the average in the reference's tap order (op_pooling.zig:373-408) instead of the maximum
__global__ void __launch_bounds__(kThreads) pool_2x2s2_planes_f32_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                           int64_t NC, int G, int H, int W, int OH, int OW,
                                                                           float inv_ohw, float inv_ow) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) float pl[kPoolLdsFloats];
    const int64_t p0 = int64_t(blockIdx.x) * G;
    const int planes = int(min<int64_t>(G, NC - p0));
    const int HW = H * W, OHW = OH * OW;
    const int n_in = planes * HW, n_out = planes * OHW;  // n_in is a multiple of 4 unless this is the tensor's tail
    const float *src = x + p0 * HW;
    const int n_in4 = n_in >> 2;
    constexpr int B = kPoolLdsFloats / 4 / kThreads;  // every vector of a full LDS buffer in flight at once: 12 per thread
    for (int i0 = 0; i0 < n_in4; i0 += kThreads * B) {
        f4 v[B];
#pragma unroll
        for (int u = 0; u < B; ++u) {
            const int i = i0 + u * kThreads + int(threadIdx.x);
            if (i < n_in4) v[u] = __builtin_nontemporal_load(reinterpret_cast<const f4 *>(src) + i);
        }
#pragma unroll
        for (int u = 0; u < B; ++u) {
            const int i = i0 + u * kThreads + int(threadIdx.x);
            if (i < n_in4) reinterpret_cast<f4 *>(pl)[i] = v[u];
        }
    }
    for (int i = (n_in4 << 2) + int(threadIdx.x); i < n_in; i += kThreads) pl[i] = src[i];
    __syncthreads();
    float *dst = y + p0 * OHW;
    auto one = [&](int o) {
        const int pz = small_div_host(o, OHW, inv_ohw), rem = o - pz * OHW;
        const int oh = small_div_host(rem, OW, inv_ow), ow = rem - oh * OW;
        const float *r = pl + pz * HW + 2 * oh * W + 2 * ow;
        const f2 a = *reinterpret_cast<const f2 *>(r), b = *reinterpret_cast<const f2 *>(r + W);
        if (AVG) return (((a[0] + a[1]) + b[0]) + b[1]) / 4.0f;  // taps (0,0), (0,1), (1,0), (1,1), divided by their count
        return fmaxf(fmaxf(a[0], a[1]), fmaxf(b[0], b[1]));
    };
    const int n_out4 = n_out >> 2;
    for (int i = int(threadIdx.x); i < n_out4; i += kThreads) {
        f4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = one(4 * i + e);
        __builtin_nontemporal_store(o, reinterpret_cast<f4 *>(dst) + i);
    }
    for (int o = (n_out4 << 2) + int(threadIdx.x); o < n_out; o += kThreads) dst[o] = one(o);
}

// The same for u8 planes whose rows are whole 16-byte vectors but whose result rows are not (48 x 48 -> 24 x 24 ...): a
// thread turns two pairs of 16-byte LDS row segments into two groups of eight results (each group lies inside one result
// row: OW is a multiple of 8) and stores them as one 16-byte vector.  H * W and OH * OW are multiples of 16.
__global__ void __launch_bounds__(kThreads) maxpool_2x2s2_planes_u8_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ y,
                                                                          int64_t NC, int G, int H, int W, int OH, int OW,
                                                                          float inv_ohw8, float inv_ow8) {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    __shared__ __attribute__((aligned(16))) uint8_t pl[kPoolLdsFloats * 4];
    const int64_t p0 = int64_t(blockIdx.x) * G;
    const int planes = int(min<int64_t>(G, NC - p0));
    const int HW = H * W, OHW = OH * OW;
    const int n_in16 = planes * HW / 16, n_out16 = planes * OHW / 16;
    const u4 *src = reinterpret_cast<const u4 *>(x + p0 * HW);
    constexpr int B = kPoolLdsFloats / 4 / kThreads;
    for (int i0 = 0; i0 < n_in16; i0 += kThreads * B) {
        u4 v[B];
#pragma unroll
        for (int u = 0; u < B; ++u) {
            const int i = i0 + u * kThreads + int(threadIdx.x);
            if (i < n_in16) v[u] = __builtin_nontemporal_load(src + i);
        }
#pragma unroll
        for (int u = 0; u < B; ++u) {
            const int i = i0 + u * kThreads + int(threadIdx.x);
            if (i < n_in16) reinterpret_cast<u4 *>(pl)[i] = v[u];
        }
    }
    __syncthreads();
    auto pk = [](uint32_t v) { us2 r; r[0] = (unsigned short)(v & 0xffffu); r[1] = (unsigned short)(v >> 16); return r; };
    auto window_max = [&](uint32_t a, uint32_t b) -> uint32_t {  // -> max(bytes 0,1) | max(bytes 2,3) << 16
        const us2 e = __builtin_elementwise_max(pk(a & 0x00ff00ffu), pk(b & 0x00ff00ffu));
        const us2 od = __builtin_elementwise_max(pk((a >> 8) & 0x00ff00ffu), pk((b >> 8) & 0x00ff00ffu));
        const us2 h = __builtin_elementwise_max(e, od);
        return uint32_t(h[0]) | (uint32_t(h[1]) << 16);
    };
    const int ohw8 = OHW / 8, ow8 = OW / 8;
    u4 *dst = reinterpret_cast<u4 *>(y + p0 * OHW);
    for (int i = int(threadIdx.x); i < n_out16; i += kThreads) {
        u4 o;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int g8 = 2 * i + h;  // group of eight results: plane, result row, eight columns
            const int pz = small_div_host(g8, ohw8, inv_ohw8), rem = g8 - pz * ohw8;
            const int oh = small_div_host(rem, ow8, inv_ow8), oc = rem - oh * ow8;
            const uint8_t *r = pl + pz * HW + 2 * oh * W + 16 * oc;
            const u4 a = *reinterpret_cast<const u4 *>(r), b = *reinterpret_cast<const u4 *>(r + W);
            o[2 * h] = __builtin_amdgcn_perm(window_max(a[1], b[1]), window_max(a[0], b[0]), 0x06040200u);
            o[2 * h + 1] = __builtin_amdgcn_perm(window_max(a[3], b[3]), window_max(a[2], b[2]), 0x06040200u);
        }
        __builtin_nontemporal_store(o, dst + i);
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
    constexpr int VEC = sizeof(T) == 1 ? 8 : 1;
    const bool stream = fast && g.H >= 2 * g.OH && g.OW % VEC == 0 && g.W % (sizeof(T) == 1 ? 16 : 2) == 0 &&
                        (reinterpret_cast<uintptr_t>(x) % (sizeof(T) == 1 ? 16 : 8)) == 0 &&
                        (reinterpret_cast<uintptr_t>(y) % (sizeof(T) == 1 ? 8 : 4)) == 0 && g.OW / VEC < (1 << 18) && g.OH < (1 << 18);
    // f32 planes of a few KB whose rows are not whole vectors: the plane-staged kernel reads and writes 16-byte vectors
    if (sizeof(T) == 4 && fast && g.W % 2 == 0 && g.W % 8 != 0 && int64_t(g.H) * g.W * 4 <= kPoolLdsFloats &&
        int64_t(g.OH) * g.OW >= 4 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0) {
        const int G = int(std::min<int64_t>((kPoolLdsFloats / (int64_t(g.H) * g.W)) & ~int64_t(3), 64));
        if (G >= 4 && ceil_div64(g.NC, G) < (int64_t(1) << 31)) {
            KernelTimer kt(ctx);
            ZANT_KERNEL_NAME(ctx, "pool_2x2s2_planes_f32_kernel<false>");
            hipLaunchKernelGGL(pool_2x2s2_planes_f32_kernel<false>, dim3(unsigned(ceil_div64(g.NC, G))), dim3(kThreads), 0, ctx->stream,
                               reinterpret_cast<const float *>(x), reinterpret_cast<float *>(y), g.NC, G, g.H, g.W, g.OH, g.OW,
                               1.0f / float(g.OH * g.OW), 1.0f / float(g.OW));
            ZANT_LAUNCH_CHECK(ctx);
            return ZANT_OK;
        }
    }
    if (sizeof(T) == 1 && fast && g.W % 16 == 0 && g.OW % 8 == 0 && g.OW % 16 != 0 && (int64_t(g.OH) * g.OW) % 16 == 0 &&
        int64_t(g.H) * g.W <= kPoolLdsFloats * 4 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0) {
        const int G = int(std::min<int64_t>(kPoolLdsFloats * 4 / (int64_t(g.H) * g.W), 64));
        if (G >= 1 && ceil_div64(g.NC, G) < (int64_t(1) << 31)) {
            KernelTimer kt(ctx);
            ZANT_KERNEL_NAME(ctx, "maxpool_2x2s2_planes_u8_kernel");
            hipLaunchKernelGGL(maxpool_2x2s2_planes_u8_kernel, dim3(unsigned(ceil_div64(g.NC, G))), dim3(kThreads), 0, ctx->stream,
                               reinterpret_cast<const uint8_t *>(x), reinterpret_cast<uint8_t *>(y), g.NC, G, g.H, g.W, g.OH, g.OW,
                               1.0f / float(g.OH * g.OW / 8), 1.0f / float(g.OW / 8));
            ZANT_LAUNCH_CHECK(ctx);
            return ZANT_OK;
        }
    }
    if (stream) {
        const int ow_vec = g.OW / VEC;
        const int64_t total_vec = g.NC * g.OH * ow_vec;
        KernelTimer kt(ctx);
        hipLaunchKernelGGL((maxpool_2x2s2_stream_kernel<T, VEC>), dim3(zant_stream_grid(total_vec)), dim3(kThreads), 0, ctx->stream,
                           x, y, g, total_vec, ow_vec, 1.0f / float(ow_vec), 1.0f / float(g.OH));
    } else if (fast) {
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

// ---- average pool (pool_forward, .Avg: op_pooling.zig:373-408) -------------------------------------------------------
// One thread per output: the sum of the window's taps that lie inside the input, in (row, column) order like the
// reference, divided by their count -- or, with count_include_pad, by the number of taps inside the padded input.
struct AvgGeom {
    int64_t NC;
    int H, W, OH, OW, kh, kw, sh, sw, pt, pl, pb, pr, include_pad;
};

__global__ void __launch_bounds__(kThreads) avgpool_f32_kernel(const float *__restrict__ x, float *__restrict__ y, AvgGeom g) {
    const int64_t total = g.NC * g.OH * g.OW;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int ow = int(i % g.OW);
        const int oh = int((i / g.OW) % g.OH);
        const int64_t nc = i / (int64_t(g.OW) * g.OH);
        const float *src = x + nc * g.H * g.W;
        const int ih0 = oh * g.sh - g.pt, iw0 = ow * g.sw - g.pl;
        float sum = 0.0f;
        for (int kr = 0; kr < g.kh; ++kr) {
            const int ih = ih0 + kr;
            if (ih < 0 || ih >= g.H) continue;
            for (int kc = 0; kc < g.kw; ++kc) {
                const int iw = iw0 + kc;
                if (iw >= 0 && iw < g.W) sum += src[ih * g.W + iw];
            }
        }
        // taps inside the input / inside the padded input: products of the row and column overlaps
        const int rows_in = min(ih0 + g.kh, g.H) - max(ih0, 0), cols_in = min(iw0 + g.kw, g.W) - max(iw0, 0);
        const int rows_pad = min(ih0 + g.kh, g.H + g.pb) - ih0, cols_pad = min(iw0 + g.kw, g.W + g.pr) - iw0;
        const int cnt = g.include_pad ? rows_pad * cols_pad : max(rows_in, 0) * max(cols_in, 0);
        y[i] = cnt > 0 ? sum / float(cnt) : 0.0f;
    }
}

// 2x2 / stride 2, no padding: each thread produces two outputs of one row from two 16-byte row segments.
__global__ void __launch_bounds__(kThreads) avgpool_2x2s2_f32_kernel(const float *__restrict__ x, float *__restrict__ y, AvgGeom g,
                                                                     int64_t total2) {
    const int ow2 = g.OW >> 1;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total2; i += step) {
        const int c = int(i % ow2);
        const int64_t row = i / ow2;            // (nc, oh)
        const int oh = int(row % g.OH);
        const int64_t nc = row / g.OH;
        const float *src = x + (nc * g.H + 2 * oh) * g.W + 4 * c;
        const float4 a = *reinterpret_cast<const float4 *>(src), b = *reinterpret_cast<const float4 *>(src + g.W);
        float2 o;
        o.x = (((a.x + a.y) + b.x) + b.y) / 4.0f;  // the reference's tap order: (0,0), (0,1), (1,0), (1,1)
        o.y = (((a.z + a.w) + b.z) + b.w) / 4.0f;
        *reinterpret_cast<float2 *>(y + row * g.OW + 2 * c) = o;
    }
}

// ---- BatchNormalization, inference form (BatchNormLayer.forward, batchNormLayer.zig:130-148) -------------------------
// y = (x - mean[f]) / sqrt(var[f] + eps) * gamma[f] + beta[f] in the reference's order of operations; f = the index on
// axis 1, `inner` elements per (batch, feature) pair.
__global__ void __launch_bounds__(kThreads) batchnorm_f32_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                 const float *__restrict__ gamma, const float *__restrict__ beta,
                                                                 const float *__restrict__ mean, const float *__restrict__ var,
                                                                 float eps, int64_t total, int64_t inner, int features) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int f = int((i / inner) % features);
        const float sd = sqrtf(var[f] + eps);
        const float xn = (x[i] - mean[f]) / sd;
        y[i] = xn * gamma[f] + beta[f];
    }
}
// inner a multiple of 4 and 16-byte aligned pointers: one feature per vector
__global__ void __launch_bounds__(kThreads) batchnorm_vec_f32_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                     const float *__restrict__ gamma, const float *__restrict__ beta,
                                                                     const float *__restrict__ mean, const float *__restrict__ var,
                                                                     float eps, int64_t total4, uint32_t inner4, uint32_t features) {
    // the streaming pattern: a workgroup's ZANT_STREAM_U x 256 vectors are all loaded before any is stored
    typedef float f4 __attribute__((ext_vector_type(4)));
    const f4 *x4 = reinterpret_cast<const f4 *>(x);
    f4 *y4 = reinterpret_cast<f4 *>(y);
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    // (batch, feature) pair of the workgroup's first vector; the vectors of a thread are kThreads apart
    const int64_t pair0 = (int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U)) / inner4;
    const uint32_t off0 = uint32_t(int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) - pair0 * inner4);
    const uint32_t f0 = uint32_t(pair0 % features);
    f4 v[ZANT_STREAM_U];
    float sd[ZANT_STREAM_U], m[ZANT_STREAM_U], ga[ZANT_STREAM_U], be[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < total4) {
            v[u] = __builtin_nontemporal_load(x4 + j);
            const uint32_t f = (f0 + (off0 + uint32_t(threadIdx.x) + uint32_t(u * kThreads)) / inner4) % features;
            sd[u] = sqrtf(var[f] + eps); m[u] = mean[f]; ga[u] = gamma[f]; be[u] = beta[f];
        }
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < total4) {
            f4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (v[u][e] - m[u]) / sd[u] * ga[u] + be[u];
            __builtin_nontemporal_store(o, y4 + j);
        }
    }
}

}  // namespace

// -------------------------------------------------------------------------------------------------

extern "C" int zant_hip_relu_f32(zant_ctx *ctx, const float *x, float *y, int64_t n) {
    return launch_unary<UN_RELU>(ctx, x, y, n, 0.0f);
}

extern "C" int zant_hip_leaky_relu_f32(zant_ctx *ctx, const float *x, float slope, float *y, int64_t n) {
    return launch_unary<UN_LEAKY>(ctx, x, y, n, slope);
}

extern "C" int zant_hip_sigmoid_f32(zant_ctx *ctx, const float *x, float *y, int64_t n) {
    return launch_unary<UN_SIGMOID>(ctx, x, y, n, 0.0f);
}

extern "C" int zant_hip_softmax_f32(zant_ctx *ctx, const float *x, float *y, int64_t rows, int64_t cols) {
    if (!ctx) return ZANT_NullPointer;
    if (rows < 0 || cols < 0) return ZANT_InvalidDimensions;
    if (rows == 0 || cols == 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    if (cols <= 16)
        // four workgroups (32 KB of LDS each) per compute unit walk the chunks of 256 rows
        hipLaunchKernelGGL(softmax_small_f32_kernel,
                           dim3(unsigned(std::min<int64_t>((rows + kThreads - 1) / kThreads, int64_t(ctx->num_cus) * 4))), dim3(kThreads), 0,
                           ctx->stream, x, y, rows, int(cols),
                           // every workgroup's span starts on a 16-byte boundary when 256 * cols floats do
                           ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0 ? 1 : 0);
    else
        hipLaunchKernelGGL(softmax_f32_kernel, dim3(grid_for(rows, kThreads / 64, ctx->num_cus)), dim3(kThreads), 0,
                           ctx->stream, x, y, rows, cols);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_add_f32(zant_ctx *ctx, const float *a, const int64_t *adim, int a_rank, const float *b,
                                const int64_t *bdim, int b_rank, float *y, int64_t *ydim_out, int *y_rank_out) {
    if (!adim || !bdim) return ZANT_NullPointer;  // ctx is looked at with the data pointers: shape queries pass none
    if (a_rank < 0 || b_rank < 0 || a_rank > 8 || b_rank > 8) return ZANT_InvalidDimensions;
    const int64_t asz = prod_dims(adim, a_rank), bsz = prod_dims(bdim, b_rank);
    if (asz == bsz) {  // lib_elementWise_math.zig:72-110
        if (y_rank_out) *y_rank_out = a_rank;
        if (ydim_out) for (int i = 0; i < a_rank; ++i) ydim_out[i] = adim[i];
        if (asz == 0) return ZANT_OK;
        if (!ctx || !a || !b || !y) return ZANT_NullPointer;
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
    if (!ctx || !a || !b || !y) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    {
        // per-channel fast path: one operand is the whole output, the other varies along exactly one axis
        auto single_axis = [&](const int64_t *sv, int64_t *axis_len, int64_t *inner) {
            int axis = -1;
            for (int i = 0; i < g.rank; ++i)
                if (sv[i] > 1) { if (axis >= 0) return false; axis = i; }
            if (axis < 0) return false;
            *axis_len = sv[axis];
            *inner = 1;
            for (int i = axis + 1; i < g.rank; ++i) *inner *= g.out_dim[i];
            return sv[axis] == g.out_dim[axis];
        };
        int64_t clen = 0, inner = 0;
        const float *big = nullptr, *small = nullptr;
        if (asz == osz && single_axis(s2, &clen, &inner)) { big = a; small = b; }
        else if (bsz == osz && single_axis(s1, &clen, &inner)) { big = b; small = a; }
        if (big && inner % 4 == 0 && osz < (int64_t(1) << 32) &&
            ((reinterpret_cast<uintptr_t>(big) | reinterpret_cast<uintptr_t>(y)) & 15) == 0) {
            hipLaunchKernelGGL(add_channel_f32_kernel, dim3(zant_stream_grid(osz >> 2)), dim3(kThreads), 0, ctx->stream, big, small,
                               y, uint32_t(osz >> 2), uint32_t(inner >> 2), uint32_t(clen));
            ZANT_LAUNCH_CHECK(ctx);
            return ZANT_OK;
        }
    }
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
    if (!xdim || !new_shape || !ydim_out) return ZANT_NullPointer;
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
    if (!ctx || !x || !y) return ZANT_NullPointer;
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

// AveragePool: pool_forward with PoolingType.Avg (op_pooling.zig:223-260, 373-408), plus ONNX AveragePool's pads and
// count_include_pad.
extern "C" int zant_hip_avgpool2d_f32(zant_ctx *ctx, const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4],
                                      const int64_t kernel[2], const int64_t strides[2], const int64_t pads[4],
                                      int count_include_pad) {
    if (!ctx || !xdim || !ydim || !kernel || !strides) return ZANT_NullPointer;
    for (int i = 0; i < 4; ++i)
        if (xdim[i] < 0 || ydim[i] < 0 || xdim[i] > INT32_MAX || ydim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    if (kernel[0] <= 0 || kernel[1] <= 0 || strides[0] <= 0 || strides[1] <= 0) return ZANT_InvalidDimensions;  // :233-236
    if (kernel[0] > INT32_MAX / 4 || kernel[1] > INT32_MAX / 4 || strides[0] > INT32_MAX / 4 || strides[1] > INT32_MAX / 4)
        return ZANT_InvalidDimensions;
    if (ydim[0] != xdim[0] || ydim[1] != xdim[1]) return ZANT_InvalidDimensions;
    AvgGeom g;
    g.pt = g.pl = g.pb = g.pr = 0;
    if (pads) {
        for (int i = 0; i < 4; ++i)
            if (pads[i] < 0 || pads[i] >= (i & 1 ? kernel[1] : kernel[0])) return ZANT_InvalidPadding;
        g.pt = int(pads[0]); g.pl = int(pads[1]); g.pb = int(pads[2]); g.pr = int(pads[3]);
    }
    // every window must start inside the input or its top / left padding
    if (ydim[2] > 0 && (ydim[2] - 1) * strides[0] - g.pt >= xdim[2]) return ZANT_InvalidDimensions;
    if (ydim[3] > 0 && (ydim[3] - 1) * strides[1] - g.pl >= xdim[3]) return ZANT_InvalidDimensions;
    g.NC = xdim[0] * xdim[1];
    g.H = int(xdim[2]); g.W = int(xdim[3]); g.OH = int(ydim[2]); g.OW = int(ydim[3]);
    g.kh = int(kernel[0]); g.kw = int(kernel[1]); g.sh = int(strides[0]); g.sw = int(strides[1]);
    g.include_pad = count_include_pad != 0;
    const int64_t total = g.NC * g.OH * g.OW;
    if (total == 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    const bool fast = g.kh == 2 && g.kw == 2 && g.sh == 2 && g.sw == 2 && !g.pt && !g.pl && 2 * g.OH <= g.H && 2 * g.OW <= g.W &&
                      g.OW % 2 == 0 && g.W % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 8 == 0;
    // small planes, 2x2 / stride 2, no padding: the plane-staged kernel of the max pool
    if (g.kh == 2 && g.kw == 2 && g.sh == 2 && g.sw == 2 && !g.pt && !g.pl && 2 * g.OH <= g.H && 2 * g.OW <= g.W && g.W % 2 == 0 &&
        int64_t(g.H) * g.W * 4 <= kPoolLdsFloats && int64_t(g.OH) * g.OW >= 4 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(y) % 16 == 0) {
        const int G = int(std::min<int64_t>((kPoolLdsFloats / (int64_t(g.H) * g.W)) & ~int64_t(3), 64));
        if (G >= 4 && ceil_div64(g.NC, G) < (int64_t(1) << 31)) {
            KernelTimer kt(ctx);
            ZANT_KERNEL_NAME(ctx, "pool_2x2s2_planes_f32_kernel<true>");
            hipLaunchKernelGGL(pool_2x2s2_planes_f32_kernel<true>, dim3(unsigned(ceil_div64(g.NC, G))), dim3(kThreads), 0, ctx->stream, x, y,
                               g.NC, G, g.H, g.W, g.OH, g.OW, 1.0f / float(g.OH * g.OW), 1.0f / float(g.OW));
            ZANT_LAUNCH_CHECK(ctx);
            return ZANT_OK;
        }
    }
    KernelTimer kt(ctx);
    if (fast) {
        const int64_t total2 = total / 2;
        hipLaunchKernelGGL(avgpool_2x2s2_f32_kernel, dim3(grid_for(total2, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x,
                           y, g, total2);
    } else {
        hipLaunchKernelGGL(avgpool_f32_kernel, dim3(grid_for(total, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x, y, g);
    }
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// Output shape of an average pool: pool_forward's (H - k) / s + 1 (op_pooling.zig:239-240) over the padded input, with
// ONNX AveragePool's ceil_mode (a last window that would start in the bottom / right padding is dropped).  Host only.
extern "C" int zant_hip_avgpool2d_out_shape(const int64_t xdim[4], const int64_t kernel[2], const int64_t strides[2],
                                            const int64_t pads[4], int ceil_mode, int64_t ydim[4]) {
    if (!xdim || !kernel || !strides || !ydim) return ZANT_NullPointer;
    if (kernel[0] <= 0 || kernel[1] <= 0 || strides[0] <= 0 || strides[1] <= 0) return ZANT_InvalidDimensions;
    for (int ax = 0; ax < 2; ++ax) {
        const int64_t lead = pads ? pads[ax] : 0, trail = pads ? pads[2 + ax] : 0;
        const int64_t n = xdim[2 + ax] + lead + trail - kernel[ax];
        if (lead < 0 || trail < 0) return ZANT_InvalidPadding;
        if (n < 0) return ZANT_InvalidDimensions;  // :243-245
        int64_t o = (ceil_mode ? (n + strides[ax] - 1) / strides[ax] : n / strides[ax]) + 1;
        if (ceil_mode && (o - 1) * strides[ax] >= xdim[2 + ax] + lead) --o;
        ydim[2 + ax] = o;
    }
    ydim[0] = xdim[0]; ydim[1] = xdim[1];
    return ZANT_OK;
}

// BatchNormalization, inference form: features on axis 1; gamma / beta / mean / var are device arrays of xdim[1] floats.
extern "C" int zant_hip_batchnorm_f32(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank, const float *gamma,
                                      const float *beta, const float *mean, const float *var, float epsilon, float *y) {
    if (!ctx || !xdim) return ZANT_NullPointer;
    if (rank < 2 || rank > 8) return ZANT_InvalidDimensions;
    int64_t total = 1, inner = 1;
    for (int i = 0; i < rank; ++i) {
        if (xdim[i] < 0) return ZANT_InvalidDimensions;
        total *= xdim[i];
        if (i >= 2) inner *= xdim[i];
    }
    if (total == 0) return ZANT_OK;
    if (xdim[1] > INT32_MAX) return ZANT_InvalidDimensions;
    if (!x || !y || !gamma || !beta || !mean || !var) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    if (inner % 4 == 0 && inner / 4 < (int64_t(1) << 31) && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0) {
        hipLaunchKernelGGL(batchnorm_vec_f32_kernel, dim3(zant_stream_grid(total / 4)), dim3(kThreads), 0, ctx->stream,
                           x, y, gamma, beta, mean, var, epsilon, total / 4, uint32_t(inner / 4), uint32_t(xdim[1]));
    } else {
        hipLaunchKernelGGL(batchnorm_f32_kernel, dim3(grid_for(total, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x, y,
                           gamma, beta, mean, var, epsilon, total, inner, int(xdim[1]));
    }
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
