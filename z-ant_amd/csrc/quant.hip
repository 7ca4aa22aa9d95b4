// int8 elementwise family: QuantizeLinear, DequantizeLinear, the fused Dequantize -> activation ->
// Quantize, the quantised residual add and the quantised global average pool.  The reference holds no
// quantised operators; these follow the ONNX definitions with ONE fixed f32 sequence so that results
// are bit-identical with the CPU checker: IEEE divide, round-half-to-even, add zero point, saturate.
// All are HBM-bound byte streams: 16 bytes per lane per access on the contiguous axis.
#include "quant_common.h"
#include "quant_layout.h"

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

__device__ __forceinline__ int8_t sat_i8_rne(float v, int8_t zp) {
    float r = __builtin_rintf(v) + float(zp);
    r = __builtin_fmaxf(r, -128.0f);  // NaN -> -128
    r = __builtin_fminf(r, 127.0f);
    return int8_t(r);
}
__device__ __forceinline__ uint8_t sat_q(float v, uint8_t zp) { return sat_u8_rne(v, zp); }
__device__ __forceinline__ int8_t sat_q(float v, int8_t zp) { return sat_i8_rne(v, zp); }

// Any axis layout, u8 or i8 codes.
template <typename Q>
__global__ void __launch_bounds__(kThreads) quantize_kernel(const float *__restrict__ x, const float *__restrict__ scale,
                                                           const Q *__restrict__ zp, Q *__restrict__ y, AxisGeom g) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < g.n; i += step) {
        const int64_t c = g.per_axis ? (i / g.inner) % g.alen : 0;
        y[i] = sat_q(x[i] / scale[c], zp ? zp[c] : Q(0));
    }
}

// Per-tensor scale, 16-byte aligned x: one float4 in, four bytes out per vector (both coalesced across the lanes).
__global__ void __launch_bounds__(kThreads) quantize_vec_kernel(const float *__restrict__ x, const float *__restrict__ scale,
                                                               const uint8_t *__restrict__ zp, uint8_t *__restrict__ y,
                                                               int64_t n) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const float s = scale[0];
    const uint8_t z = zp ? zp[0] : uint8_t(0);
    const int64_t n4 = n >> 2;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const f4 *x4 = reinterpret_cast<const f4 *>(x);
    uint32_t *y4 = reinterpret_cast<uint32_t *>(y);
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
            const uint32_t r = uint32_t(sat_u8_rne(v[u].x / s, z)) | (uint32_t(sat_u8_rne(v[u].y / s, z)) << 8) |
                               (uint32_t(sat_u8_rne(v[u].z / s, z)) << 16) | (uint32_t(sat_u8_rne(v[u].w / s, z)) << 24);
            __builtin_nontemporal_store(r, y4 + j);
        }
    }
    if (blockIdx.x == 0) {
        const int64_t j = (n4 << 2) + threadIdx.x;
        if (j < n) y[j] = sat_u8_rne(x[j] / s, z);
    }
}

__global__ void __launch_bounds__(kThreads) dequantize_vec_kernel(const uint8_t *__restrict__ x, const float *__restrict__ scale,
                                                                 const uint8_t *__restrict__ zp, float *__restrict__ y,
                                                                 int64_t n) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const float s = scale[0];
    const int z = zp ? int(zp[0]) : 0;
    const int64_t n4 = n >> 2;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const uint32_t *x4 = reinterpret_cast<const uint32_t *>(x);
    f4 *y4 = reinterpret_cast<f4 *>(y);
    uint32_t v[ZANT_STREAM_U];
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
            r.x = float(int(v[u] & 255) - z) * s;
            r.y = float(int((v[u] >> 8) & 255) - z) * s;
            r.z = float(int((v[u] >> 16) & 255) - z) * s;
            r.w = float(int(v[u] >> 24) - z) * s;
            __builtin_nontemporal_store(r, y4 + j);
        }
    }
    if (blockIdx.x == 0) {
        const int64_t j = (n4 << 2) + threadIdx.x;
        if (j < n) y[j] = float(int(x[j]) - z) * s;
    }
}

// Any axis layout; u8, i8 or i32 codes (the difference is taken in 64 bits: an i32 pair can differ by 2^32).
template <typename Q>
__global__ void __launch_bounds__(kThreads) dequantize_kernel(const Q *__restrict__ x, const float *__restrict__ scale,
                                                             const Q *__restrict__ zp, float *__restrict__ y, AxisGeom g) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < g.n; i += step) {
        const int64_t c = g.per_axis ? (i / g.inner) % g.alen : 0;
        y[i] = float(int64_t(x[i]) - int64_t(zp ? zp[c] : Q(0))) * scale[c];
    }
}

// u8 -> u8 through a 256-entry table held in LDS (the function of one byte is evaluated 256 times
// with the exact f32 sequence, then applied 16 bytes per lane).
// flip: the bytes of x and y hold value ^ flip (0x80 for the blocked signed layout), folded into the table.
__global__ void __launch_bounds__(kThreads) qlinear_act_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ y,
                                                              int64_t n, QAct qa, int vec, int flip) {
    __shared__ uint8_t lut[256];
    lut[threadIdx.x] = uint8_t(qact_apply(uint8_t(threadIdx.x ^ flip), qa) ^ flip);
    __syncthreads();
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    if (!vec) {
        const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U * 16) + threadIdx.x;
        for (int u = 0; u < ZANT_STREAM_U * 16; ++u) {
            const int64_t j = base + u * kThreads;
            if (j < n) y[j] = lut[x[j]];
        }
        return;
    }
    const int64_t n16 = n >> 4;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const u4 *x16 = reinterpret_cast<const u4 *>(x);
    u4 *y16 = reinterpret_cast<u4 *>(y);
    u4 v[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n16) v[u] = __builtin_nontemporal_load(x16 + j);
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n16) {
            u4 r;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t w = v[u][k];
                r[k] = uint32_t(lut[w & 255]) | (uint32_t(lut[(w >> 8) & 255]) << 8) | (uint32_t(lut[(w >> 16) & 255]) << 16) |
                       (uint32_t(lut[w >> 24]) << 24);
            }
            __builtin_nontemporal_store(r, y16 + j);
        }
    }
    if (blockIdx.x == 0) {
        const int64_t j = (n16 << 4) + threadIdx.x;
        if (j < n) y[j] = lut[x[j]];
    }
}

struct QAddArgs {
    float a_scale, b_scale, y_scale;
    int a_zp, b_zp;
    uint8_t y_zp;
    int fast_div;   // the unscaled division sequence applies (see div_by)
    float y_rcp;    // refined reciprocal of y_scale for it
};

__device__ __forceinline__ uint8_t qadd_one(uint8_t a, uint8_t b, const QAddArgs &q) {
    const float fa = float(int(a) - q.a_zp) * q.a_scale;
    const float fb = float(int(b) - q.b_zp) * q.b_scale;
    return sat_u8_rne((fa + fb) / q.y_scale, q.y_zp);
}

__global__ void __launch_bounds__(kThreads) qlinear_add_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                              uint8_t *__restrict__ y, int64_t n, QAddArgs q, int vec,
                                                              uint32_t flip4) {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const uint8_t f = uint8_t(flip4);
    if (!vec) {
        const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U * 16) + threadIdx.x;
        for (int u = 0; u < ZANT_STREAM_U * 16; ++u) {
            const int64_t j = base + u * kThreads;
            if (j < n) y[j] = uint8_t(qadd_one(a[j] ^ f, b[j] ^ f, q) ^ f);
        }
        return;
    }
    // Every byte is dequantised with arithmetic (byte -> float conversion, subtract, multiply: the conversion picks its
    // byte out of the dword itself).  Two 256-entry float tables in LDS, which cost one vector instruction less per
    // byte, made the kernel LDS-bound: random table indices of a wave collide in the banks (the LDS pipe was busy 75 % of
    // the kernel's time, two thirds of that in bank conflicts).
    const float za = float(q.a_zp), zb = float(q.b_zp);
    const int64_t n16 = n >> 4;
    const int64_t base = int64_t(blockIdx.x) * (kThreads * ZANT_STREAM_U) + threadIdx.x;
    const u4 *a16 = reinterpret_cast<const u4 *>(a);
    const u4 *b16 = reinterpret_cast<const u4 *>(b);
    u4 *y16 = reinterpret_cast<u4 *>(y);
    u4 va[ZANT_STREAM_U], vb[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const int64_t j = base + u * kThreads;
        if (j < n16) { va[u] = __builtin_nontemporal_load(a16 + j); vb[u] = __builtin_nontemporal_load(b16 + j); }
    }
    const float zpf = float(q.y_zp);
    // The choice of division sequence is made once, outside the element loops: taken per element it split the sixteen
    // bytes of a vector into sixteen basic blocks, whose dependent chains then ran one after another instead of
    // interleaved.
    auto requantise = [&](auto fast_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
#pragma unroll
        for (int u = 0; u < ZANT_STREAM_U; ++u) {
            const int64_t j = base + u * kThreads;
            if (j < n16) {
                u4 r;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t wa = va[u][w] ^ flip4, wb = vb[u][w] ^ flip4;
                    uint32_t o = 0;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float ca = float((wa >> (8 * k)) & 0xffu), cb = float((wb >> (8 * k)) & 0xffu);  // v_cvt_f32_ubyte<k>
                        // (the integer difference byte - zero point, exact as a float difference, times the scale)
                        const float sum = (ca - za) * q.a_scale + (cb - zb) * q.b_scale;
                        if (FAST)  // finite: the saturating conversion clamps and packs
                            o = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(div_by(sum, q.y_scale, q.y_rcp, 1)) + zpf, unsigned(k), o);
                        else
                            o |= uint32_t(sat_u8_rne(sum / q.y_scale, q.y_zp)) << (8 * k);
                    }
                    r[w] = o ^ flip4;
                }
                __builtin_nontemporal_store(r, y16 + j);
            }
        }
    };
    if (q.fast_div) requantise(std::true_type());
    else requantise(std::false_type());
    if (blockIdx.x == 0) {
        const int64_t j = (n16 << 4) + threadIdx.x;
        if (j < n) y[j] = uint8_t(qadd_one(a[j] ^ f, b[j] ^ f, q) ^ f);
    }
}

// [N][CB][HW][16] signed -> NCHW u8.  One thread per (n, cb, 4 positions): four 16-byte loads, byte transpose,
// sixteen 4-byte stores (one per channel row).
__global__ void __launch_bounds__(kThreads) from_blocked_kernel(const uint4 *__restrict__ xb, uint8_t *__restrict__ y, int N,
                                                               int C, int CB, int64_t HW, int vec_ok) {
    const int64_t HW4 = (HW + 3) >> 2;
    const int64_t total = int64_t(N) * CB * HW4;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int64_t hw = (i % HW4) << 2;
        const int cb = int((i / HW4) % CB);
        const int64_t n = i / (HW4 * CB);
        const int valid = int(min(int64_t(4), HW - hw));
        const uint4 *src = xb + (n * CB + cb) * HW + hw;
        uint32_t u[4][4];  // [position][dword of 4 channels]
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint4 v = b < valid ? src[b] : make_uint4(0, 0, 0, 0);
            u[b][0] = v.x ^ 0x80808080u; u[b][1] = v.y ^ 0x80808080u; u[b][2] = v.z ^ 0x80808080u; u[b][3] = v.w ^ 0x80808080u;
        }
        uint8_t *dst = y + (n * C + int64_t(cb) * 16) * HW + hw;
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            if (cb * 16 + c < C) {
                const int q = c >> 2, sh = 8 * (c & 3);
                const uint32_t row = ((u[0][q] >> sh) & 0xff) | (((u[1][q] >> sh) & 0xff) << 8) |
                                     (((u[2][q] >> sh) & 0xff) << 16) | (((u[3][q] >> sh) & 0xff) << 24);
                uint8_t *p = dst + int64_t(c) * HW;
                if (vec_ok && valid == 4) {
                    *reinterpret_cast<uint32_t *>(p) = row;
                } else {
                    for (int b = 0; b < valid; ++b) p[b] = uint8_t(row >> (8 * b));
                }
            }
        }
    }
}

// Signed byte-wise max of two dwords (the blocked layout stores value - 128, so signed order = value order).
__device__ __forceinline__ uint32_t max_s8x4(uint32_t a, uint32_t b) {
    uint32_t r = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int x = int8_t(a >> (8 * k)), y = int8_t(b >> (8 * k));
        r |= uint32_t(uint8_t(x > y ? x : y)) << (8 * k);
    }
    return r;
}
__device__ __forceinline__ uint4 max_s8x16(uint4 a, uint4 b) {
    return make_uint4(max_s8x4(a.x, b.x), max_s8x4(a.y, b.y), max_s8x4(a.z, b.z), max_s8x4(a.w, b.w));
}

// 2x2 / stride 2 max pool on [planes][H][W] 16-byte units: one thread per output unit.
__global__ void __launch_bounds__(kThreads) maxpool2x2_blocked_kernel(const uint4 *__restrict__ x, uint4 *__restrict__ y,
                                                                     int64_t planes, int H, int W, int OH, int OW) {
    const int64_t total = planes * OH * OW;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int ow = int(i % OW);
        const int oh = int((i / OW) % OH);
        const int64_t p = i / (int64_t(OW) * OH);
        const uint4 *r0 = x + (p * H + 2 * oh) * W + 2 * ow;
        y[i] = max_s8x16(max_s8x16(r0[0], r0[1]), max_s8x16(r0[W], r0[W + 1]));
    }
}

// Global average pool of a blocked tensor: one thread per (n, cb, 4-channel dword); exact i32 sums, then the fixed
// f32 sequence.  Writes NCHW u8 ([N][C]) or the blocked form ([N][CB][16], value ^ 0x80).
__global__ void __launch_bounds__(kThreads) qgap_blocked_kernel(const uint32_t *__restrict__ x, uint8_t *__restrict__ y,
                                                               int64_t planes, int C, int CB, int hw, float x_scale,
                                                               int x_zp, float y_scale, uint8_t y_zp, int y_blocked) {
    const int64_t total = planes * 4;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int64_t p = i >> 2;
        const int q = int(i & 3);
        const uint32_t *src = x + p * int64_t(hw) * 4 + q;
        // Eight positions at a time, their loads issued together (one load per loop turn put a memory round trip on
        // every position: a 3 x 3 map cost nine of them in a row).  Bytes 0 and 2 of a dword are summed in the two
        // 16-bit halves of one register, bytes 1 and 3 in another: 8 x 255 fits 16 bits.  (A thread per 16 channels
        // with 16-byte loads was slower on the 3 x 3 maps of MobileNetV2's head: a quarter of the threads.)
        int s[4] = {0, 0, 0, 0};
        for (int j0 = 0; j0 < hw; j0 += 8) {
            uint32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[int64_t(min(j0 + u, hw - 1)) * 4];
            uint32_t even = 0, odd = 0;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t b = j0 + u < hw ? v[u] ^ 0x80808080u : 0u;
                even += b & 0x00ff00ffu;
                odd += (b >> 8) & 0x00ff00ffu;
            }
            s[0] += int(even & 0xffffu); s[2] += int(even >> 16);
            s[1] += int(odd & 0xffffu); s[3] += int(odd >> 16);
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) s[k] -= hw * x_zp;
        uint32_t out = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const float mean = (float(s[k]) * x_scale) / float(hw);
            out |= uint32_t(sat_u8_rne(mean / y_scale, y_zp)) << (8 * k);
        }
        if (y_blocked) {
            reinterpret_cast<uint32_t *>(y)[i] = out ^ 0x80808080u;
        } else {
            const int64_t n = p / CB;
            const int c0 = int(p % CB) * 16 + q * 4;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (c0 + k < C) y[n * C + c0 + k] = uint8_t(out >> (8 * k));
        }
    }
}

// One wavefront per (n, c) plane: exact i32 sum, then the fixed f32 sequence.
__global__ void __launch_bounds__(kThreads) qgap_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ y, int64_t planes,
                                                       int hw, float x_scale, int x_zp, float y_scale, uint8_t y_zp, int vec) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t(blockIdx.x) * blockDim.x + threadIdx.x) >> 6;
    const int64_t nwaves = (int64_t(gridDim.x) * blockDim.x) >> 6;
    for (int64_t p = wave; p < planes; p += nwaves) {
        const uint8_t *src = x + p * hw;
        int s = 0;
        if (vec) {  // planes of whole 16-byte vectors: v_sad_u8 adds the four bytes of a dword in one instruction
            typedef unsigned u4 __attribute__((ext_vector_type(4)));
            const u4 *src16 = reinterpret_cast<const u4 *>(src);
            unsigned su = 0;
            for (int j = lane; j < (hw >> 4); j += 64) {
                const u4 v = __builtin_nontemporal_load(src16 + j);
                su = __builtin_amdgcn_sad_u8(v[0], 0u, su);
                su = __builtin_amdgcn_sad_u8(v[1], 0u, su);
                su = __builtin_amdgcn_sad_u8(v[2], 0u, su);
                su = __builtin_amdgcn_sad_u8(v[3], 0u, su);
            }
            s = int(su) - (lane == 0 ? hw * x_zp : 0);
        } else {
            for (int j = lane; j < hw; j += 64) s += int(src[j]) - x_zp;
        }
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
    if (!g.per_axis && ((reinterpret_cast<uintptr_t>(x) & 15) | (reinterpret_cast<uintptr_t>(y) & 3)) == 0)
        hipLaunchKernelGGL(quantize_vec_kernel, dim3(zant_stream_grid((g.n + 3) >> 2)), dim3(kThreads), 0, ctx->stream, x, y_scale,
                           y_zp, y, g.n);
    else
        hipLaunchKernelGGL(quantize_kernel<uint8_t>, dim3(grid_for(g.n, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                           x, y_scale, y_zp, y, g);
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
    if (!g.per_axis && ((reinterpret_cast<uintptr_t>(y) & 15) | (reinterpret_cast<uintptr_t>(x) & 3)) == 0)
        hipLaunchKernelGGL(dequantize_vec_kernel, dim3(zant_stream_grid((g.n + 3) >> 2)), dim3(kThreads), 0, ctx->stream, x,
                           x_scale, x_zp, y, g.n);
    else
        hipLaunchKernelGGL(dequantize_kernel<uint8_t>, dim3(grid_for(g.n, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                           x, x_scale, x_zp, y, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

namespace {

template <typename Q>
int launch_quantize(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank, const float *y_scale, const Q *y_zp,
                    int64_t n_scale, int axis, Q *y) {
    if (!ctx) return ZANT_NullPointer;
    AxisGeom g;
    int rc = axis_geom(xdim, rank, n_scale, axis, &g);
    if (rc) return rc;
    if (g.n == 0) return ZANT_OK;
    if (!x || !y || !y_scale) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(quantize_kernel<Q>, dim3(grid_for(g.n, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x, y_scale,
                       y_zp, y, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

template <typename Q>
int launch_dequantize(zant_ctx *ctx, const Q *x, const int64_t *xdim, int rank, const float *x_scale, const Q *x_zp,
                      int64_t n_scale, int axis, float *y) {
    if (!ctx) return ZANT_NullPointer;
    AxisGeom g;
    int rc = axis_geom(xdim, rank, n_scale, axis, &g);
    if (rc) return rc;
    if (g.n == 0) return ZANT_OK;
    if (!x || !y || !x_scale) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(dequantize_kernel<Q>, dim3(grid_for(g.n, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream, x,
                       x_scale, x_zp, y, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

}  // namespace

extern "C" int zant_hip_quantize_linear_f32_i8(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank,
                                               const float *y_scale, const int8_t *y_zp, int64_t n_scale, int axis, int8_t *y) {
    return launch_quantize<int8_t>(ctx, x, xdim, rank, y_scale, y_zp, n_scale, axis, y);
}

extern "C" int zant_hip_dequantize_linear_i8_f32(zant_ctx *ctx, const int8_t *x, const int64_t *xdim, int rank,
                                                 const float *x_scale, const int8_t *x_zp, int64_t n_scale, int axis, float *y) {
    return launch_dequantize<int8_t>(ctx, x, xdim, rank, x_scale, x_zp, n_scale, axis, y);
}

extern "C" int zant_hip_dequantize_linear_i32_f32(zant_ctx *ctx, const int32_t *x, const int64_t *xdim, int rank,
                                                  const float *x_scale, const int32_t *x_zp, int64_t n_scale, int axis, float *y) {
    return launch_dequantize<int32_t>(ctx, x, xdim, rank, x_scale, x_zp, n_scale, axis, y);
}

int zant_qlinear_act_flip(zant_ctx *ctx, const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act, float alpha,
                          float y_scale, uint8_t y_zp, uint8_t *y, int flip) {
    if (!ctx) return ZANT_NullPointer;
    if (act < ZANT_ACT_NONE || act > ZANT_ACT_RELU6) return ZANT_InvalidInput;
    if (n <= 0) return ZANT_OK;
    if (!x || !y) return ZANT_NullPointer;
    QAct qa;
    qa.act = act; qa.alpha = alpha; qa.in_scale = x_scale; qa.in_zp = x_zp; qa.out_scale = y_scale; qa.out_zp = y_zp;
    const int vec = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qlinear_act_kernel, dim3(zant_stream_grid((n + 15) >> 4)), dim3(kThreads), 0, ctx->stream, x, y, n, qa,
                       vec, flip & 0xff);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_qlinear_act_u8(zant_ctx *ctx, const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act,
                                       float alpha, float y_scale, uint8_t y_zp, uint8_t *y) {
    return zant_qlinear_act_flip(ctx, x, n, x_scale, x_zp, act, alpha, y_scale, y_zp, y, 0);
}

int zant_qlinear_add_flip(zant_ctx *ctx, const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b, float b_scale,
                          uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n, int flip) {
    if (!ctx) return ZANT_NullPointer;
    if (n <= 0) return ZANT_OK;
    if (!a || !b || !y) return ZANT_NullPointer;
    QAddArgs q;
    q.a_scale = a_scale; q.b_scale = b_scale; q.y_scale = y_scale; q.a_zp = a_zp; q.b_zp = b_zp; q.y_zp = y_zp;
    q.fast_div = zant_fast_div_ok(a_scale, b_scale, y_scale) ? 1 : 0;
    q.y_rcp = q.fast_div ? zant_refined_rcp(y_scale) : 0.0f;
    const int vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qlinear_add_kernel, dim3(zant_stream_grid((n + 15) >> 4)), dim3(kThreads), 0, ctx->stream, a, b, y, n, q,
                       vec, uint32_t(flip & 0xff) * 0x01010101u);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_qlinear_add_u8(zant_ctx *ctx, const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b,
                                       float b_scale, uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n) {
    return zant_qlinear_add_flip(ctx, a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp, y, n, 0);
}

int zant_from_blocked(zant_ctx *ctx, const uint8_t *xb, int64_t N, int64_t C, int64_t HW, uint8_t *y) {
    if (!ctx) return ZANT_NullPointer;
    if (N <= 0 || C <= 0 || HW <= 0) return ZANT_OK;
    if (!xb || !y) return ZANT_NullPointer;
    const int64_t CB = (C + 15) / 16, units = N * CB * ((HW + 3) / 4);
    const int vec_ok = (HW % 4 == 0) && (reinterpret_cast<uintptr_t>(y) % 4 == 0);
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(from_blocked_kernel, dim3(grid_for(units, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                       reinterpret_cast<const uint4 *>(xb), y, int(N), int(C), int(CB), HW, vec_ok);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

int zant_maxpool2x2_blocked(zant_ctx *ctx, const uint8_t *xb, const int64_t xdim[4], uint8_t *yb) {
    if (!ctx || !xdim) return ZANT_NullPointer;
    const int64_t planes = xdim[0] * ((xdim[1] + 15) / 16), OH = xdim[2] / 2, OW = xdim[3] / 2;
    if (planes <= 0 || OH <= 0 || OW <= 0) return ZANT_OK;
    if (!xb || !yb) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(maxpool2x2_blocked_kernel, dim3(grid_for(planes * OH * OW, kThreads, ctx->num_cus)), dim3(kThreads), 0,
                       ctx->stream, reinterpret_cast<const uint4 *>(xb), reinterpret_cast<uint4 *>(yb), planes, int(xdim[2]),
                       int(xdim[3]), int(OH), int(OW));
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

int zant_qgap_blocked(zant_ctx *ctx, const uint8_t *xb, const int64_t xdim[4], float x_scale, uint8_t x_zp, float y_scale,
                      uint8_t y_zp, uint8_t *y, int y_layout) {
    if (!ctx || !xdim) return ZANT_NullPointer;
    const int64_t CB = (xdim[1] + 15) / 16, planes = xdim[0] * CB, hw = xdim[2] * xdim[3];
    if (planes < 0 || hw <= 0 || hw > (1 << 23)) return ZANT_InvalidDimensions;
    if (planes == 0) return ZANT_OK;
    if (!xb || !y) return ZANT_NullPointer;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qgap_blocked_kernel, dim3(grid_for(planes * 4, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                       reinterpret_cast<const uint32_t *>(xb), y, planes, int(xdim[1]), int(CB), int(hw), x_scale, int(x_zp),
                       y_scale, y_zp, y_layout == ZANT_LAYOUT_BLOCKED16);
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
                       y, planes, int(hw), x_scale, int(x_zp), y_scale, y_zp,
                       (hw % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) ? 1 : 0);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
