// ReduceMean, Concat and Resize(nearest): the HBM-bound shape / reduction operators around the convolution path
// (lib_reduction_math.zig:30-268, lib_shape_math.zig:22-160, 307-630 in the reference).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "common.h"
#include "zant_hip.h"

namespace {

constexpr int kThreads = 256;

static inline unsigned grid_for(int64_t items, int per_block, int num_cus) {
    int64_t b = ceil_div64(items, per_block);
    const int64_t cap = int64_t(num_cus) * 32;
    if (b > cap) b = cap;
    return unsigned(b < 1 ? 1 : b);
}

// ---- ReduceMean --------------------------------------------------------------------------------
// Adjacent axes of the same kind (kept / reduced) are merged on the host, so at most four groups of each kind remain,
// outermost first.
struct ReduceGeom {
    int nk, nr;
    int64_t ksize[4], kstride[4];  // kept groups
    int64_t rsize[4], rstride[4];  // reduced groups
    int64_t outputs, count;        // number of results, elements per result
};

__device__ __forceinline__ int64_t kept_base(const ReduceGeom &g, int64_t o) {
    int64_t base = 0;
    for (int i = g.nk - 1; i >= 0; --i) {
        const int64_t q = o / g.ksize[i];
        base += (o - q * g.ksize[i]) * g.kstride[i];
        o = q;
    }
    return base;
}

// The innermost group is reduced (unit stride): LANES lanes share one result and walk the contiguous run together.
// `seg` > 1 splits the run of a result into segments (few results, long runs); partial sums go to `part`.
template <int LANES>
__global__ void __launch_bounds__(kThreads) reduce_mean_lanes_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                    ReduceGeom g, int seg, int64_t seg_len, int vec4) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x % LANES;
    const int64_t step = int64_t(gridDim.x) * (kThreads / LANES);
    const int64_t items = g.outputs * seg;
    const int64_t inner = g.rsize[g.nr - 1];
    int64_t outer = 1;
    for (int i = 0; i < g.nr - 1; ++i) outer *= g.rsize[i];
    for (int64_t it = int64_t(blockIdx.x) * (kThreads / LANES) + threadIdx.x / LANES; it < items; it += step) {
        const int64_t o = it / seg;
        const int s = int(it - o * seg);
        const float *row = x + kept_base(g, o);
        const int64_t lo = s * seg_len, hi = lo + seg_len < inner ? lo + seg_len : inner;
        float sum = 0.0f;
        for (int64_t c = 0; c < outer; ++c) {  // outer reduced groups (none in the common trailing-axes case)
            int64_t off = 0, r = c;
            for (int i = g.nr - 2; i >= 0; --i) {
                const int64_t q = r / g.rsize[i];
                off += (r - q * g.rsize[i]) * g.rstride[i];
                r = q;
            }
            const float *p = row + off;
            if (vec4) {  // the host checked: base 16-byte aligned, every run start and length a multiple of 4
                const f4 *p4 = reinterpret_cast<const f4 *>(p);
                float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
                int64_t j = (lo >> 2) + lane;
                const int64_t j_end = hi >> 2;
                for (; j + 3 * LANES < j_end; j += 4 * LANES) {  // four loads in flight per lane
                    const f4 v0 = __builtin_nontemporal_load(p4 + j), v1 = __builtin_nontemporal_load(p4 + j + LANES);
                    const f4 v2 = __builtin_nontemporal_load(p4 + j + 2 * LANES), v3 = __builtin_nontemporal_load(p4 + j + 3 * LANES);
                    a0 += (v0.x + v1.x) + (v2.x + v3.x); a1 += (v0.y + v1.y) + (v2.y + v3.y);
                    a2 += (v0.z + v1.z) + (v2.z + v3.z); a3 += (v0.w + v1.w) + (v2.w + v3.w);
                }
                for (; j < j_end; j += LANES) {
                    const f4 v = __builtin_nontemporal_load(p4 + j);
                    a0 += v.x; a1 += v.y; a2 += v.z; a3 += v.w;
                }
                sum += (a0 + a1) + (a2 + a3);
            } else {
                for (int64_t j = lo + lane; j < hi; j += LANES) sum += p[j];
            }
        }
#pragma unroll
        for (int m = LANES / 2; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
        if (lane == 0) y[it] = seg > 1 ? sum : sum / float(g.count);
    }
}

// Second pass of a segmented reduction: `seg` partial sums per result.
__global__ void __launch_bounds__(kThreads) reduce_mean_finish_kernel(const float *__restrict__ part, float *__restrict__ y,
                                                                     int64_t outputs, int seg, float count) {
    const int64_t o = int64_t(blockIdx.x) * (kThreads / 64) + threadIdx.x / 64;
    if (o >= outputs) return;
    float sum = 0.0f;
    for (int j = threadIdx.x % 64; j < seg; j += 64) sum += part[o * seg + j];
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) sum += __shfl_xor(sum, m, 64);
    if (threadIdx.x % 64 == 0) y[o] = sum / count;
}

// The innermost group is kept: one thread per result, neighbouring threads read neighbouring addresses.
__global__ void __launch_bounds__(kThreads) reduce_mean_threads_kernel(const float *__restrict__ x, float *__restrict__ y,
                                                                      ReduceGeom g) {
    const int64_t step = int64_t(gridDim.x) * kThreads;
    for (int64_t o = int64_t(blockIdx.x) * kThreads + threadIdx.x; o < g.outputs; o += step) {
        const float *row = x + kept_base(g, o);
        float sum = 0.0f;
        for (int64_t c = 0; c < g.count; ++c) {
            int64_t off = 0, r = c;
            for (int i = g.nr - 1; i >= 0; --i) {
                const int64_t q = r / g.rsize[i];
                off += (r - q * g.rsize[i]) * g.rstride[i];
                r = q;
            }
            sum += row[off];
        }
        y[o] = sum / float(g.count);
    }
}

// ---- Concat ------------------------------------------------------------------------------------
// One launch per input: `slices` chunks of `chunk` units each go to pitch-strided places in the output.
template <typename U, typename I>
__global__ void __launch_bounds__(kThreads) concat_copy_kernel(const U *__restrict__ x, U *__restrict__ y, I total, I chunk,
                                                              int64_t pitch, int64_t offset) {
    // streaming pattern: ZANT_STREAM_U x 256 consecutive units per workgroup, all loads before the stores
    const I base = I(blockIdx.x) * I(kThreads * ZANT_STREAM_U) + threadIdx.x;
    U v[ZANT_STREAM_U];
#pragma unroll
    for (int k = 0; k < ZANT_STREAM_U; ++k) {
        const I u = base + I(k * kThreads);
        if (u < total) v[k] = __builtin_nontemporal_load(x + u);
    }
#pragma unroll
    for (int k = 0; k < ZANT_STREAM_U; ++k) {
        const I u = base + I(k * kThreads);
        if (u < total) {
            const I sl = u / chunk, r = u - sl * chunk;
            __builtin_nontemporal_store(v[k], y + (int64_t(sl) * pitch + offset + int64_t(r)));
        }
    }
}

// ---- Resize (nearest) --------------------------------------------------------------------------
struct ResizeGeom {
    int rank;
    int64_t xdim[8], ydim[8], xstride[8];
    int64_t tab_off[8];  // where each axis starts in the offset table
    int64_t tab_total, total;
    int coord_mode;
    FastDiv ydiv[8];  // division by ydim[d] (the vector kernel, whose indices stay below 2^31)
    FastDiv owdiv;    // ... by the number of vectors in an output row
};

// Input offset (index * stride) of every output coordinate of every axis, in the reference's f32 arithmetic
// (lib_shape_math.zig:128-145): scale = out / in; half_pixel (o + 0.5) / scale - 0.5; align_corners o (in-1) / (out-1);
// otherwise o / scale; round half away from zero; clamp.
// Written twice: as 64-bit offsets, and (for inputs of fewer than 2^31 elements) as 32-bit ones behind them.
__global__ void __launch_bounds__(kThreads) resize_table_kernel(int64_t *__restrict__ tab, ResizeGeom g) {
    const int64_t t = int64_t(blockIdx.x) * kThreads + threadIdx.x;
    if (t >= g.tab_total) return;
    int d = 0;
    while (d + 1 < g.rank && t >= g.tab_off[d + 1]) ++d;
    const int64_t o = t - g.tab_off[d];
    const float scale = float(g.ydim[d]) / float(g.xdim[d]);
    float pos;
    if (g.coord_mode == 0) pos = (float(o) + 0.5f) / scale - 0.5f;
    else if (g.coord_mode == 1) pos = float(o) * float(g.xdim[d] - 1) / float(g.ydim[d] - 1);
    else pos = float(o) / scale;
    if (!(pos == pos)) pos = 0.0f;  // 0 / 0 of a one-element axis under align_corners
    int64_t i = int64_t(roundf(pos));
    i = i < 0 ? 0 : i;
    i = i > g.xdim[d] - 1 ? g.xdim[d] - 1 : i;
    tab[t] = i * g.xstride[d];
    reinterpret_cast<int *>(tab + g.tab_total)[t] = int(i * g.xstride[d]);
}

template <typename U>
__global__ void __launch_bounds__(kThreads) resize_gather_kernel(const U *__restrict__ x, U *__restrict__ y,
                                                                const int64_t *__restrict__ tab, ResizeGeom g) {
    const int64_t step = int64_t(gridDim.x) * kThreads;
    for (int64_t o = int64_t(blockIdx.x) * kThreads + threadIdx.x; o < g.total; o += step) {
        int64_t r = o, off = 0;
        if (g.total < (int64_t(1) << 31)) {
            unsigned r32 = unsigned(r);
            for (int d = g.rank - 1; d >= 0; --d) {
                const unsigned n = unsigned(g.ydim[d]), q = r32 / n;
                off += tab[g.tab_off[d] + (r32 - q * n)];
                r32 = q;
            }
        } else {
            for (int d = g.rank - 1; d >= 0; --d) {
                const int64_t q = r / g.ydim[d];
                off += tab[g.tab_off[d] + (r - q * g.ydim[d])];
                r = q;
            }
        }
        y[o] = x[off];
    }
}

// VEC consecutive outputs of the innermost axis per thread (one 16-byte store); the outer axes are decoded once per thread.
// Streaming pattern: a workgroup takes ZANT_STREAM_U x 256 consecutive output vectors and issues all its gathers before its
// stores.  Stores are what this kernel is built around: whole, aligned, consecutive vectors (a variant that loaded whole
// input vectors and wrote each to its repeated places was twice as slow on rows that are not multiples of a cache line).
// What then bounds it is the address unit of the vector memory path, which takes every lane of every load whatever the
// lanes point at: so the tables of the innermost `lds_axes` axes (kResizeLdsEntries entries at most, 32-bit) are first
// copied to LDS and looked up there, and only the VEC gathers and the outer axes' 32-bit lookups go through it.
constexpr int kResizeLdsEntries = 2048;
template <typename U, int VEC>
__global__ void __launch_bounds__(kThreads) resize_gather_vec_kernel(const U *__restrict__ x, U *__restrict__ y,
                                                                    const int *__restrict__ tab, ResizeGeom g,
                                                                    unsigned nvec, unsigned ow_vec, int lds_axes, unsigned n_chunks) {
    typedef U UV __attribute__((ext_vector_type(VEC)));
    __shared__ __attribute__((aligned(16))) int tab_lds[kResizeLdsEntries];
    const int first = g.rank - lds_axes;  // axes first .. rank-1 are looked up in LDS
    const int lds_base = first < g.rank ? int(g.tab_off[first]) : int(g.tab_total);
    for (int c = threadIdx.x; c < int(g.tab_total) - lds_base; c += kThreads) tab_lds[c] = tab[lds_base + c];
    __syncthreads();
    const int *tw = tab + g.tab_off[g.rank - 1];
    const int tw_lds = int(g.tab_off[g.rank - 1]) - lds_base;
    // a workgroup stays for several chunks so that the table copy above is paid once and its waves drift apart
    for (unsigned chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const unsigned base = chunk * unsigned(kThreads * ZANT_STREAM_U) + threadIdx.x;
    UV out[ZANT_STREAM_U];
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const unsigned v = base + unsigned(u * kThreads);
        if (v < nvec) {
            unsigned r = fastdiv(v, g.owdiv);
            const unsigned cv = v - r * ow_vec;
            int off = 0;  // below 2^31: the input has fewer elements than that
            for (int d = g.rank - 2; d >= 0; --d) {
                const unsigned n = unsigned(g.ydim[d]), q = fastdiv(r, g.ydiv[d]);
                const int e = int(g.tab_off[d]) + int(r - q * n);
                off += d >= first ? tab_lds[e - lds_base] : tab[e];
                r = q;
            }
            const U *row = x + off;
            if (lds_axes > 0) {
                int col[VEC];
#pragma unroll
                for (int k = 0; k < VEC; ++k) col[k] = tab_lds[tw_lds + int(cv) * VEC + k];
                bool wide = false;
                if constexpr (VEC <= 4) {
                    // up-sampling: the VEC sources lie within VEC consecutive input elements, so one (unaligned) 16-byte
                    // load and a register select replace VEC gathers -- a 4-byte gather at an 8-byte lane stride makes
                    // some thirty cache accesses per wave, a contiguous load four
                    int lo = col[0], hi = col[0];
#pragma unroll
                    for (int k = 1; k < VEC; ++k) { lo = min(lo, col[k]); hi = max(hi, col[k]); }
                    const int row_len = int(g.xdim[g.rank - 1]);
                    if (hi - lo < VEC && row_len >= VEC) {
                        wide = true;
                        const int b0 = min(lo, row_len - VEC);  // keep the window inside the row
                        UV w;
                        __builtin_memcpy(&w, row + b0, sizeof(UV));
#pragma unroll
                        for (int k = 0; k < VEC; ++k) {
                            const int sel = col[k] - b0;
                            U e = w[0];
#pragma unroll
                            for (int j = 1; j < VEC; ++j) e = sel == j ? w[j] : e;
                            out[u][k] = e;
                        }
                    }
                }
                if (!wide) {
#pragma unroll
                    for (int k = 0; k < VEC; ++k) out[u][k] = row[col[k]];
                }
            } else {
#pragma unroll
                for (int k = 0; k < VEC; ++k) out[u][k] = row[tw[cv * VEC + k]];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < ZANT_STREAM_U; ++u) {
        const unsigned v = base + unsigned(u * kThreads);
        if (v < nvec) __builtin_nontemporal_store(out[u], reinterpret_cast<UV *>(y) + v);
    }
    }
}

template <typename U>
int launch_resize(zant_ctx *ctx, const void *x, void *y, const int64_t *tab, ResizeGeom &g) {
    constexpr int VEC = 16 / int(sizeof(U));
    const int64_t ow = g.ydim[g.rank - 1];
    int64_t in_total = 1;
    for (int d = 0; d < g.rank; ++d) in_total *= g.xdim[d];
    KernelTimer kt(ctx);
    if (ow % VEC == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 && g.total / VEC < (int64_t(1) << 31) &&
        in_total < (int64_t(1) << 31) && g.tab_total < (int64_t(1) << 31)) {
        for (int d = 0; d < g.rank; ++d) g.ydiv[d] = make_fastdiv(unsigned(g.ydim[d]));  // ydim[d] <= total / VEC here for d < rank - 1
        g.owdiv = make_fastdiv(unsigned(ow / VEC));
        int lds_axes = 0;  // as many innermost axes as fit
        while (lds_axes < g.rank && g.tab_total - g.tab_off[g.rank - 1 - lds_axes] <= kResizeLdsEntries) ++lds_axes;
        const unsigned n_chunks = zant_stream_grid(g.total / VEC);
        hipLaunchKernelGGL((resize_gather_vec_kernel<U, VEC>), dim3(std::min(n_chunks, unsigned(ctx->num_cus) * 8u)), dim3(kThreads), 0,
                           ctx->stream, static_cast<const U *>(x), static_cast<U *>(y), reinterpret_cast<const int *>(tab + g.tab_total),
                           g, unsigned(g.total / VEC), unsigned(ow / VEC), lds_axes, n_chunks);
    } else
        hipLaunchKernelGGL(resize_gather_kernel<U>, dim3(grid_for(g.total, kThreads, ctx->num_cus)), dim3(kThreads), 0, ctx->stream,
                           static_cast<const U *>(x), static_cast<U *>(y), tab, g);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

template <typename U>
int launch_concat(zant_ctx *ctx, const void *x, void *y, int64_t slices, int64_t chunk, int64_t pitch, int64_t offset) {
    const int64_t total = slices * chunk;
    if (total < (int64_t(1) << 31))
        hipLaunchKernelGGL((concat_copy_kernel<U, unsigned>), dim3(zant_stream_grid(total)), dim3(kThreads), 0,
                           ctx->stream, static_cast<const U *>(x), static_cast<U *>(y), unsigned(total), unsigned(chunk), pitch,
                           offset);
    else
        hipLaunchKernelGGL((concat_copy_kernel<U, int64_t>), dim3(zant_stream_grid(total)), dim3(kThreads), 0,
                           ctx->stream, static_cast<const U *>(x), static_cast<U *>(y), total, chunk, pitch, offset);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

typedef unsigned u4 __attribute__((ext_vector_type(4)));

}  // namespace

// -------------------------------------------------------------------------------------------------

extern "C" int zant_hip_reduce_mean_f32(zant_ctx *ctx, const float *x, const int64_t *xdim, int rank, const int64_t *axes,
                                        int n_axes, int keepdims, int noop_with_empty_axes, float *y, int64_t *ydim_out,
                                        int *y_rank_out) {
    if (!xdim || !ydim_out || !y_rank_out) return ZANT_NullPointer;
    if (rank < 0 || rank > 8) return ZANT_InvalidDimensions;
    for (int i = 0; i < rank; ++i)
        if (xdim[i] < 0) return ZANT_InvalidDimensions;
    const int64_t size = prod_dims(xdim, rank);
    bool reduced[8] = {false, false, false, false, false, false, false, false};
    if (!axes || n_axes == 0) {  // lib_reduction_math.zig:35-46, 111-128
        if (noop_with_empty_axes) {
            for (int i = 0; i < rank; ++i) ydim_out[i] = xdim[i];
            *y_rank_out = rank;
            if (!y || size == 0) return ZANT_OK;
            if (!ctx || !x) return ZANT_NullPointer;
            if (y != x) ZANT_HIP_TRY(ctx, hipMemcpyAsync(y, x, size_t(size) * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream));
            return ZANT_OK;
        }
        if (keepdims) {
            for (int i = 0; i < rank; ++i) ydim_out[i] = 1;
            *y_rank_out = rank;
        } else {
            ydim_out[0] = 1;
            *y_rank_out = 1;
        }
        for (int i = 0; i < rank; ++i) reduced[i] = true;
    } else {
        if (n_axes > 8) return ZANT_InvalidAxes;
        for (int i = 0; i < n_axes; ++i) {  // :131-141; a repeated axis is rejected (the reference would read out of bounds)
            const int64_t a = axes[i] < 0 ? axes[i] + rank : axes[i];
            if (a < 0 || a >= rank || reduced[a]) return ZANT_InvalidAxes;
            reduced[a] = true;
        }
        int out_rank = 0;
        for (int i = 0; i < rank; ++i)  // :62-76
            if (!reduced[i] || keepdims) ydim_out[out_rank++] = reduced[i] ? 1 : xdim[i];
        *y_rank_out = out_rank;
    }
    if (!y) return ZANT_OK;
    if (!ctx || !x) return ZANT_NullPointer;
    if (size == 0) return ZANT_ZeroSizeTensor;

    // merge neighbouring axes of one kind; axes of extent 1 join whatever is next to them
    ReduceGeom g = {};
    g.outputs = 1;
    g.count = 1;
    int64_t stride[8], st = 1;
    for (int i = rank - 1; i >= 0; --i) { stride[i] = st; st *= xdim[i]; }
    int last_kind = -1;  // 0 kept, 1 reduced
    for (int i = 0; i < rank; ++i) {
        if (xdim[i] == 1) continue;
        const int kind = reduced[i] ? 1 : 0;
        if (kind == last_kind) {
            if (kind) { g.rsize[g.nr - 1] *= xdim[i]; g.rstride[g.nr - 1] = stride[i]; }
            else { g.ksize[g.nk - 1] *= xdim[i]; g.kstride[g.nk - 1] = stride[i]; }
        } else if (kind) {
            g.rsize[g.nr] = xdim[i]; g.rstride[g.nr++] = stride[i];
        } else {
            g.ksize[g.nk] = xdim[i]; g.kstride[g.nk++] = stride[i];
        }
        last_kind = kind;
        if (kind) g.count *= xdim[i]; else g.outputs *= xdim[i];
    }
    if (g.nr == 0) {  // only axes of extent 1 were reduced: a copy
        if (y != x) ZANT_HIP_TRY(ctx, hipMemcpyAsync(y, x, size_t(size) * sizeof(float), hipMemcpyDeviceToDevice, ctx->stream));
        return ZANT_OK;
    }
    if (last_kind == 0) {
        KernelTimer kt(ctx);
        hipLaunchKernelGGL(reduce_mean_threads_kernel, dim3(grid_for(g.outputs, kThreads, ctx->num_cus)), dim3(kThreads), 0,
                           ctx->stream, x, y, g);
        ZANT_LAUNCH_CHECK(ctx);
        return ZANT_OK;
    }
    const int64_t inner = g.rsize[g.nr - 1];
    // few results with long runs: cut each run into segments so the whole chip reads, then add the partial sums
    int seg = 1;
    int64_t seg_len = inner;
    if (g.nr == 1 && g.outputs < int64_t(ctx->num_cus) * 16 && inner >= (1 << 16)) {
        int64_t want = ceil_div64(int64_t(ctx->num_cus) * 32, g.outputs);
        const int64_t most = inner >> 14;  // at least 16 Ki elements per segment
        if (want > most) want = most;
        if (want > 4096) want = 4096;
        if (want > 1) {
            seg_len = ceil_div64(ceil_div64(inner, want), 4) * 4;
            seg = int(ceil_div64(inner, seg_len));
        }
    }
    bool vec4 = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && inner % 4 == 0 && inner >= 256;
    for (int i = 0; i < g.nk && vec4; ++i) vec4 = g.kstride[i] % 4 == 0;
    for (int i = 0; i + 1 < g.nr && vec4; ++i) vec4 = g.rstride[i] % 4 == 0;
    float *dst = y;
    if (seg > 1) {
        void *ws = nullptr;
        const int rc = zant_workspace(ctx, size_t(g.outputs) * seg * sizeof(float), &ws);
        if (rc != ZANT_OK) return rc;
        dst = static_cast<float *>(ws);
    }
    const int64_t items = g.outputs * seg;
    const int64_t per_lane_run = vec4 ? inner / 4 : inner;
    {
        KernelTimer kt(ctx);
        if (per_lane_run >= 64)
            hipLaunchKernelGGL(reduce_mean_lanes_kernel<64>, dim3(grid_for(items, kThreads / 64, ctx->num_cus)), dim3(kThreads), 0,
                               ctx->stream, x, dst, g, seg, seg_len, vec4 ? 1 : 0);
        else if (per_lane_run >= 16)
            hipLaunchKernelGGL(reduce_mean_lanes_kernel<16>, dim3(grid_for(items, kThreads / 16, ctx->num_cus)), dim3(kThreads), 0,
                               ctx->stream, x, dst, g, seg, seg_len, vec4 ? 1 : 0);
        else
            hipLaunchKernelGGL(reduce_mean_lanes_kernel<4>, dim3(grid_for(items, kThreads / 4, ctx->num_cus)), dim3(kThreads), 0,
                               ctx->stream, x, dst, g, seg, seg_len, vec4 ? 1 : 0);
    }
    ZANT_LAUNCH_CHECK(ctx);
    if (seg > 1) {
        hipLaunchKernelGGL(reduce_mean_finish_kernel, dim3(unsigned(ceil_div64(g.outputs, kThreads / 64))), dim3(kThreads), 0,
                           ctx->stream, dst, y, g.outputs, seg, float(g.count));
        ZANT_LAUNCH_CHECK(ctx);
    }
    return ZANT_OK;
}

extern "C" int zant_hip_concatenate(zant_ctx *ctx, const void *const *xs, const int64_t *const *dims, const int *ranks, int n,
                                    int64_t axis, size_t elem_size, void *y, int64_t *ydim_out, int *y_rank_out) {
    if (n <= 0) return ZANT_EmptyTensorList;  // lib_shape_math.zig:308
    if (!dims || !ranks || !ydim_out || !y_rank_out) return ZANT_NullPointer;
    if (n > 16) return ZANT_InvalidDimensions;
    int rank = 0;
    for (int t = 0; t < n; ++t) {
        if (ranks[t] < 0 || ranks[t] > 8 || !dims[t]) return ZANT_InvalidDimensions;
        if (ranks[t] > rank) rank = ranks[t];  // :314-320
    }
    if (axis < 0) axis += rank;  // :363-370
    if (axis < 0 || axis >= rank) return ZANT_AxisOutOfBounds;
    int64_t shp[16][8];
    for (int t = 0; t < n; ++t) {  // lower ranks get leading ones (:335-358)
        const int off = rank - ranks[t];
        for (int d = 0; d < rank; ++d) shp[t][d] = d < off ? 1 : dims[t][d - off];
    }
    int64_t total_cd = 0;
    for (int t = 0; t < n; ++t) {  // :374-380
        for (int d = 0; d < rank; ++d)
            if (d != axis && shp[t][d] != shp[0][d]) return ZANT_MismatchedShape;
        total_cd += shp[t][axis];
    }
    for (int d = 0; d < rank; ++d) ydim_out[d] = d == axis ? total_cd : shp[0][d];
    *y_rank_out = rank;
    if (!y) return ZANT_OK;
    if (!ctx || !xs) return ZANT_NullPointer;
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8) return ZANT_InvalidInput;
    int64_t slices = 1, inner = 1;
    for (int d = 0; d < axis; ++d) slices *= shp[0][d];
    for (int d = int(axis) + 1; d < rank; ++d) inner *= shp[0][d];
    const int64_t pitch_b = total_cd * inner * int64_t(elem_size);
    int64_t off_b = 0;
    KernelTimer kt(ctx);
    for (int t = 0; t < n; ++t) {
        const int64_t chunk_b = shp[t][axis] * inner * int64_t(elem_size);
        if (chunk_b > 0 && slices > 0) {
            if (!xs[t]) return ZANT_NullPointer;
            const uintptr_t a = reinterpret_cast<uintptr_t>(xs[t]) | reinterpret_cast<uintptr_t>(y) | uintptr_t(chunk_b) |
                                uintptr_t(pitch_b) | uintptr_t(off_b);
            int rc;
            if (slices == 1) {  // one contiguous block
                ZANT_HIP_TRY(ctx, hipMemcpyAsync(static_cast<char *>(y) + off_b, xs[t], size_t(chunk_b), hipMemcpyDeviceToDevice,
                                                 ctx->stream));
                rc = ZANT_OK;
            } else if ((a & 15) == 0) rc = launch_concat<u4>(ctx, xs[t], y, slices, chunk_b / 16, pitch_b / 16, off_b / 16);
            else if ((a & 3) == 0) rc = launch_concat<uint32_t>(ctx, xs[t], y, slices, chunk_b / 4, pitch_b / 4, off_b / 4);
            else rc = launch_concat<uint8_t>(ctx, xs[t], y, slices, chunk_b, pitch_b, off_b);
            if (rc != ZANT_OK) return rc;
        }
        off_b += chunk_b;
    }
    return ZANT_OK;
}

extern "C" int zant_hip_resize_nearest(zant_ctx *ctx, const void *x, const int64_t *xdim, int rank, size_t elem_size,
                                       const float *scales, const int64_t *sizes, int n_param, int coord_mode, void *y,
                                       int64_t *ydim_out) {
    if ((!scales && !sizes) || (scales && sizes)) return ZANT_InvalidInput;  // lib_shape_math.zig:23-28
    if (!xdim || !ydim_out) return ZANT_NullPointer;
    if (n_param != rank || rank < 1 || rank > 8) return ZANT_InvalidInput;  // :35-37, 43-45
    ResizeGeom g = {};
    g.rank = rank;
    g.coord_mode = coord_mode;
    g.total = 1;
    for (int i = 0; i < rank; ++i) {
        if (xdim[i] < 0) return ZANT_InvalidDimensions;
        ydim_out[i] = scales ? int64_t(floorf(float(xdim[i]) * scales[i])) : sizes[i];  // :38-40
        if (ydim_out[i] < 0) return ZANT_InvalidInput;
        g.xdim[i] = xdim[i];
        g.ydim[i] = ydim_out[i];
        g.tab_off[i] = g.tab_total;
        g.tab_total += ydim_out[i];
        g.total *= ydim_out[i];
    }
    if (!y) return ZANT_OK;
    if (g.total == 0) return ZANT_OK;
    if (!ctx || !x) return ZANT_NullPointer;
    if (prod_dims(xdim, rank) == 0) return ZANT_ZeroSizeTensor;
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8) return ZANT_InvalidInput;
    int64_t st = 1;
    for (int i = rank - 1; i >= 0; --i) { g.xstride[i] = st; st *= xdim[i]; }
    void *ws = nullptr;
    const int rc = zant_workspace(ctx, size_t(g.tab_total) * (sizeof(int64_t) + sizeof(int)), &ws);
    if (rc != ZANT_OK) return rc;
    int64_t *tab = static_cast<int64_t *>(ws);
    hipLaunchKernelGGL(resize_table_kernel, dim3(unsigned(ceil_div64(g.tab_total, kThreads))), dim3(kThreads), 0, ctx->stream, tab, g);
    ZANT_LAUNCH_CHECK(ctx);
    switch (elem_size) {
    case 1: return launch_resize<uint8_t>(ctx, x, y, tab, g);
    case 2: return launch_resize<uint16_t>(ctx, x, y, tab, g);
    case 4: return launch_resize<uint32_t>(ctx, x, y, tab, g);
    default: return launch_resize<uint64_t>(ctx, x, y, tab, g);
    }
}
