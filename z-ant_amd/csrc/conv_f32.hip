// f32 convolution (conv_lean / OnnxConvLean, reference op_convolution.zig:42-331).
//
// The reference materialises a zero-padded copy, an im2col matrix, a transposed weight matrix and a
// matmul result.  Here the convolution is one implicit-GEMM kernel:
//   D[k, p] = sum_{c,kh,kw} W[k, c, kh, kw] * X[n(p), c, ih(p,kh), iw(p,kw)]
// computed on the f32 matrix cores (v_mfma_f32_32x32x2_f32).  A workgroup owns a tile of output
// positions (whole output rows of one image, or several whole small images) for up to 64 output
// channels.  Per chunk of 8 input channels it stages the input patch (with its halo, zero filled at
// the borders: no padded copy) and the matching weight slab in LDS, and every tap of the filter is a
// constant LDS offset from a lane's base address: no im2col buffer exists anywhere.
// Output channels are the MFMA rows and output positions the MFMA columns, so each accumulator
// register holds 32 consecutive NCHW positions and stores are 128-byte coalesced.
// A direct kernel (one thread per output element) covers shapes the tiled kernel does not take.
#include "common.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int CC = 8;  // input channels staged per chunk (4 MFMA k-steps per filter tap)

struct TileGeom {
    int NB, TH;          // images per workgroup, output rows per workgroup
    int PH, PW, P1;      // staged patch rows / cols, floats per channel (NB*PH*PW)
    int n_row_tiles;     // ceil(OH / TH)
    int n_chunks;        // ceil(C / CC)
    int n_kblocks;       // ceil(K / K_BLK)
    int n_sblocks;       // spatial workgroups
    int positions;       // NB*TH*OW valid positions per workgroup
};

// Packs OIHW weights into [chunk][kblock][tap][cc][K_BLK] (zero padded) so a chunk's slab is one
// contiguous, 16-byte aligned run whose LDS image has the output channel as the fastest axis.
__global__ void pack_weights_f32_kernel(const float *__restrict__ w, float *__restrict__ wp, int K, int C, int T,
                                        int n_chunks, int n_kblocks, int k_blk) {
    const int64_t total = int64_t(n_chunks) * n_kblocks * T * CC * k_blk;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        int64_t r = i;
        const int kk = int(r % k_blk); r /= k_blk;
        const int cc = int(r % CC); r /= CC;
        const int tap = int(r % T); r /= T;
        const int kb = int(r % n_kblocks); r /= n_kblocks;
        const int chunk = int(r);
        const int k = kb * k_blk + kk, c = chunk * CC + cc;
        wp[i] = (k < K && c < C) ? w[(int64_t(k) * C + c) * T + tap] : 0.0f;
    }
}

// MT: 32-position MFMA tiles per wave; WM x WN waves per workgroup (positions x output channels).
template <int MT, int WM, int WN>
__global__ void __launch_bounds__(WM *WN * 64, 2)
conv_f32_mfma_kernel(const float *__restrict__ x, const float *__restrict__ wp, const float *__restrict__ bias,
                     float *__restrict__ y, ConvGeom g, TileGeom t, int relu) {
    constexpr int NT = WM * WN * 64;
    constexpr int K_BLK = WN * 32;
    extern __shared__ float lds[];
    const int T = g.KH * g.KW;
    float *patch = lds;                 // [CC][P1]
    float *wl = lds + CC * t.P1;        // [T][CC][K_BLK]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;

    // XCD-aware order: consecutive workgroup ids go to different XCDs, so give each XCD a
    // contiguous run of spatial tiles (neighbours share halo rows in that XCD's L2).
    int sb = blockIdx.x;
    if ((t.n_sblocks & 7) == 0) sb = (sb & 7) * (t.n_sblocks >> 3) + (sb >> 3);
    const int kb = blockIdx.y;
    const int ig = sb / t.n_row_tiles, rt = sb - ig * t.n_row_tiles;
    const int n0 = ig * t.NB, oh0 = rt * t.TH;
    const int64_t x_img = int64_t(g.C) * g.H * g.W;
    const float *xb = x + int64_t(n0) * x_img;

    // ---- per-lane constants: LDS base offset and output offset of each of this wave's tiles ----
    int lds_off[MT];
    int64_t out_off[MT];
    const int rows_here = min(t.TH, g.OH - oh0);
    const int imgs_here = min(t.NB, g.N - n0);
    const int per_img = t.TH * g.OW;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int p = (wm * MT + i) * 32 + l32;
        const int img = p / per_img, rem = p - img * per_img;
        const int r = rem / g.OW, c = rem - r * g.OW;
        const bool ok = img < imgs_here && r < rows_here;
        lds_off[i] = ok ? (img * t.PH + r * g.sh) * t.PW + c * g.sw : 0;
        out_off[i] = ok ? (int64_t(n0 + img) * g.K * g.OH + (oh0 + r)) * g.OW + c : -1;
    }

    f32x16 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

    const int ih0 = oh0 * g.sh - g.pt;
    const int patch_hw = t.PH * t.PW;
    const int w_chunk = T * CC * K_BLK;  // floats per (chunk, kblock) slab, a multiple of 4

    for (int chunk = 0; chunk < t.n_chunks; ++chunk) {
        __syncthreads();  // every wave is done reading the previous chunk
        // ---- stage the input patch: [cc][img][ph][pw], zero outside the image ----
        for (int e = tid; e < t.P1; e += NT) {
            const int img = e / patch_hw, rem = e - img * patch_hw;
            const int ph = rem / t.PW, pw = rem - ph * t.PW;
            const int ih = ih0 + ph, iw = pw - g.pl;
            const bool ok = img < imgs_here && ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
            const int64_t goff = int64_t(img) * x_img + int64_t(ih) * g.W + iw;
#pragma unroll
            for (int cc = 0; cc < CC; ++cc) {
                const int c = chunk * CC + cc;
                float v = 0.0f;
                if (ok && c < g.C) v = xb[goff + int64_t(c) * g.H * g.W];
                patch[cc * t.P1 + e] = v;
            }
        }
        // ---- stage the weight slab (already in LDS order) ----
        {
            const float4 *src = reinterpret_cast<const float4 *>(wp + (int64_t(chunk) * t.n_kblocks + kb) * w_chunk);
            float4 *dst = reinterpret_cast<float4 *>(wl);
            for (int e = tid; e < (w_chunk >> 2); e += NT) dst[e] = src[e];
        }
        __syncthreads();
        // ---- MFMA: per tap, 4 k-steps of 2 channels ----
        const float *wa = wl + lh * K_BLK + wn * 32 + l32;
        const float *pb = patch + lh * t.P1;
        for (int kh = 0; kh < g.KH; ++kh) {
            for (int kw = 0; kw < g.KW; ++kw) {
                const int tap_off = kh * g.dh * t.PW + kw * g.dw;
                const float *wt = wa + (kh * g.KW + kw) * CC * K_BLK;
#pragma unroll
                for (int cp = 0; cp < CC / 2; ++cp) {
                    const float a = wt[cp * 2 * K_BLK];
                    const float *pc = pb + cp * 2 * t.P1 + tap_off;
                    float b[MT];
#pragma unroll
                    for (int i = 0; i < MT; ++i) b[i] = pc[lds_off[i]];
#pragma unroll
                    for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b[i], acc[i], 0, 0, 0);
                }
            }
        }
    }

    // ---- epilogue: bias (+ReLU), coalesced NCHW stores ----
    const int64_t plane = int64_t(g.OH) * g.OW;
    float bv[16];
    int kv[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        kv[v] = kb * K_BLK + wn * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
        bv[v] = (bias != nullptr && kv[v] < g.K) ? bias[kv[v]] : 0.0f;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        if (out_off[i] < 0) continue;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            if (kv[v] < g.K) {
                float r = acc[i][v] + bv[v];
                if (relu) r = r > 0.0f ? r : 0.0f;
                y[out_off[i] + int64_t(kv[v]) * plane] = r;
            }
        }
    }
}

// One thread per output element; any stride / dilation / pads / kernel size.
__global__ void __launch_bounds__(256) conv_f32_direct_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                             const float *__restrict__ bias, float *__restrict__ y,
                                                             ConvGeom g, int relu) {
    const int64_t total = int64_t(g.N) * g.K * g.OH * g.OW;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int ow = int(i % g.OW);
        const int oh = int((i / g.OW) % g.OH);
        const int k = int((i / (int64_t(g.OW) * g.OH)) % g.K);
        const int n = int(i / (int64_t(g.OW) * g.OH * g.K));
        float acc = 0.0f;
        for (int c = 0; c < g.C; ++c) {
            const float *xp = x + (int64_t(n) * g.C + c) * g.H * g.W;
            const float *wq = w + (int64_t(k) * g.C + c) * g.KH * g.KW;
            for (int kh = 0; kh < g.KH; ++kh) {
                const int ih = oh * g.sh - g.pt + kh * g.dh;
                if (ih < 0 || ih >= g.H) continue;
                for (int kw = 0; kw < g.KW; ++kw) {
                    const int iw = ow * g.sw - g.pl + kw * g.dw;
                    if (iw < 0 || iw >= g.W) continue;
                    acc = __builtin_fmaf(xp[ih * g.W + iw], wq[kh * g.KW + kw], acc);
                }
            }
        }
        float r = acc + (bias ? bias[k] : 0.0f);
        if (relu) r = r > 0.0f ? r : 0.0f;
        y[i] = r;
    }
}

struct MfmaPlan {
    int MT, WM, WN;
    TileGeom t;
    size_t lds_bytes;
    double eff;
};

// Picks the tile shape with the best useful-lane fraction whose LDS footprint allows two workgroups per CU.
bool plan_mfma(const ConvGeom &g, MfmaPlan *best) {
    static const int kMT[] = {8, 7, 6, 5, 4, 3, 2, 1};
    const size_t lds_cap = 72 * 1024;
    const int T = g.KH * g.KW;
    bool found = false;
    const int WN = g.K > 32 ? 2 : 1, WM = 4 / WN;
    const int K_BLK = WN * 32;
    for (int mt : kMT) {
        const int S = WM * mt * 32;
        const int per_img = g.OH * g.OW;
        TileGeom t;
        if (per_img <= S) {
            t.NB = S / per_img; t.TH = g.OH;
            if (t.NB > g.N) t.NB = g.N;
        } else {
            t.NB = 1; t.TH = S / g.OW;
            if (t.TH < 1) continue;
        }
        t.n_row_tiles = (g.OH + t.TH - 1) / t.TH;
        // even out the rows so the last tile is not nearly empty
        t.TH = (g.OH + t.n_row_tiles - 1) / t.n_row_tiles;
        t.PH = (t.TH - 1) * g.sh + (g.KH - 1) * g.dh + 1;
        t.PW = (g.OW - 1) * g.sw + (g.KW - 1) * g.dw + 1;
        t.P1 = t.NB * t.PH * t.PW;
        t.n_chunks = (g.C + CC - 1) / CC;
        t.n_kblocks = (g.K + K_BLK - 1) / K_BLK;
        t.n_sblocks = ((g.N + t.NB - 1) / t.NB) * t.n_row_tiles;
        t.positions = t.NB * t.TH * g.OW;
        const size_t lds = (size_t(CC) * t.P1 + size_t(T) * CC * K_BLK) * sizeof(float);
        if (lds > lds_cap) continue;
        const double useful = double(g.N) * g.OH * g.OW;
        const double eff = useful / (double(t.n_sblocks) * S);
        if (!found || eff > best->eff + 1e-9) {
            best->MT = mt; best->WM = WM; best->WN = WN; best->t = t; best->lds_bytes = lds; best->eff = eff;
            found = true;
        }
    }
    return found;
}

template <int MT, int WM, int WN>
void launch_mfma(zant_ctx *ctx, const float *x, const float *wp, const float *bias, float *y, const ConvGeom &g,
                 const MfmaPlan &p, int relu) {
    hipLaunchKernelGGL((conv_f32_mfma_kernel<MT, WM, WN>), dim3(p.t.n_sblocks, p.t.n_kblocks), dim3(WM * WN * 64),
                       p.lds_bytes, ctx->stream, x, wp, bias, y, g, p.t, relu);
}

template <int WM, int WN>
bool dispatch_mt(zant_ctx *ctx, const float *x, const float *wp, const float *bias, float *y, const ConvGeom &g,
                 const MfmaPlan &p, int relu) {
    switch (p.MT) {
    case 1: launch_mfma<1, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 2: launch_mfma<2, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 3: launch_mfma<3, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 4: launch_mfma<4, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 5: launch_mfma<5, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 6: launch_mfma<6, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 7: launch_mfma<7, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    case 8: launch_mfma<8, WM, WN>(ctx, x, wp, bias, y, g, p, relu); return true;
    default: return false;
    }
}

}  // namespace

int zant_conv_resolve(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride, int n_stride,
                      const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                      const char *auto_pad, int64_t s[2], int64_t d[2], int64_t p[4]) {
    if (group >= 0 && group != 1) return ZANT_InvalidDimensions;  // op_convolution.zig:60-65
    if (!stride || n_stride < 1) return ZANT_WrongStride;
    s[0] = stride[0];                                              // :68
    s[1] = n_stride > 1 ? stride[1] : stride[0];                   // :69
    d[0] = (dil && n_dil > 0) ? dil[0] : 1;                        // :70
    d[1] = dil ? (n_dil > 1 ? dil[1] : (n_dil > 0 ? dil[0] : 1)) : 1;  // :71
    if (s[0] <= 0 || s[1] <= 0 || d[0] <= 0 || d[1] <= 0) return ZANT_WrongStride;
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1;  // :74-75
    p[0] = p[1] = p[2] = p[3] = 0;  // h_begin, w_begin, h_end, w_end
    if (auto_pad) {
        const bool upper = !strcmp(auto_pad, "SAME_UPPER"), lower = !strcmp(auto_pad, "SAME_LOWER");
        if (upper || lower) {
            const int64_t oh = ceil_div64(xdim[2], s[0]), ow = ceil_div64(xdim[3], s[1]);  // :92-93
            int64_t th = (oh - 1) * s[0] + dkh - xdim[2], tw = (ow - 1) * s[1] + dkw - xdim[3];  // :96-97
            if (th < 0) th = 0;
            if (tw < 0) tw = 0;
            if (upper) { p[0] = th / 2; p[2] = th - p[0]; p[1] = tw / 2; p[3] = tw - p[1]; }  // :101-104
            else { p[2] = th / 2; p[0] = th - p[2]; p[3] = tw / 2; p[1] = tw - p[3]; }         // :106-109
        } else if (!strcmp(auto_pad, "NOTSET")) {
            if (!pads) return ZANT_InvalidPadding;  // :120-125
            if (n_pads >= 4) { p[0] = pads[0]; p[1] = pads[1]; p[2] = pads[2]; p[3] = pads[3]; }  // :114-119
        }
        // "VALID" and unknown strings: no padding (:88-89, :126-128)
    }
    // auto_pad == null: pads are ignored (:86)
    return ZANT_OK;
}

extern "C" int zant_hip_conv2d_out_shape(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride,
                                         int n_stride, const int64_t *pads, int n_pads, const int64_t *dil, int n_dil,
                                         int64_t group, const char *auto_pad, int64_t ydim[4]) {
    // OnnxConv, op_convolution.zig:647-732
    if (!xdim || !wdim || !ydim) return ZANT_NullPointer;
    if (group >= 0 && group != 1) return ZANT_InvalidDimensions;
    if (!stride || n_stride < 1) return ZANT_WrongStride;
    const int64_t sh = stride[0], sw = n_stride > 1 ? stride[1] : stride[0];
    const int64_t dh = (dil && n_dil > 0) ? dil[0] : 1;
    const int64_t dw = dil ? (n_dil > 1 ? dil[1] : (n_dil > 0 ? dil[0] : 1)) : 1;
    if (sh <= 0 || sw <= 0) return ZANT_WrongStride;
    const int64_t dkh = (wdim[2] - 1) * dh + 1, dkw = (wdim[3] - 1) * dw + 1;
    const int64_t H = xdim[2], W = xdim[3];
    int64_t oh, ow;
    if (auto_pad) {
        if (!strcmp(auto_pad, "VALID")) {
            oh = (H - dkh) / sh + 1; ow = (W - dkw) / sw + 1;
        } else if (!strcmp(auto_pad, "SAME_UPPER") || !strcmp(auto_pad, "SAME_LOWER")) {
            oh = ceil_div64(H, sh); ow = ceil_div64(W, sw);
        } else if (!strcmp(auto_pad, "NOTSET")) {
            if (pads) {
                if (n_pads < 4) return ZANT_InvalidPadding;  // :713-715
                oh = (H + pads[0] + pads[2] - dkh) / sh + 1;
                ow = (W + pads[1] + pads[3] - dkw) / sw + 1;
            } else {
                oh = (H - dkh) / sh + 1; ow = (W - dkw) / sw + 1;  // :717-718
            }
        } else {
            return ZANT_InvalidPadding;  // :720-722
        }
    } else {
        const int64_t th = (pads && n_pads >= 4) ? pads[0] + pads[2] : 0;  // :725-728
        const int64_t tw = (pads && n_pads >= 4) ? pads[1] + pads[3] : 0;
        oh = (H + th - dkh) / sh + 1; ow = (W + tw - dkw) / sw + 1;
    }
    ydim[0] = xdim[0]; ydim[1] = wdim[0]; ydim[2] = oh; ydim[3] = ow;
    return ZANT_OK;
}

extern "C" int zant_hip_conv2d_f32(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w,
                                   const int64_t wdim[4], const float *bias, float *y, const int64_t ydim[4],
                                   const int64_t *stride, int n_stride, const int64_t *pads, int n_pads,
                                   const int64_t *dil, int n_dil, int64_t group, const char *auto_pad, int fuse_act) {
    if (!ctx || !xdim || !wdim || !ydim) return ZANT_NullPointer;
    zant_log("OnnxConvLean1");
    int64_t s[2], d[2], p[4];
    int rc = zant_conv_resolve(xdim, wdim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad, s, d, p);
    if (rc) { zant_log(rc == ZANT_InvalidPadding ? "OnnxConvLeanError2" : "OnnxConvLeanError1"); return rc; }
    for (int i = 0; i < 4; ++i)
        if (xdim[i] <= 0 || wdim[i] <= 0 || xdim[i] > INT32_MAX || wdim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    const int64_t PH = xdim[2] + p[0] + p[2], PW = xdim[3] + p[1] + p[3];
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1;
    if (PH < dkh || PW < dkw) return ZANT_InvalidDimensions;               // op_convolution.zig:250, :394
    if (xdim[1] != wdim[1]) return ZANT_InputTensorsWrongShape;            // im2col cols != kernel rows (op_mat_mul.zig:34)
    const int64_t OH = (PH - dkh) / s[0] + 1, OW = (PW - dkw) / s[1] + 1;  // :247-248
    if (ydim[0] != xdim[0] || ydim[1] != wdim[0] || ydim[2] != OH || ydim[3] != OW) return ZANT_InvalidDimensions;  // :212-217
    if (OH > INT32_MAX || OW > INT32_MAX || PH > INT32_MAX || PW > INT32_MAX) return ZANT_InvalidDimensions;
    if (!x || !w || !y) return ZANT_NullPointer;
    if (fuse_act != ZANT_ACT_NONE && fuse_act != ZANT_ACT_RELU) return ZANT_InvalidInput;

    ConvGeom g;
    g.N = int(xdim[0]); g.C = int(xdim[1]); g.H = int(xdim[2]); g.W = int(xdim[3]);
    g.K = int(wdim[0]); g.CG = int(wdim[1]); g.KH = int(wdim[2]); g.KW = int(wdim[3]);
    g.OH = int(OH); g.OW = int(OW);
    g.sh = int(s[0]); g.sw = int(s[1]); g.dh = int(d[0]); g.dw = int(d[1]);
    g.pt = int(p[0]); g.pl = int(p[1]); g.groups = 1;
    const int relu = fuse_act == ZANT_ACT_RELU;
    zant_log("OnnxConvLean2");

    MfmaPlan plan;
    const int64_t macs_per_out = int64_t(g.C) * g.KH * g.KW;
    const bool want_mfma = g.C >= 4 && macs_per_out >= 32 && int64_t(g.N) * g.OH * g.OW >= 64 &&
                           int64_t(g.N) * g.C * g.H * g.W < (int64_t(1) << 40);
    if (want_mfma && plan_mfma(g, &plan) && plan.eff >= 0.5) {
        const int T = g.KH * g.KW, K_BLK = plan.WN * 32;
        const size_t wp_floats = size_t(plan.t.n_chunks) * plan.t.n_kblocks * T * CC * K_BLK;
        void *ws = nullptr;
        rc = zant_workspace(ctx, wp_floats * sizeof(float), &ws);
        if (rc) return rc;
        float *wp = static_cast<float *>(ws);
        const unsigned pb = unsigned(std::min<int64_t>(ceil_div64(int64_t(wp_floats), 256), 1024));
        hipLaunchKernelGGL(pack_weights_f32_kernel, dim3(pb), dim3(256), 0, ctx->stream, w, wp, g.K, g.C, T,
                           plan.t.n_chunks, plan.t.n_kblocks, K_BLK);
        ZANT_LAUNCH_CHECK(ctx);
        bool ok = plan.WN == 2 ? dispatch_mt<2, 2>(ctx, x, wp, bias, y, g, plan, relu)
                               : dispatch_mt<4, 1>(ctx, x, wp, bias, y, g, plan, relu);
        if (ok) {
            ZANT_LAUNCH_CHECK(ctx);
            zant_log("OnnxConvLean4");
            return ZANT_OK;
        }
    }
    const int64_t total = int64_t(g.N) * g.K * g.OH * g.OW;
    int64_t blocks = ceil_div64(total, 256);
    if (blocks > int64_t(ctx->num_cus) * 32) blocks = int64_t(ctx->num_cus) * 32;
    hipLaunchKernelGGL(conv_f32_direct_kernel, dim3(unsigned(blocks)), dim3(256), 0, ctx->stream, x, w, bias, y, g, relu);
    ZANT_LAUNCH_CHECK(ctx);
    zant_log("OnnxConvLean4");
    return ZANT_OK;
}
