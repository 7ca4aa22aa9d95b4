// QLinearConv: u8 activations x i8 weights -> i32 accumulators -> u8 (ONNX definition; the reference has
// no quantised or grouped convolution).  Accumulation is exact integer arithmetic; the epilogue is the
// single f32 requantisation sequence shared with the CPU checker, optionally followed by the fused
// Dequantize -> activation -> Quantize step.
//
// Dense (group = 1) layers with >= 16 input channels run as an implicit GEMM on the int8 matrix cores
// (v_mfma_i32_32x32x32_i8).  The MFMA wants 16 consecutive input channels per lane, which NCHW does
// not have, so a first pass rewrites the activations once into a channel-blocked signed layout
// [N][C/16][H][W][16] (u8 ^ 0x80 = value - 128); one 16-byte global->LDS copy then moves the 16
// channels of a position, and one 128-bit LDS read is one MFMA operand.  The u8 zero point is folded
// into a per-channel integer correction: sum (x - x_zp) w = sum (x - 128) w + (128 - x_zp) sum w,
// with padding positions holding x_zp so that they contribute exactly 0.  Tiling, the asynchronous
// double-buffered staging and the persistent tile loop are those of the f32 kernel.
#include <algorithm>
#include <type_traits>

#include "conv_tile.h"
#include "quant_common.h"
#include "quant_layout.h"

namespace {

// Requantises one accumulator of output channel k.
__device__ __forceinline__ uint8_t requant(int acc, float m, const QConvArgs &q) {
    uint8_t r = sat_u8_rne(float(acc) * m, q.y_zp);
    if (q.has_act) r = qact_apply(r, q.act);
    return r;
}
// The same with the fused activation taken from a 256-entry byte table (identity without one): the activation is a
// function of one byte, and evaluating its f32 sequence (an IEEE divide among it) per output costs more than the MFMAs.
__device__ __forceinline__ uint8_t requant_lut(int acc, float m, const QConvArgs &q, const uint8_t *lut) {
    return lut[sat_u8_rne_finite(float(acc) * m, float(q.y_zp))];
}

// One thread per output element; any stride / dilation / pads / group.
__global__ void __launch_bounds__(256)
qconv_direct_kernel(const uint8_t *__restrict__ x, const int8_t *__restrict__ w, const float *__restrict__ w_scale,
                    const int8_t *__restrict__ w_zp, const int32_t *__restrict__ bias, uint8_t *__restrict__ y,
                    ConvGeom g, QConvArgs q) {
    const int64_t total = int64_t(g.N) * g.K * g.OH * g.OW;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    const int KG = g.K / g.groups;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int ow = int(i % g.OW);
        const int oh = int((i / g.OW) % g.OH);
        const int k = int((i / (int64_t(g.OW) * g.OH)) % g.K);
        const int n = int(i / (int64_t(g.OW) * g.OH * g.K));
        const int grp = k / KG;
        const int wz = w_zp ? int(w_zp[k]) : 0;
        int acc = bias ? bias[k] : 0;
        for (int c = 0; c < g.CG; ++c) {
            const uint8_t *xp = x + (int64_t(n) * g.C + grp * g.CG + c) * g.H * g.W;
            const int8_t *wq = w + (int64_t(k) * g.CG + c) * g.KH * g.KW;
            for (int kh = 0; kh < g.KH; ++kh) {
                const int ih = oh * g.sh - g.pt + kh * g.dh;
                if (ih < 0 || ih >= g.H) continue;
                for (int kw = 0; kw < g.KW; ++kw) {
                    const int iw = ow * g.sw - g.pl + kw * g.dw;
                    if (iw < 0 || iw >= g.W) continue;  // a pad pixel equals x_zp and contributes 0
                    acc += (int(xp[ih * g.W + iw]) - q.x_zp) * (int(wq[kh * g.KW + kw]) - wz);
                }
            }
        }
        const float m = (q.x_scale * w_scale[q.n_wscale == 1 ? 0 : k]) / q.y_scale;
        y[i] = requant(acc, m, q);
    }
}

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

constexpr int QCC = 32;  // input channels per chunk = one MFMA k-step per filter tap

__device__ __forceinline__ i32x4 as_i32x4_q(const uint4 &v) {
    i32x4 r;
    r[0] = int(v.x); r[1] = int(v.y); r[2] = int(v.z); r[3] = int(v.w);
    return r;
}

// NCHW u8 -> [N][CB][H][W][16] signed (value - 128); channels beyond C are 0 (their weights are 0 too).
// Each thread turns 4 consecutive positions x 16 channels: sixteen 4-byte loads (one per channel
// row), a 4x4 byte transpose per group of 4 channels, four 16-byte stores.
__global__ void __launch_bounds__(256) to_blocked_s8_kernel(const uint8_t *__restrict__ x, uint4 *__restrict__ xb, int N,
                                                           int C, int CB, int64_t HW, int vec_ok) {
    const int64_t HW4 = (HW + 3) >> 2;
    const int64_t total = int64_t(N) * CB * HW4;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int64_t hw = (i % HW4) << 2;
        const int cb = int((i / HW4) % CB);
        const int64_t n = i / (HW4 * CB);
        const uint8_t *src = x + (n * C + int64_t(cb) * 16) * HW + hw;
        const int valid = int(min(int64_t(4), HW - hw));
        uint32_t rows[16];  // rows[c] = 4 consecutive positions of channel c
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            uint32_t v = 0;
            if (cb * 16 + c < C) {
                const uint8_t *p = src + int64_t(c) * HW;
                if (vec_ok && valid == 4) {
                    v = *reinterpret_cast<const uint32_t *>(p);
                } else {
                    for (int b = 0; b < valid; ++b) v |= uint32_t(p[b]) << (8 * b);
                }
                v ^= 0x80808080u;
            }
            rows[c] = v;
        }
        uint4 *dst = xb + (n * CB + cb) * HW + hw;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            if (b < valid) {
                uint32_t o[4];
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    o[q] = ((rows[q * 4 + 0] >> (8 * b)) & 0xff) | (((rows[q * 4 + 1] >> (8 * b)) & 0xff) << 8) |
                           (((rows[q * 4 + 2] >> (8 * b)) & 0xff) << 16) | (((rows[q * 4 + 3] >> (8 * b)) & 0xff) << 24);
                dst[b] = make_uint4(o[0], o[1], o[2], o[3]);
            }
        }
    }
}

// The same for planes of whole dwords (HW a multiple of 4, an aligned base) and fewer than 2^31 units.  A workgroup
// turns 64 quads of positions (counted through the whole tensor: rows of (image, channel block) follow each other in
// the output) x 16 channels.  Wavefront g loads the dwords of channels 4g .. 4g+3, a quad per lane (256 contiguous bytes
// per load), transposes its 4 x 4 bytes with byte permutes (dword b: position b, channels 4g .. 4g+3) and writes the
// four dwords to LDS row g; then thread u gathers unit u's four dwords (one per row, consecutive lanes on consecutive
// banks) and stores its 16 bytes: a workgroup's stores are one run of 4 KB.
// (One tile per workgroup: with two, all eight loads of a thread in flight together, the kernel was slower.)
__global__ void __launch_bounds__(256) to_blocked_s8_quads_kernel(const uint8_t *__restrict__ x, uint4 *__restrict__ xb,
                                                                 unsigned n_quads, int C, unsigned CB, unsigned HW4) {
    __shared__ __attribute__((aligned(16))) uint32_t stage[4][256];
    const unsigned g = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const unsigned qi = blockIdx.x * 64u + lane;
    uint32_t r[4] = {0u, 0u, 0u, 0u};  // r[j] = 4 consecutive positions of channel c0 + j
    if (qi < n_quads) {
        const unsigned row = qi / HW4, q = qi - row * HW4;  // row = image * CB + channel block
        const unsigned n = row / CB, cb = row - n * CB;
        const int c0 = int(cb) * 16 + int(g) * 4;
        const uint32_t *src = reinterpret_cast<const uint32_t *>(x) + (int64_t(n) * C * HW4 + q);
        // The four loads leave together: a channel past C reads channel C - 1 instead of branching around its load
        // (with a branch per load the compiler waited for each one before the next), and is zeroed afterwards.
        uint32_t v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = __builtin_nontemporal_load(src + int64_t(min(c0 + j, C - 1)) * HW4);
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = c0 + j < C ? v[j] ^ 0x80808080u : 0u;
    }
    const uint32_t lo01 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);  // r0.0 r1.0 r0.1 r1.1
    const uint32_t hi01 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);  // r0.2 r1.2 r0.3 r1.3
    const uint32_t lo23 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
    const uint32_t hi23 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    uint4 o;  // dword b: position b, channels c0 .. c0+3
    o.x = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    o.y = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    o.z = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    o.w = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
    *reinterpret_cast<uint4 *>(&stage[g][lane * 4]) = o;
    __syncthreads();
    const unsigned u = threadIdx.x;
    if (blockIdx.x * 64u + (u >> 2) < n_quads)
        xb[int64_t(blockIdx.x) * 256 + u] = make_uint4(stage[0][u], stage[1][u], stage[2][u], stage[3][u]);
}

// Packs OIHW int8 weights into [chunk][kblock][tap][half][K_BLK][16] (zero padded; fc_g > 0: the weights of a 1x1
// layer with c_orig channels, read as a 1 x fc_g filter over C = 16 * ceil(c_orig / 16) / fc_g channels), and writes the
// per-channel requantisation multiplier, the integer correction (bias + (128 - x_zp) * sum w), the
// 16-byte padding vector (x_zp - 128 in every lane).
__global__ void __launch_bounds__(256)
qpack_kernel(const int8_t *__restrict__ w, const float *__restrict__ w_scale, const int32_t *__restrict__ bias,
             int8_t *__restrict__ wp, float *__restrict__ mult, int32_t *__restrict__ corr, int8_t *__restrict__ padvec,
             int K, int C, int T, int n_chunks, int n_kblocks, int k_blk,
             float x_scale, float y_scale, int x_zp, int n_wscale, int fc_g, int c_orig) {
    const int64_t total = int64_t(n_chunks) * n_kblocks * T * QCC * k_blk;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    const int64_t gid = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (gid < 16) padvec[gid] = int8_t(x_zp - 128);
    for (int64_t i = gid; i < total; i += step) {
        int64_t r = i;
        const int j = int(r & 15); r >>= 4;
        const int kk = int(r % k_blk); r /= k_blk;
        const int half = int(r & 1); r >>= 1;
        const int tap = int(r % T); r /= T;
        const int kb = int(r % n_kblocks); r /= n_kblocks;
        const int chunk = int(r);
        const int k = kb * k_blk + kk, c = chunk * QCC + half * 16 + j;
        if (fc_g) {
            // regrouped 1x1 layer: "tap" t of 16-channel block b is channel block b * fc_g + t of the c_orig real channels
            const int oc = ((c >> 4) * fc_g + tap) * 16 + j;
            wp[i] = (k < K && oc < c_orig) ? w[int64_t(k) * c_orig + oc] : int8_t(0);
        } else {
            wp[i] = (k < K && c < C) ? w[(int64_t(k) * C + c) * T + tap] : int8_t(0);
        }
    }
    // per output channel: one wavefront sums the channel's weights
    const int kpad = n_kblocks * k_blk;
    const int lane = threadIdx.x & 63;
    const int64_t wave = gid >> 6, n_waves = step >> 6;
    for (int64_t k = wave; k < kpad; k += n_waves) {
        int sum = 0;
        if (k < K) {
            const int row = fc_g ? c_orig : C * T;
            const int8_t *wk = w + k * int64_t(row);
            for (int e = lane; e < row; e += 64) sum += int(wk[e]);
        }
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        if (lane == 0) {
            if (k < K) {
                corr[k] = (bias ? bias[k] : 0) + (128 - x_zp) * sum;
                mult[k] = (x_scale * w_scale[n_wscale == 1 ? 0 : k]) / y_scale;
            } else {
                corr[k] = 0;
                mult[k] = 0.0f;
            }
        }
    }
}

// Bytes of the weight region of a staging buffer: the slab rounded up to one 16-byte unit per thread and round.
__device__ __host__ __forceinline__ int w_region_bytes(int w_chunk, int nt) { return ((w_chunk / 16 + nt - 1) / nt) * nt * 16; }

// Where this thread's patch slots of one tile come from: byte offset of the first 16-channel half of chunk 0 from the
// start of the blocked input, per copy round, and which rounds read real data (the others copy the padding vector).
// Filled once per tile (qconv_describe), so a step's copies cost an address add and a select each.
constexpr int QR_MAX = 4;  // copy rounds of the patch region: P1s / threads
struct PatchDesc {
    unsigned long long off[QR_MAX];
    unsigned ok;      // bit r: round r reads the input
    int kb;           // output-channel block of the tile (selects the weight slab)
};

template <int NT>
__device__ __forceinline__ void qconv_describe(PatchDesc &d, const int2 *__restrict__ ptab, const ConvGeom &g, const TileGeom &t,
                                               int CB, int itile) {
    int n0, oh0, kb;
    decode_tile(t, itile, n0, oh0, kb);
    d.kb = kb;
    d.ok = 0;
    const int64_t plane = int64_t(g.H) * g.W;
    const int ih0 = oh0 * g.sh - g.pt;
    const int imgs_here = min(t.NB, g.N - n0);
    const int64_t tile_base = int64_t(n0) * CB * plane + int64_t(ih0) * g.W;
#pragma unroll
    for (int r = 0; r < QR_MAX; ++r) {
        d.off[r] = 0;
        if (r * NT < t.P1s) {
            const int2 e = ptab[r * NT + int(threadIdx.x)];  // entries past P1 say "padding"
            const int ih = ih0 + (e.y & 0xffff);
            const bool ok = e.x >= 0 && ih >= 0 && ih < g.H && (e.y >> 16) < imgs_here;
            d.off[r] = ok ? (unsigned long long)((tile_base + e.x) * 16) : 0ull;
            d.ok |= ok ? 1u << r : 0u;
        }
    }
}

// The asynchronous copies of one (tile, chunk) step into the staging buffer `dma`.  Every thread issues the same
// number of copies whatever the geometry (lanes past the end of the slab repeat its last unit, patch slots past P1
// -- the patch region is padded to a multiple of the workgroup size -- copy the padding vector), so the number of
// copies a wave has in flight per step is a constant the ring's waits can count with.
template <int WM, int WN, int TT>
__device__ __forceinline__ void qconv_issue(char *__restrict__ dma, const PatchDesc &d, const int8_t *__restrict__ xb,
                                            const int8_t *__restrict__ wp, const int8_t *__restrict__ padvec,
                                            const ConvGeom &g, const TileGeom &t, int CB, int ichunk) {
    constexpr int NT = WM * WN * 64;
    constexpr int K_BLK = WN * 32;
    const int T = TT > 0 ? TT : g.KH * g.KW;
    const int w_chunk = T * QCC * K_BLK;  // bytes
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    char *xl = dma + w_region_bytes(w_chunk, NT);
    const int8_t *wsrc = wp + (int64_t(ichunk) * t.n_kblocks + d.kb) * w_chunk;
    const int units = w_chunk >> 4;
    for (int u0 = 0; u0 < units; u0 += NT) {
        const int u = min(u0 + tid, units - 1);
        __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + u * 16), (lptr_t)(dma + (u0 + wave * 64) * 16), 16, 0, 0);
    }
    const int64_t plane16 = int64_t(g.H) * g.W * 16;
    const int8_t *xc = xb + int64_t(ichunk * 2) * plane16;   // first half of this chunk
    const bool second = ichunk * 2 + 1 < CB;                 // an odd block count leaves the last chunk half empty
#pragma unroll
    for (int r = 0; r < QR_MAX; ++r) {
        if (r * NT < t.P1s) {
            const bool ok = (d.ok >> r) & 1u;
            const int8_t *src = xc + d.off[r];
            const int8_t *s0 = ok ? src : padvec;
            const int8_t *s1 = (ok && second) ? src + plane16 : padvec;
            __builtin_amdgcn_global_load_lds((gptr_t)s0, (lptr_t)(xl + (r * NT + wave * 64) * 16), 16, 0, 0);
            // A layer of at most 16 input channels has no second half anywhere: its slots stay as they are -- whatever
            // integers they hold meet zero weights.
            if (CB > 1) __builtin_amdgcn_global_load_lds((gptr_t)s1, (lptr_t)(xl + (t.P1s + r * NT + wave * 64) * 16), 16, 0, 0);
        }
    }
}

// LDS reads the compiler does not see (it would drain every outstanding asynchronous copy before an LDS read of its
// own that it cannot prove independent of them).  The *_wait functions take the values as in/out operands so that their
// users stay behind the wait; nothing read this way is kept in flight across a loop edge.
__device__ __forceinline__ unsigned lds_addr_of(const void *p) {
    return unsigned(reinterpret_cast<uintptr_t>((lptr_t) const_cast<void *>(p)));
}
__device__ __forceinline__ uint32_t lds_read_u8_async(unsigned addr) {
    uint32_t v;
    asm volatile("ds_read_u8 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
__device__ __forceinline__ uint32_t lds_read_b32_async(unsigned addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
__device__ __forceinline__ void lds_wait16(uint32_t (&v)[16]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                   "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]));
}

// Waits until at most n of this wave's vector-memory operations are outstanding (n is wave-uniform, 0..63).
__device__ __forceinline__ void wait_vmcnt(int n) {
#define ZANT_VM(k) case k: __builtin_amdgcn_s_waitcnt(((k) & 15) | (((k) >> 4) << 14) | 0x0F70); break;
#define ZANT_VM8(b) ZANT_VM(b) ZANT_VM(b + 1) ZANT_VM(b + 2) ZANT_VM(b + 3) ZANT_VM(b + 4) ZANT_VM(b + 5) ZANT_VM(b + 6) ZANT_VM(b + 7)
    switch (n) {
        ZANT_VM8(0) ZANT_VM8(8) ZANT_VM8(16) ZANT_VM8(24) ZANT_VM8(32) ZANT_VM8(40) ZANT_VM8(48) ZANT_VM8(56)
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    }
#undef ZANT_VM8
#undef ZANT_VM
}

// One (tile, chunk) step: start the global->LDS copies of the next step into `dma`, run the int8
// matrix cores over this step's operands in `cmp`.  The LDS regions never overlap within a step and
// are __restrict__ so that the copies stay in flight across this step's LDS reads.
template <int MT, int WM, int WN, int TT>
__device__ __forceinline__ void qconv_step(char *__restrict__ dma, const char *__restrict__ cmp, const PatchDesc &desc,
                                           const int8_t *__restrict__ xb, const int8_t *__restrict__ wp,
                                           const int8_t *__restrict__ padvec, const ConvGeom &g, const TileGeom &t, int CB,
                                           bool do_issue, int ichunk, const int (&lds_off)[MT], i32x16 (&acc)[MT]) {
    constexpr int NT = WM * WN * 64;
    constexpr int K_BLK = WN * 32;
    const int T = TT > 0 ? TT : g.KH * g.KW;
    const int w_chunk = T * QCC * K_BLK;  // bytes
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;

    if (do_issue) qconv_issue<WM, WN, TT>(dma, desc, xb, wp, padvec, g, t, CB, ichunk);
    __builtin_amdgcn_sched_barrier(0);

    const char *wl = cmp + (lh * K_BLK + wn * 32 + l32) * 16;
    const char *xl = cmp + w_region_bytes(w_chunk, NT) + lh * t.P1s * 16;
    i32x4 a0, a1, b0[MT], b1[MT];
    int lkh = 0, lkw = 0, ltap = 0;
    auto load_tap = [&](i32x4 &a, i32x4 (&b)[MT]) {
        const int off = (lkh * g.dh * t.PW + lkw * g.dw) * 16;
        a = *reinterpret_cast<const i32x4 *>(wl + ltap * 2 * K_BLK * 16);
#pragma unroll
        for (int i = 0; i < MT; ++i) b[i] = *reinterpret_cast<const i32x4 *>(xl + lds_off[i] * 16 + off);
        ++ltap;
        if (++lkw == g.KW) { lkw = 0; ++lkh; }
    };
    auto mfma_tap = [&](const i32x4 &a, const i32x4 (&b)[MT]) {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b[i], acc[i], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
    };
    if (TT > 0) {
        constexpr int NTAP = TT > 0 ? TT : 1;
        load_tap(a0, b0);
#pragma unroll
        for (int tp = 0; tp < NTAP; tp += 2) {
            if (tp + 1 < NTAP) load_tap(a1, b1);
            mfma_tap(a0, b0);
            if (tp + 1 < NTAP) {
                if (tp + 2 < NTAP) load_tap(a0, b0);
                mfma_tap(a1, b1);
            }
        }
    } else {
        load_tap(a0, b0);
        for (int tp = 0; tp < T; tp += 2) {
            if (tp + 1 < T) load_tap(a1, b1);
            mfma_tap(a0, b0);
            if (tp + 1 < T) {
                if (tp + 2 < T) load_tap(a0, b0);
                mfma_tap(a1, b1);
            }
        }
    }
}

// Persistent int8 implicit-GEMM convolution over the channel-blocked input.  A workgroup walks its tiles
// (blockIdx.x, blockIdx.x + gridDim.x, ...) chunk by chunk; the (tile, chunk) steps form one sequence whose operand
// copies run n_stages - 1 steps ahead of the matrix cores through a ring of n_stages LDS buffers, so that a step's
// copy latency is hidden even when the step itself is only a few MFMAs (1x1 layers, small feature maps).
template <int MT, int WM, int WN, int TT, bool POOL = false>
__global__ void __launch_bounds__(WM *WN * 64, 2)
qconv_mfma_kernel(const int8_t *__restrict__ xb, const int8_t *__restrict__ wp, const float *__restrict__ mult,
                  const int32_t *__restrict__ corr, const int8_t *__restrict__ padvec, uint8_t *__restrict__ y, ConvGeom g,
                  TileGeom t, int CB, QConvArgs q, int n_stages, int y_blocked) {
    constexpr int NT = WM * WN * 64;
    constexpr int K_BLK = WN * 32;
    extern __shared__ __attribute__((aligned(256))) char qlds_raw[];
    const int T = TT > 0 ? TT : g.KH * g.KW;
    const int w_chunk = T * QCC * K_BLK;                           // bytes per (chunk, kblock) weight slab
    const int buf_bytes = w_region_bytes(w_chunk, NT) + QCC * t.P1s;  // one staging buffer (P1s: multiple of NT)
    // LDS: [256-byte activation table, 256-aligned][n_stages staging buffers][patch table][multipliers][corrections]
    const unsigned lut_a = (lds_addr_of(qlds_raw) + 255u) & ~255u;
    char *qlds = qlds_raw + (lut_a - lds_addr_of(qlds_raw));
    uint8_t *lut = reinterpret_cast<uint8_t *>(qlds);
    char *ring = qlds + 256;
    int2 *ptab = reinterpret_cast<int2 *>(ring + n_stages * buf_bytes);
    const int kpad = t.n_kblocks * K_BLK;
    float *mult_l = reinterpret_cast<float *>(ptab + t.P1s);    // [kpad] requantisation multipliers ...
    int *corr_l = reinterpret_cast<int *>(mult_l + kpad);       // [kpad] ... and integer corrections, copied once

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;
    const int64_t plane_in = int64_t(g.H) * g.W;
    const int per_img = t.TH * g.OW;
    const int patch_hw = t.PH * t.PW;
    const float inv_per_img = 1.0f / float(per_img), inv_ow = 1.0f / float(g.OW);
    // The tables first (plain LDS writes), the copies after them: an LDS write behind an asynchronous copy would wait
    // for the copy.  The activation table holds output bytes as they are stored (blocked tensors keep value ^ 0x80).
    {
        const uint8_t b = uint8_t(tid & 255);
        lut[tid & 255] = uint8_t((q.has_act ? qact_apply(b, q.act) : b) ^ (y_blocked ? 0x80 : 0));  // NT == 256
    }
    {
        const float inv_patch = 1.0f / float(patch_hw), inv_pw = 1.0f / float(t.PW);
        for (int e = tid; e < t.P1s; e += NT) {
            const int img = small_div(e, patch_hw, inv_patch), rem = e - img * patch_hw;
            const int ph = small_div(rem, t.PW, inv_pw), pw = rem - ph * t.PW;
            const int iw = pw - g.pl;
            int2 v;
            v.x = (e < t.P1 && iw >= 0 && iw < g.W) ? int(img * CB * plane_in) + ph * g.W + iw : -1;
            v.y = (img << 16) | ph;
            ptab[e] = v;   // read back by this same thread only (qconv_issue)
        }
    }
    if (int(blockIdx.x) >= t.n_tiles) return;
    const int my_tiles = (t.n_tiles - int(blockIdx.x) + int(gridDim.x) - 1) / int(gridDim.x);
    const int n_steps = my_tiles * t.n_chunks;
    // The requantisation tables go to LDS as asynchronous copies at the head of the copy stream: copies land in order,
    // so they are there when the first step's operands are, and nobody waits for a global load before the first
    // operand copy is on its way.
    for (int k0 = 0; k0 < kpad; k0 += NT)
        if (k0 + tid < kpad) {
            __builtin_amdgcn_global_load_lds((gptr_t)(mult + k0 + tid), (lptr_t)(mult_l + k0 + wave * 64), 4, 0, 0);
            __builtin_amdgcn_global_load_lds((gptr_t)(corr + k0 + tid), (lptr_t)(corr_l + k0 + wave * 64), 4, 0, 0);
        }
    // copies per thread and step (see qconv_issue)
    const int P = w_region_bytes(w_chunk, NT) / (16 * NT) + (CB > 1 ? 2 : 1) * (t.P1s / NT);
    // prologue: the first n_stages - 1 steps' copies, in flight behind the index arithmetic below
    PatchDesc desc;
    for (int s0 = 0; s0 < n_stages - 1 && s0 < n_steps; ++s0) {
        if (s0 % t.n_chunks == 0) qconv_describe<NT>(desc, ptab, g, t, CB, int(blockIdx.x) + (s0 / t.n_chunks) * int(gridDim.x));
        qconv_issue<WM, WN, TT>(ring + s0 * buf_bytes, desc, xb, wp, padvec, g, t, CB, s0 % t.n_chunks);
    }
    __builtin_amdgcn_sched_barrier(0);

    // Position slot i of this lane: image, row and column inside the tile.  pos[i] packs them for the epilogue
    // (image << 20 | row << 10 | column; -1 = the slot is beyond the tile).  With a fused 2x2/2 max pool, slots
    // 4j .. 4j+3 are the four members of ONE pooling window (pooled position (wm*MT/4 + j)*32 + l32) and pos[4j] holds
    // the POOLED row and column: the pool is a register-wise reduction in the epilogue.
    int lds_off[MT], pos[MT];
    const int per_img_p = POOL ? (t.TH / 2) * t.POW : 1;
    const float inv_per_img_p = 1.0f / float(per_img_p), inv_pow = 1.0f / float(POOL ? t.POW : 1);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        int img, r, c, pr = 0, pc = 0;
        if (POOL) {
            const int pp = (wm * (MT / 4) + i / 4) * 32 + l32;
            img = small_div(pp, per_img_p, inv_per_img_p);
            const int rem = pp - img * per_img_p;
            pr = small_div(rem, t.POW, inv_pow);
            pc = rem - pr * t.POW;
            r = 2 * pr + ((i & 3) >> 1);
            c = 2 * pc + (i & 1);
        } else {
            const int p = (wm * MT + i) * 32 + l32;
            img = small_div(p, per_img, inv_per_img);
            const int rem = p - img * per_img;
            r = small_div(rem, g.OW, inv_ow);
            c = rem - r * g.OW;
        }
        const bool in_tile = img < t.NB && r < t.TH;
        lds_off[i] = in_tile ? (img * t.PH + r * g.sh) * t.PW + c * g.sw : 0;
        pos[i] = in_tile ? (img << 20) | ((POOL ? pr : r) << 10) | (POOL ? pc : c) : -1;
    }
    // everybody's table writes are visible after the first barrier of the loop below
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0) only
    const unsigned mult_a = lds_addr_of(mult_l), corr_a = lds_addr_of(corr_l);

    i32x16 acc[MT];
    int cbuf = 0, dbuf = n_stages - 1;    // ring slots of the step being multiplied / of the step being copied
    int itile = int(blockIdx.x), ichunk = 0;  // (tile, chunk) of the step whose copies are issued next
    for (int s0 = 0; s0 < n_stages - 1; ++s0)
        if (++ichunk == t.n_chunks) { ichunk = 0; itile += int(gridDim.x); }
    int cur = int(blockIdx.x), chunk = 0;
    for (int s0 = 0; s0 < n_steps; ++s0) {
        // This wave's copies of step s0 have landed once no more than the copies of the later steps are outstanding
        // (loads complete in order); after the barrier everybody's have, and everybody is done with step s0 - 1,
        // whose ring slot is refilled now.  A bare s_barrier: __syncthreads() would drain every outstanding copy.
        {
            const int pending = P * min(n_stages - 2, n_steps - 1 - s0);
            if (pending == 0) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): two-stage rings and the last step
            else wait_vmcnt(pending);
        }
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (chunk == 0) {
            // accumulators start from the integer corrections of this lane's 16 output channels
            const int kb = cur % t.n_kblocks;
            const int kbase = kb * K_BLK + wn * 32 + lh * 4;
            uint32_t craw[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) craw[v] = lds_read_b32_async(corr_a + unsigned(kbase + (v >> 2) * 8 + (v & 3)) * 4u);
            lds_wait16(craw);
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][v] = int(craw[v]);
        }
        const bool do_issue = s0 + n_stages - 1 < n_steps;
        if (do_issue && ichunk == 0) qconv_describe<NT>(desc, ptab, g, t, CB, itile);
        qconv_step<MT, WM, WN, TT>(ring + dbuf * buf_bytes, ring + cbuf * buf_bytes, desc, xb, wp, padvec, g, t, CB, do_issue,
                                   ichunk, lds_off, acc);
        if (++ichunk == t.n_chunks) { ichunk = 0; itile += int(gridDim.x); }
        cbuf = cbuf + 1 == n_stages ? 0 : cbuf + 1;
        dbuf = dbuf + 1 == n_stages ? 0 : dbuf + 1;
        if (++chunk < t.n_chunks) continue;
        chunk = 0;

        // ---- epilogue: requantisation (+ fused activation), stores ----
        {
            int n0, oh0, kb;
            decode_tile(t, cur, n0, oh0, kb);
            // output geometry: the convolution's own, or the pooled one
            const int OHo = POOL ? g.OH / 2 : g.OH, OWo = POOL ? t.POW : g.OW;
            if (POOL) oh0 >>= 1;
            const int rows_here = min(POOL ? t.TH / 2 : t.TH, OHo - oh0);
            const int imgs_here = min(t.NB, g.N - n0);
            const int64_t plane = int64_t(OHo) * OWo;
            const int kbase = kb * K_BLK + wn * 32 + lh * 4;
            // multipliers of this lane's 16 channels, then per position the 16 activation-table lookups, all through
            // hand-issued LDS reads: the next steps' copies stay in flight behind the epilogue
            uint32_t mraw[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) mraw[v] = lds_read_b32_async(mult_a + unsigned(kbase + (v >> 2) * 8 + (v & 3)) * 4u);
            lds_wait16(mraw);
            float mv[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) mv[v] = __uint_as_float(mraw[v]);
            const float zpf = float(q.y_zp);
            const int KB = (g.K + 15) >> 4;
            const int cb0 = (kb * K_BLK + wn * 32) >> 4;
            const bool use_lut = q.has_act || !y_blocked;
            const bool y_dwords = !POOL && plane == 1 && (g.K & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 3) == 0;
            if (POOL) {
                // Requantisation and the activation are monotone (non-decreasing for a positive multiplier, non-increasing
                // for a negative one), so the window's maximum output comes from its largest or smallest accumulator.
#pragma unroll
                for (int j = 0; j < MT / 4; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int a0 = acc[4 * j][v], a1 = acc[4 * j + 1][v], a2 = acc[4 * j + 2][v], a3 = acc[4 * j + 3][v];
                        const int mx = max(max(a0, a1), max(a2, a3)), mn = min(min(a0, a1), min(a2, a3));
                        acc[4 * j][v] = mv[v] >= 0.0f ? mx : mn;
                    }
            }
#pragma unroll
            for (int i = 0; i < MT; i += (POOL ? 4 : 1)) {
                const int img = pos[i] >> 20, r = (pos[i] >> 10) & 1023, c = pos[i] & 1023;
                const bool ok = pos[i] >= 0 && img < imgs_here && r < rows_here;
                if (y_blocked) {
                    // [N][KB][OH][OW][16] signed.  A lane holds 4 groups of 4 consecutive channels; lanes l and l+32
                    // swap one dword per 16-channel block so that each stores 8 consecutive bytes: a half-wave then
                    // writes 32 positions x 16 bytes without gaps.
                    uint32_t d[4];
                    if (use_lut) {
                        uint32_t ob[16];
                        // the converted byte lands in the low byte of the (256-aligned) table address
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            ob[v] = lds_read_u8_async(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[i][v]) * mv[v]) + zpf, 0u, lut_a));
                        lds_wait16(ob);
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq)
                            d[gq] = ob[gq * 4] | (ob[gq * 4 + 1] << 8) | (ob[gq * 4 + 2] << 16) | (ob[gq * 4 + 3] << 24);
                    } else {
                        // no activation: the saturating conversion packs the four bytes of a dword itself
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq) {
                            uint32_t w4 = 0;
#pragma unroll
                            for (int e = 0; e < 4; ++e)
                                w4 = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[i][gq * 4 + e]) * mv[gq * 4 + e]) + zpf, unsigned(e), w4);
                            d[gq] = w4 ^ 0x80808080u;
                        }
                    }
#pragma unroll
                    for (int b = 0; b < 2; ++b) {
                        const uint32_t send = lh ? d[2 * b] : d[2 * b + 1];
                        const uint32_t recv = uint32_t(__shfl_xor(int(send), 32, 64));
                        const uint2 out = lh ? make_uint2(recv, d[2 * b + 1]) : make_uint2(d[2 * b], recv);
                        if (ok && cb0 + b < KB) {
                            uint8_t *yp = y + (((int64_t(n0 + img) * KB + cb0 + b) * OHo + oh0 + r) * OWo + c) * 16 + lh * 8;
                            __builtin_nontemporal_store(*reinterpret_cast<const unsigned long long *>(&out), reinterpret_cast<unsigned long long *>(yp));
                        }
                    }
                } else {
                    uint32_t ob[16];  // the 16 output bytes of this position
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        ob[v] = lds_read_u8_async(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[i][v]) * mv[v]) + zpf, 0u, lut_a));
                    lds_wait16(ob);
                    if (ok) {
                        uint8_t *yp = y + (int64_t(n0 + img) * g.K + kbase) * plane + int64_t(oh0 + r) * OWo + c;
                        if (y_dwords) {
                            // one output position per image: a lane's four consecutive channels are four consecutive bytes
#pragma unroll
                            for (int gq = 0; gq < 4; ++gq)
                                if (kbase + gq * 8 < g.K)
                                    *reinterpret_cast<uint32_t *>(yp + gq * 8) =
                                        ob[gq * 4] | (ob[gq * 4 + 1] << 8) | (ob[gq * 4 + 2] << 16) | (ob[gq * 4 + 3] << 24);
                        } else {
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                const int dk = (v >> 2) * 8 + (v & 3);
                                if (kbase + dk < g.K) yp[dk * plane] = uint8_t(ob[v]);
                            }
                        }
                    }
                }
            }
        }
        cur += int(gridDim.x);
    }
}

template <int MT, int WM, int WN, int TT, bool POOL = false>
void launch_qmfma_tt(zant_ctx *ctx, const int8_t *xb, const int8_t *wp, const float *mult, const int32_t *corr,
                     const int8_t *padvec, uint8_t *y, const ConvGeom &g, const TilePlan &p, int CB, const QConvArgs &q,
                     int grid, int yb, int n_stages) {
    if (!zant_raise_lds_limit(ctx, reinterpret_cast<const void *>(&qconv_mfma_kernel<MT, WM, WN, TT, POOL>), 160 * 1024)) return;
    ZANT_KERNEL_NAME(ctx, "qconv_mfma_kernel<%d,%d,%d,%d,%s>", MT, WM, WN, TT, POOL ? "true" : "false");
    hipLaunchKernelGGL((qconv_mfma_kernel<MT, WM, WN, TT, POOL>), dim3(grid), dim3(WM * WN * 64), p.lds_bytes, ctx->stream, xb,
                       wp, mult, corr, padvec, y, g, p.t, CB, q, n_stages, yb);
}

template <int MT, int WM, int WN>
void launch_qmfma(zant_ctx *ctx, const int8_t *xb, const int8_t *wp, const float *mult, const int32_t *corr,
                  const int8_t *padvec, uint8_t *y, const ConvGeom &g, const TilePlan &p, int CB, const QConvArgs &q,
                  int grid, int yb, int n_stages) {
    const int T = g.KH * g.KW;
    if (T == 9) launch_qmfma_tt<MT, WM, WN, 9>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages);
    else if (T == 1) launch_qmfma_tt<MT, WM, WN, 1>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages);
    else launch_qmfma_tt<MT, WM, WN, 0>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages);
}

template <int WM, int WN>
bool dispatch_qmt(zant_ctx *ctx, const int8_t *xb, const int8_t *wp, const float *mult, const int32_t *corr,
                  const int8_t *padvec, uint8_t *y, const ConvGeom &g, const TilePlan &p, int CB, const QConvArgs &q,
                  int grid, int yb, int n_stages, bool pool) {
    if (pool) {  // four window members per lane: MT = 4
        if (p.MT != 4) return false;
        const int T = g.KH * g.KW;
        if (T == 9) launch_qmfma_tt<4, WM, WN, 9, true>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages);
        else if (T == 1) launch_qmfma_tt<4, WM, WN, 1, true>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages);
        else launch_qmfma_tt<4, WM, WN, 0, true>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages);
        return true;
    }
    switch (p.MT) {
    case 1: launch_qmfma<1, WM, WN>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages); return true;
    case 2: launch_qmfma<2, WM, WN>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages); return true;
    case 3: launch_qmfma<3, WM, WN>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages); return true;
    case 4: launch_qmfma<4, WM, WN>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages); return true;
    case 5: launch_qmfma<5, WM, WN>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages); return true;
    case 6: launch_qmfma<6, WM, WN>(ctx, xb, wp, mult, corr, padvec, y, g, p, CB, q, grid, yb, n_stages); return true;
    default: return false;
    }
}

static size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

unsigned to_blocked_grid(zant_ctx *ctx, int64_t N, int64_t CB, int64_t hw) {
    const int64_t units = N * CB * ((hw + 3) / 4);
    return unsigned(std::min<int64_t>(std::max<int64_t>(ceil_div64(units, 256), 1), int64_t(ctx->num_cus) * 16));
}

// The matrix-core path; returns ZANT_OK when it ran, 1 when the shape is left to the other kernels.
// x_blocked / y_blocked: x, y are already / are to be written in the blocked signed layout.
int run_qconv_mfma(zant_ctx *ctx, const uint8_t *x, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *y,
                   const ConvGeom &g0, const QConvArgs &q, bool x_blocked, bool y_blocked, zant_pack_slot *slot, bool pool = false,
                   bool plan_only = false) {
    if (g0.groups != 1 || g0.C < 5 || int64_t(g0.N) * g0.OH * g0.OW < 64) return 1;
    // What the planning below decides depends on the geometry only: a node or plan that calls again with the same one
    // reuses it (the searches for a tile shape cost the host as much time as a small layer takes on the GPU).
    struct PlanKey { ConvGeom g; int x_blocked, y_blocked, pool, cus, act_ok, kind; } pkey;
    struct PlanVal { ConvGeom g; TilePlan plan; int WN, n_stages, fc_g; } pval;
    std::memset(&pkey, 0, sizeof(pkey));
    pkey.g = g0; pkey.x_blocked = x_blocked; pkey.y_blocked = y_blocked; pkey.pool = pool; pkey.cus = ctx->num_cus;
    pkey.act_ok = !q.has_act || (q.act.alpha >= 0.0f && q.act.in_scale > 0.0f && q.act.out_scale > 0.0f);
    pkey.kind = 0x54494c45;  // "TILE"
    const bool cached = !plan_only && zant_plan_cached(slot, pkey, &pval);
    if (!cached) {
        // 3x3 / stride 1 layers with at least 32 channels on both sides: the patch-stationary kernel
        const int rc = zant_qconv_ps(ctx, x, w, w_scale, bias, y, g0, q, x_blocked, y_blocked, slot, plan_only, pool);
        if (rc <= 0) return rc;
    }
    ConvGeom g = g0;
    int fc_g = 0, WN = 1, n_stages = 2;
    TilePlan plan;
    constexpr int NT = 256;
    if (cached) {
        g = pval.g; plan = pval.plan; WN = pval.WN; n_stages = pval.n_stages; fc_g = pval.fc_g;
    } else {
    // A 1x1 layer over 1x1 feature maps (a classifier head behind a global pool) is a matrix product whose rows, the
    // images, are ceil(C / 16) * 16 contiguous bytes each.  Staged 32 channels at a time it runs C / 32 short steps of
    // 32-byte copies, one cache line each.  Read instead as a 1 x G filter over a 1 x G "image" of C / G channels -- G
    // consecutive 16-channel blocks taken as G columns: the same bytes, the same sums -- it runs G times fewer steps,
    // each copying G times longer contiguous runs.  Only the weight packing knows the difference.
    if (!pool && g0.H == 1 && g0.W == 1 && g0.KH == 1 && g0.KW == 1 && g0.OH == 1 && g0.OW == 1 && g0.pt == 0 && g0.pl == 0) {
        const int cb = (g0.C + 15) / 16;
        for (int cand = 8; cand >= 2 && !fc_g; cand >>= 1)
            if (cb % cand == 0 && cb / cand >= 2) fc_g = cand;
        if (fc_g) {
            g.C = cb / fc_g * 16;
            g.CG = g.C;
            g.W = g.KW = fc_g;
            g.sh = g.sw = g.dh = g.dw = 1;
        }
    }
    // a fused 2x2/2 max pool needs whole windows and an activation that keeps the order of its inputs
    if (pool && (g.OH < 2 || g.OW < 2 || (q.has_act && !(q.act.alpha >= 0.0f && q.act.in_scale > 0.0f && q.act.out_scale > 0.0f))))
        return 1;
    const int CB = (g.C + 15) / 16;
    if (int64_t(g.N) * CB * g.H * g.W >= (int64_t(1) << 27)) return 1;  // 16-byte units addressed with 32-bit offsets
    ConvGeom gp = g;
    gp.C = CB;  // the planner's 32-bit offset check works in 16-byte units here
    // at most 6 position tiles per wave: with 7 the epilogue spills, and a scratch reload drains the copy ring.
    // Both workgroup shapes are tried for more than 32 output channels; plans are ranked by the planner's time estimate
    // over the GPU's 2 x CUs workgroup slots.
    const int target = 2 * ctx->num_cus;
    // The footprint counts two staging buffers: larger tiles (more operand reuse per staged byte) beat a deeper ring.
    bool have = zant_plan_conv_tiles(gp, 4, 1, 6, 2, 16, 80 * 1024, &plan, pool, target, 32, 256);
    if (g.K > 32) {
        TilePlan wide;
        if (zant_plan_conv_tiles(gp, 2, 2, 6, 2, 16, 80 * 1024, &wide, pool, target, 32, 256) && (!have || wide.score >= plan.score * 0.98)) {
            plan = wide; WN = 2; have = true;
        }
    }
    if (!have || plan.eff < 0.4) return 1;
    const int T = g.KH * g.KW, K_BLK = WN * 32;
    plan.t.n_chunks = (g.C + QCC - 1) / QCC;
    // Ring of staging buffers: as many stages as fit beside the tables in the LDS share of a workgroup -- half a CU's
    // 160 KB when two workgroups share a CU, all of it when the layer has no more tiles than the GPU has CUs (short
    // per-tile sequences, where a deeper ring hides more of the copy latency) -- and as the 6-bit vmcnt counter can
    // tell apart.  The patch region is padded to one slot per thread and round.
    // The patch row pitch: a few columns of padding where they take bank conflicts out of the operand reads (the extra
    // columns are copied as padding and never read), as long as two staging buffers still fit.
    {
        const size_t cap2 = plan.t.n_tiles <= ctx->num_cus ? 160 * 1024 : 80 * 1024;
        const int pw0 = plan.t.PW;
        double best_c = zant_patch_read_cycles(plan, g, pool, pw0);
        int best_pw = pw0;
        for (int pw = pw0 + 1; pw <= pw0 + 9 && best_c > 1.0; ++pw) {
            const int p1 = plan.t.NB * plan.t.PH * pw, p1s = ((p1 + NT - 1) / NT) * NT;
            const size_t need = 2 * (size_t(w_region_bytes(T * QCC * K_BLK, NT)) + size_t(QCC) * p1s) + size_t(p1s) * 8 + 512 +
                                size_t(plan.t.n_kblocks) * K_BLK * 8;
            if (p1s / NT > QR_MAX || need > cap2) break;
            const double c = zant_patch_read_cycles(plan, g, pool, pw);
            if (c < best_c * 0.9) { best_c = c; best_pw = pw; }
        }
        plan.t.PW = best_pw;
        plan.t.P1 = plan.t.NB * plan.t.PH * best_pw;
    }
    plan.t.P1s = ((plan.t.P1 + NT - 1) / NT) * NT;
    if (plan.t.P1s / NT > QR_MAX) return 1;  // more copy rounds than the per-tile descriptors hold
    const size_t buf_bytes = size_t(w_region_bytes(T * QCC * K_BLK, NT)) + size_t(QCC) * plan.t.P1s;
    const size_t fixed_bytes = size_t(plan.t.P1s) * 8 + 512 + size_t(plan.t.n_kblocks) * K_BLK * 8;  // 256: table, 256: its alignment
    const int copies = w_region_bytes(T * QCC * K_BLK, NT) / (16 * NT) + (CB > 1 ? 2 : 1) * (plan.t.P1s / NT);
    const bool sparse = plan.t.n_tiles <= ctx->num_cus;
    const size_t lds_cap = sparse ? 160 * 1024 : 80 * 1024;
    n_stages = sparse ? 8 : 4;
    if (n_stages > plan.t.n_chunks + 1) n_stages = std::max(plan.t.n_chunks + 1, 2);
    while (n_stages > 2 && (n_stages * buf_bytes + fixed_bytes > lds_cap || copies * (n_stages - 2) > 63)) --n_stages;
    if (n_stages * buf_bytes + fixed_bytes > lds_cap) return 1;
        if (!plan_only) {
            std::memset(&pval, 0, sizeof(pval));
            pval.g = g; pval.plan = plan; pval.WN = WN; pval.n_stages = n_stages; pval.fc_g = fc_g;
            zant_plan_remember(slot, pkey, pval);
        }
    }
    const int CB = (g.C + 15) / 16;
    const int T = g.KH * g.KW, K_BLK = WN * 32;
    const size_t buf_bytes = size_t(w_region_bytes(T * QCC * K_BLK, NT)) + size_t(QCC) * plan.t.P1s;
    const size_t fixed_bytes = size_t(plan.t.P1s) * 8 + 512 + size_t(plan.t.n_kblocks) * K_BLK * 8;  // 256: table, 256: its alignment
    if (plan_only) return ZANT_OK;
    plan.lds_bytes = n_stages * buf_bytes + fixed_bytes;
    const size_t wp_bytes = size_t(plan.t.n_chunks) * plan.t.n_kblocks * T * QCC * K_BLK;
    const size_t kpad = size_t(plan.t.n_kblocks) * K_BLK;
    const int CB0 = (g0.C + 15) / 16;
    const size_t xb_bytes = x_blocked ? 0 : size_t(g0.N) * CB0 * g0.H * g0.W * 16;
    const size_t o_pad = 256, o_mult = 512, o_corr = o_mult + align256(kpad * 4), o_wp = o_corr + align256(kpad * 4),
                 static_bytes = o_wp + align256(wp_bytes);
    void *ws = nullptr, *dyn = nullptr;
    bool need_pack = true;
    int parity = 0;
    int rc = zant_pack_region(ctx, slot, static_bytes, xb_bytes, &ws, &dyn, &need_pack, &parity);
    if (rc) return rc;
    char *base = static_cast<char *>(ws);
    int8_t *padvec = reinterpret_cast<int8_t *>(base + o_pad);
    float *mult = reinterpret_cast<float *>(base + o_mult);
    int32_t *corr = reinterpret_cast<int32_t *>(base + o_corr);
    int8_t *wp = reinterpret_cast<int8_t *>(base + o_wp);
    const int8_t *xb = x_blocked ? reinterpret_cast<const int8_t *>(x) : static_cast<const int8_t *>(dyn);
    const int grid = int(std::min<int64_t>(plan.t.n_tiles, int64_t(ctx->num_cus) * 2));
    const unsigned pb = unsigned(std::min<int64_t>(std::max<int64_t>(ceil_div64(int64_t(wp_bytes), 256), ceil_div64(int64_t(kpad), 4)), 1024));
    if (need_pack) {
        hipLaunchKernelGGL(qpack_kernel, dim3(pb), dim3(256), 0, ctx->stream, w, w_scale, bias, wp, mult, corr, padvec,
                           g.K, g.C, T, plan.t.n_chunks, plan.t.n_kblocks, K_BLK, q.x_scale, q.y_scale, q.x_zp,
                           q.n_wscale, fc_g, g0.C);
        ZANT_LAUNCH_CHECK(ctx);
    }
    if (!x_blocked) {
        const int rc2 = zant_to_blocked(ctx, x, g0.N, g0.C, int64_t(g0.H) * g0.W, static_cast<uint8_t *>(dyn));
        if (rc2) return rc2;
    }
    KernelTimer kt(ctx);
    const int yb = y_blocked ? 1 : 0;
    const bool ok = WN == 2 ? dispatch_qmt<2, 2>(ctx, xb, wp, mult, corr, padvec, y, g, plan, CB, q, grid, yb, n_stages, pool)
                            : dispatch_qmt<4, 1>(ctx, xb, wp, mult, corr, padvec, y, g, plan, CB, q, grid, yb, n_stages, pool);
    if (!ok) return 1;
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// ------------------------------------------------------------------------------------------------------------------
// First layers (1..4 input channels, 3x3): one thread per output position, 16 output channels at a time.  The C*9
// taps of a position are gathered once into signed bytes (x - 128, padding = x_zp - 128) and every output channel is
// 7 (or 3) v_dot4_i32_i8 against weights the whole wave shares (scalar loads).  The zero point is folded as in the
// matrix-core path.  Optionally max-pools 2x2/2 the four positions of a window before the store.
// Reads NCHW u8; writes NCHW u8 or the blocked signed layout (one 16-byte store per position and channel block).
// ------------------------------------------------------------------------------------------------------------------
template <int C>
__global__ void __launch_bounds__(256)
qconv_smallc_pack_kernel(const int8_t *__restrict__ w, const float *__restrict__ w_scale, const int32_t *__restrict__ bias,
                         uint32_t *__restrict__ wpk, float *__restrict__ mult, int32_t *__restrict__ corr, int K, int kpad,
                         float x_scale, float y_scale, int x_zp, int n_wscale) {
    constexpr int NT = C * 9, ND = (NT + 3) / 4;
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= kpad) return;
    int sum = 0;
    for (int d = 0; d < ND; ++d) {
        uint32_t v = 0;
        for (int e = 0; e < 4; ++e) {
            const int t = d * 4 + e;
            const int wv = (k < K && t < NT) ? int(w[int64_t(k) * NT + t]) : 0;
            sum += wv;
            v |= uint32_t(uint8_t(wv)) << (8 * e);
        }
        wpk[k * ND + d] = v;
    }
    corr[k] = k < K ? (bias ? bias[k] : 0) + (128 - x_zp) * sum : 0;
    mult[k] = k < K ? (x_scale * w_scale[n_wscale == 1 ? 0 : k]) / y_scale : 0.0f;
}

// S: stride when it is 1 or 2 (the input patch of a position -- or of a 2x2 pooling window -- then has a fixed size
// and is fetched with independent, clamped, branch-free byte loads that all stay in flight together), 0 = any stride
// (taps fetched one by one under their bounds checks).
template <int C, int S, bool POOL>
__global__ void __launch_bounds__(256)
qconv_smallc_kernel(const uint8_t *__restrict__ x, const uint32_t *__restrict__ wpk, const float *__restrict__ mult,
                    const int32_t *__restrict__ corr, uint8_t *__restrict__ y, ConvGeom g, QConvArgs q, int y_blocked) {
    constexpr int NT = C * 9, ND = (NT + 3) / 4;
    constexpr int NWIN = POOL ? 4 : 1;
    __shared__ uint8_t lut[256];  // the fused activation as a byte table (identity without one)
    lut[threadIdx.x] = q.has_act ? qact_apply(uint8_t(threadIdx.x), q.act) : uint8_t(threadIdx.x);
    __syncthreads();
    const int OHo = POOL ? g.OH / 2 : g.OH, OWo = POOL ? g.OW / 2 : g.OW;
    const int KB = (g.K + 15) >> 4;
    const uint32_t pad_byte = uint32_t(q.x_zp ^ 0x80);
    const int64_t total = int64_t(g.N) * OHo * OWo;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int owo = int(i % OWo);
        const int oho = int((i / OWo) % OHo);
        const int n = int(i / (int64_t(OWo) * OHo));
        uint32_t xs[NWIN][ND];
#pragma unroll
        for (int wd = 0; wd < NWIN; ++wd)
#pragma unroll
            for (int d = 0; d < ND; ++d) xs[wd][d] = 0;
        if constexpr (S > 0) {
            constexpr int PR = (POOL ? S : 0) + 3;  // patch rows = columns
            const int ih0 = (POOL ? 2 * oho : oho) * S - g.pt, iw0 = (POOL ? 2 * owo : owo) * S - g.pl;
            int roff[PR], coff[PR];
            bool rok[PR], cok[PR];
#pragma unroll
            for (int r = 0; r < PR; ++r) {
                const int ih = ih0 + r, iw = iw0 + r;
                rok[r] = ih >= 0 && ih < g.H;
                cok[r] = iw >= 0 && iw < g.W;
                roff[r] = min(max(ih, 0), g.H - 1) * g.W;
                coff[r] = min(max(iw, 0), g.W - 1);
            }
            uint32_t patch[C][PR][PR];
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const uint8_t *xc = x + (int64_t(n) * C + c) * g.H * g.W;
#pragma unroll
                for (int r = 0; r < PR; ++r)
#pragma unroll
                    for (int cc = 0; cc < PR; ++cc) patch[c][r][cc] = xc[roff[r] + coff[cc]];
            }
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int r = 0; r < PR; ++r)
#pragma unroll
                    for (int cc = 0; cc < PR; ++cc) patch[c][r][cc] = (rok[r] && cok[cc]) ? (patch[c][r][cc] ^ 0x80u) : pad_byte;
#pragma unroll
            for (int wd = 0; wd < NWIN; ++wd)
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int c = t / 9, kh = (t % 9) / 3, kw = t % 3;
                    xs[wd][t >> 2] |= patch[c][(wd >> 1) * S + kh][(wd & 1) * S + kw] << (8 * (t & 3));
                }
        } else {
#pragma unroll
            for (int wd = 0; wd < NWIN; ++wd) {
                const int oh = POOL ? 2 * oho + (wd >> 1) : oho, ow = POOL ? 2 * owo + (wd & 1) : owo;
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int c = t / 9, kh = (t % 9) / 3, kw = t % 3;
                    const int ih = oh * g.sh - g.pt + kh, iw = ow * g.sw - g.pl + kw;
                    uint32_t b = pad_byte;
                    if (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W)
                        b = uint32_t(x[((int64_t(n) * C + c) * g.H + ih) * g.W + iw]) ^ 0x80u;
                    xs[wd][t >> 2] |= b << (8 * (t & 3));
                }
            }
        }
        for (int kb = 0; kb < KB; ++kb) {
            uint32_t out[4] = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const int k = kb * 16 + j;  // the tables are padded to a multiple of 16 channels
                const float m = mult[k];
                const int cr = corr[k];
                uint32_t wv[ND];
#pragma unroll
                for (int d = 0; d < ND; ++d) wv[d] = wpk[k * ND + d];
                // requantisation is monotone in the accumulator (increasing for m >= 0), and so is the activation:
                // the pooled byte is the byte of the largest (smallest for m < 0) accumulator of the window
                const bool neg = m < 0.0f;
                int best = INT32_MIN;
#pragma unroll
                for (int wd = 0; wd < NWIN; ++wd) {
                    int acc = cr;
#pragma unroll
                    for (int d = 0; d < ND; ++d) acc = __builtin_amdgcn_sdot4(int(xs[wd][d]), int(wv[d]), acc, false);
                    acc = neg ? -acc : acc;
                    best = acc > best ? acc : best;
                }
                best = neg ? -best : best;
                const uint8_t r = lut[sat_u8_rne_finite(float(best) * m, float(q.y_zp))];
                out[j >> 2] |= uint32_t(r) << (8 * (j & 3));
            }
            if (y_blocked) {
                uint4 *dst = reinterpret_cast<uint4 *>(y) + ((int64_t(n) * KB + kb) * OHo + oho) * OWo + owo;
                *dst = make_uint4(out[0] ^ 0x80808080u, out[1] ^ 0x80808080u, out[2] ^ 0x80808080u, out[3] ^ 0x80808080u);
            } else {
#pragma unroll
                for (int j = 0; j < 16; ++j)
                    if (kb * 16 + j < g.K)
                        y[((int64_t(n) * g.K + kb * 16 + j) * OHo + oho) * OWo + owo] = uint8_t(out[j >> 2] >> (8 * (j & 3)));
            }
        }
    }
}

bool smallc_eligible(const ConvGeom &g) {
    return g.groups == 1 && g.C >= 1 && g.C <= 4 && g.KH == 3 && g.KW == 3 && g.dh == 1 && g.dw == 1;
}

template <int C>
int launch_smallc(zant_ctx *ctx, const uint8_t *x, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *y,
                  const ConvGeom &g, const QConvArgs &q, bool y_blocked, bool pool, zant_pack_slot *slot) {
    constexpr int ND = (C * 9 + 3) / 4;
    const int kpad = ((g.K + 15) / 16) * 16;
    const size_t o_mult = 0, o_corr = align256(size_t(kpad) * 4), o_w = 2 * o_corr, total = o_w + size_t(kpad) * ND * 4;
    void *ws = nullptr, *dyn = nullptr;
    bool need_pack = true;
    int parity = 0;
    const int rc = zant_pack_region(ctx, slot, total, 0, &ws, &dyn, &need_pack, &parity);
    if (rc) return rc;
    char *base = static_cast<char *>(ws);
    float *mult = reinterpret_cast<float *>(base + o_mult);
    int32_t *corr = reinterpret_cast<int32_t *>(base + o_corr);
    uint32_t *wpk = reinterpret_cast<uint32_t *>(base + o_w);
    if (need_pack) {
        hipLaunchKernelGGL(qconv_smallc_pack_kernel<C>, dim3((kpad + 255) / 256), dim3(256), 0, ctx->stream, w, w_scale, bias,
                           wpk, mult, corr, g.K, kpad, q.x_scale, q.y_scale, q.x_zp, q.n_wscale);
        ZANT_LAUNCH_CHECK(ctx);
    }
    const int64_t positions = int64_t(g.N) * (pool ? g.OH / 2 : g.OH) * (pool ? g.OW / 2 : g.OW);
    if (positions * ((g.K + 15) / 16) >= (int64_t(1) << 31)) return 1;  // blocked output units are addressed in 32 bits
    const unsigned blocks = unsigned(std::min<int64_t>(std::max<int64_t>(ceil_div64(positions, 256), 1), int64_t(ctx->num_cus) * 32));
    KernelTimer kt(ctx);
    const int yb = y_blocked ? 1 : 0;
    const int S = (g.sh == g.sw && (g.sh == 1 || g.sh == 2)) ? g.sh : 0;
#define ZANT_SMALLC(SV, PV) hipLaunchKernelGGL((qconv_smallc_kernel<C, SV, PV>), dim3(blocks), dim3(256), 0, ctx->stream, x, wpk, mult, corr, y, g, q, yb)
    if (pool) { if (S == 1) ZANT_SMALLC(1, true); else if (S == 2) ZANT_SMALLC(2, true); else ZANT_SMALLC(0, true); }
    else { if (S == 1) ZANT_SMALLC(1, false); else if (S == 2) ZANT_SMALLC(2, false); else ZANT_SMALLC(0, false); }
#undef ZANT_SMALLC
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// ------------------------------------------------------------------------------------------------------------------
// First layers on the matrix cores (1..4 input channels, 3x3, stride 1 or 2, pads <= 1, NCHW u8 input).
// The GEMM's reduction index is k = (channel, filter row) * 4 + filter column, the fourth column carrying a zero weight:
// 16 consecutive k are then four 4-byte pieces of input rows, each ONE (unaligned) dword load -- the B operand of
// v_mfma_i32_32x32x32_i8 needs no byte gathering at all.  A lane pair (p, 0), (p, 1) holds output position p; a
// wavefront turns 32 positions x 32 output channels per MFMA chain.  With the fused 2x2/2 max pool (stride 1) the four
// window members are four chains over shifted views of the same row dwords, reduced on the accumulators.
// ------------------------------------------------------------------------------------------------------------------
typedef uint32_t __attribute__((aligned(1))) u32_unaligned;

template <int C>
__global__ void __launch_bounds__(256)
qfirst_pack_kernel(const int8_t *__restrict__ w, const float *__restrict__ w_scale, const int32_t *__restrict__ bias,
                   int8_t *__restrict__ wpk, float *__restrict__ mult, int32_t *__restrict__ corr, int K, int kb32, float x_scale,
                   float y_scale, int x_zp, int n_wscale) {
    constexpr int RW = C * 3, NCH = (RW + 7) / 8;
    const int total = kb32 * NCH * 2 * 32 * 16;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        int r = i;
        const int kwi = r & 3; r >>= 2;
        const int j = r & 3; r >>= 2;
        const int kk = r & 31; r >>= 5;
        const int half = r & 1; r >>= 1;
        const int ch = r % NCH, kb = r / NCH;
        const int k = kb * 32 + kk, rw = ch * 8 + half * 4 + j;
        wpk[i] = (k < K && rw < RW && kwi < 3) ? w[(int64_t(k) * C + rw / 3) * 9 + (rw % 3) * 3 + kwi] : int8_t(0);
    }
    for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < kb32 * 32; k += gridDim.x * blockDim.x) {
        int sum = 0;
        if (k < K)
            for (int t = 0; t < C * 9; ++t) sum += int(w[int64_t(k) * C * 9 + t]);
        corr[k] = k < K ? (bias ? bias[k] : 0) + (128 - x_zp) * sum : 0;
        mult[k] = k < K ? (x_scale * w_scale[n_wscale == 1 ? 0 : k]) / y_scale : 0.0f;
    }
}

template <int C, int S, bool POOL, int NV>  // NV: accumulator values per lane that are real channels (8 when K <= 16)
__global__ void __launch_bounds__(256, 2)
qfirst_mfma_kernel(const uint8_t *__restrict__ x, const uint4 *__restrict__ wpk, const float *__restrict__ mult,
                   const int32_t *__restrict__ corr, uint8_t *__restrict__ y, ConvGeom g, QConvArgs q, int y_blocked, int kb32) {
    constexpr int RW = C * 3, NCH = (RW + 7) / 8;
    constexpr int PR = POOL ? 4 : 3, NWIN = POOL ? 4 : 1;
    __shared__ __attribute__((aligned(256))) uint8_t lut[256];  // the fused activation as a byte table, in the byte values the output stores
    lut[threadIdx.x] = uint8_t((q.has_act ? qact_apply(uint8_t(threadIdx.x), q.act) : uint8_t(threadIdx.x)) ^ (y_blocked ? 0x80 : 0));
    __syncthreads();
    const unsigned lut_a = lds_address(lut);  // 256-byte aligned: a converted byte is the low byte of the entry's address
    const int lane = threadIdx.x & 63, l32 = lane & 31, lh = lane >> 5;
    const int OHo = POOL ? g.OH / 2 : g.OH, OWo = POOL ? g.OW / 2 : g.OW;
    const int KB16 = (g.K + 15) >> 4;
    const unsigned per_img = unsigned(OHo) * unsigned(OWo), total = unsigned(g.N) * per_img;  // < 2^31 (host)
    const unsigned n_ptiles = (total + 31u) / 32u;
    const uint32_t padb = uint32_t(q.x_zp ^ 0x80) & 0xffu, pad4 = padb * 0x01010101u;
    const float zpf = float(q.y_zp);
    const unsigned plane_in = unsigned(g.H) * unsigned(g.W), img_in = unsigned(C) * plane_in;  // the input is < 2^32 bytes (host)
    const unsigned wave_id = unsigned(__builtin_amdgcn_readfirstlane(int((blockIdx.x * blockDim.x + threadIdx.x) >> 6)));
    const unsigned n_waves = (gridDim.x * blockDim.x) >> 6;
    i32x16 cvec;
    float mv[16];
    i32x4 wa_all[NCH], wa_dx1[NCH];
    bool tables_loaded = false, any_negative = false;
    // This lane's position in the next tile to load, as (image, row, column) of the (pooled) output.  Successive tiles
    // of a wavefront lie n_waves * 32 positions apart: the triple advances by that step's own (images, rows, columns)
    // with two carries, and is divided out only once.
    // The image is carried as the offset of its first byte in the input and of its first element (blocked: 16-byte
    // unit) in the output, so that no multiplication by the image number is left in the loop (both tensors are below
    // 2^32 bytes: the host checks).
    const unsigned out_img = (y_blocked ? unsigned(KB16) : unsigned(g.K)) * per_img;
    const unsigned in_last = unsigned(g.N - 1) * img_in, out_last = unsigned(g.N - 1) * out_img;
    // (lanes past the end of the last tile are told by the image count itself -- the offsets may wrap there -- and take
    // the last image's)
    unsigned wn, w_in, w_out;
    int woho, wowo;
    {
        const unsigned i = wave_id * 32u + unsigned(l32);
        wn = i / per_img;
        const unsigned rem = i - wn * per_img;
        woho = int(rem / unsigned(OWo));
        wowo = int(rem - unsigned(woho) * unsigned(OWo));
        w_in = wn * img_in;
        w_out = wn * out_img;
    }
    const unsigned step = n_waves * 32u;
    const unsigned d_n = step / per_img, step_r = step - d_n * per_img;
    const int d_oho = int(step_r / unsigned(OWo)), d_owo = int(step_r - unsigned(d_oho) * unsigned(OWo));
    const unsigned d_in = d_n * img_in, d_out = d_n * out_img;
    // The row loads of the NEXT tile are issued before this tile's arithmetic: with two wavefronts per SIMD the load
    // latency would otherwise sit on the critical path of every tile.
    struct TileMeta { unsigned out0; int oho, owo, ih0, sh; bool valid; };  // out0: the image's first output element
    uint32_t raw[C][PR];
    TileMeta nxt;
    auto issue = [&](TileMeta &m) {
        m.valid = wn < unsigned(g.N);           // (only the last tile has lanes past the end: they read image N - 1)
        m.out0 = m.valid ? w_out : out_last;
        m.oho = woho;
        m.owo = wowo;
        m.ih0 = (POOL ? 2 * woho : woho) * S - g.pt;
        const int iw0 = (POOL ? 2 * wowo : wowo) * S - g.pl;
        // one dword per (channel, patch row): columns iw0 .. iw0+3, read from a start clamped into the row
        const int iw0c = min(max(iw0, 0), g.W - 4);
        m.sh = iw0 - iw0c;
        const unsigned base = (m.valid ? w_in : in_last) + unsigned(iw0c);
        unsigned rowoff[PR];
#pragma unroll
        for (int r = 0; r < PR; ++r) rowoff[r] = __umul24(unsigned(min(max(m.ih0 + r, 0), g.H - 1)), unsigned(g.W));  // H, W < 2^24 (host)
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int r = 0; r < PR; ++r)
                raw[c][r] = *reinterpret_cast<const u32_unaligned *>(x + (base + rowoff[r] + unsigned(c) * plane_in));
        wowo += d_owo;
        const int c1 = wowo >= OWo ? 1 : 0;
        wowo -= c1 ? OWo : 0;
        woho += d_oho + c1;
        const bool c2 = woho >= OHo;
        woho -= c2 ? OHo : 0;
        wn += d_n + (c2 ? 1u : 0u);
        w_in += d_in + (c2 ? img_in : 0u);
        w_out += d_out + (c2 ? out_img : 0u);
    };
    if (wave_id < n_ptiles) issue(nxt);
    for (unsigned pt = wave_id; pt < n_ptiles; pt += n_waves) {
        const TileMeta cur = nxt;
        const unsigned out0 = cur.out0;
        const int oho = cur.oho, owo = cur.owo, ih0 = cur.ih0, sh = cur.sh;
        const bool valid = cur.valid;
        // Shifted into place with one byte permute per dword: selector byte b picks data byte b + sh (4 + b + sh in the
        // permute's numbering) or, where that falls outside the dword, a padding byte (0).  A start clamped at the left
        // edge (sh = -1) shifts the row up behind one padding byte, one clamped at the right edge (sh > 0) shifts it down
        // with padding bytes following; a row outside the image is padding altogether.
        const uint32_t sel = sh < 0 ? 0x06050403u : 0x07060504u >> (8 * sh);
        uint32_t row[C][PR];
#pragma unroll
        for (int r = 0; r < PR; ++r) {
            const uint32_t sel_r = unsigned(ih0 + r) < unsigned(g.H) ? sel : 0u;
#pragma unroll
            for (int c = 0; c < C; ++c) row[c][r] = __builtin_amdgcn_perm(raw[c][r] ^ 0x80808080u, pad4, sel_r);
        }
        if (pt + n_waves < n_ptiles) issue(nxt);
        for (int kb = 0; kb < kb32; ++kb) {
            const int kch = kb * 32 + lh * 4;
            if (kb32 > 1 || !tables_loaded) {  // one block of output channels: the tables stay in registers across tiles
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    cvec[v] = corr[kch + (v >> 2) * 8 + (v & 3)];
                    mv[v] = mult[kch + (v >> 2) * 8 + (v & 3)];
                }
#pragma unroll
                for (int ch = 0; ch < NCH; ++ch) {
                    wa_all[ch] = as_i32x4_q(wpk[((kb * NCH + ch) * 2 + lh) * 32 + l32]);
                    // the window member one column to the right reads the same four input columns against the filter
                    // row moved up one byte (columns 1..3 instead of 0..2): the shift is in the weights, once per table
                    // load, instead of in every activation operand
#pragma unroll
                    for (int e = 0; e < 4; ++e) wa_dx1[ch][e] = int(uint32_t(wa_all[ch][e]) << 8);
                }
                any_negative = false;
#pragma unroll
                for (int v = 0; v < NV; ++v) any_negative |= mv[v] < 0.0f;
                any_negative = __builtin_amdgcn_ballot_w64(any_negative) != 0;
                tables_loaded = true;
            }
            i32x16 acc[NWIN];
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch) {
#pragma unroll
                for (int dy = 0; dy < (POOL ? 2 : 1); ++dy) {
                    i32x4 b;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        // reduction rows ch*8 + j (lanes (p, 0)) and ch*8 + 4 + j (lanes (p, 1)): (channel, filter row)
                        const int ra = ch * 8 + j, rb = ch * 8 + 4 + j;
                        const uint32_t va = ra < RW ? row[ra / 3][ra % 3 + dy] : 0u;
                        const uint32_t vb = rb < RW ? row[rb / 3][rb % 3 + dy] : 0u;
                        b[j] = int(lh ? vb : va);
                    }
#pragma unroll
                    for (int dx = 0; dx < (POOL ? 2 : 1); ++dx) {
                        const int wd = dy * 2 + dx;
                        acc[wd] = __builtin_amdgcn_mfma_i32_32x32x32_i8(dx ? wa_dx1[ch] : wa_all[ch], b, ch == 0 ? cvec : acc[wd], 0, 0, 0);
                    }
                }
            }
            if (POOL) {
                // requantisation and the activation keep (multiplier >= 0) or reverse (< 0) the order of the accumulators;
                // scales are positive in practice, and then the minima are never computed
                if (!any_negative) {
#pragma unroll
                    for (int v = 0; v < NV; ++v) acc[0][v] = max(max(acc[0][v], acc[1][v]), max(acc[2][v], acc[3][v]));
                } else {
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        const int a0 = acc[0][v], a1 = acc[1][v], a2 = acc[2][v], a3 = acc[3][v];
                        const int mx = max(max(a0, a1), max(a2, a3)), mn = min(min(a0, a1), min(a2, a3));
                        acc[0][v] = mv[v] >= 0.0f ? mx : mn;
                    }
                }
            }
            // the table lookups of the tile as one batch behind one wait
            uint32_t d[4];
            qb_requant_lookup<NV / 4>(acc[0], mv, zpf, lut_a, d);
            if (y_blocked) {
                // the half-wave swap leaves lane (p, 0) with the 16 bytes of the first block of 16 channels of its
                // position and lane (p, 1) with those of the second: one 16-byte store per lane
                const auto s0 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
                i32x4 out;
                out[0] = int(s0[0]); out[1] = int(s0[1]); out[2] = int(s1[0]); out[3] = int(s1[1]);
                const int cbq = kb * 2 + lh;
                if (valid && cbq < KB16) {
                    const unsigned off = out0 + unsigned(cbq) * per_img + __umul24(unsigned(oho), unsigned(OWo)) + unsigned(owo);
                    *reinterpret_cast<i32x4 *>(y + size_t(off) * 16) = out;
                }
            } else if (valid) {
                // channel kch of the position; the lane's other channels are whole planes further on
                const unsigned pos = out0 + __umul24(unsigned(oho), unsigned(OWo)) + unsigned(owo) + unsigned(kch) * per_img;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int dk = (v >> 2) * 8 + (v & 3);
                    if (kch + dk < g.K) y[pos + unsigned(dk) * per_img] = uint8_t(d[v >> 2] >> (8 * (v & 3)));
                }
            }
        }
    }
}

bool qfirst_eligible(const ConvGeom &g, bool pool) {
    const int S = (g.sh == g.sw && (g.sh == 1 || g.sh == 2)) ? g.sh : 0;
    if (S == 0 || (pool && S != 1) || g.W < 4 || g.pl > 1 || g.pt > 1) return false;
    // the rightmost patch may hang over the row by at most three columns (it is read from a clamped start)
    const int last = ((pool ? (g.OW / 2) * 2 : g.OW) - 1) * S - g.pl;
    if (last + 3 - (g.W - 1) > 3) return false;
    const int64_t OHo = pool ? g.OH / 2 : g.OH, OWo = pool ? g.OW / 2 : g.OW;
    // input offsets are formed in 32 bits, row offsets with a 24-bit multiply
    if (int64_t(g.N) * g.C * g.H * g.W >= (int64_t(1) << 32) - 64 || g.H >= (1 << 24) || g.W >= (1 << 24)) return false;
    // ... and so are output offsets (NCHW: bytes; blocked: 16-byte units of 16-channel blocks)
    if (int64_t(g.N) * (int64_t(g.K + 15) / 16 * 16) * g.OH * g.OW >= (int64_t(1) << 32)) return false;
    return OHo >= 1 && OWo >= 1 && int64_t(g.N) * OHo * OWo < (int64_t(1) << 31) - 64 && OHo * OWo < (1 << 20);
}

template <int C>
int launch_qfirst(zant_ctx *ctx, const uint8_t *x, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *y,
                  const ConvGeom &g, const QConvArgs &q, bool y_blocked, bool pool, zant_pack_slot *slot) {
    constexpr int RW = C * 3, NCH = (RW + 7) / 8;
    const int kb32 = (g.K + 31) / 32;
    const size_t o_mult = 0, o_corr = align256(size_t(kb32) * 32 * 4), o_w = 2 * o_corr, w_bytes = size_t(kb32) * NCH * 2 * 32 * 16;
    void *ws = nullptr, *dyn = nullptr;
    bool need_pack = true;
    int parity = 0;
    const int rc = zant_pack_region(ctx, slot, o_w + w_bytes, 0, &ws, &dyn, &need_pack, &parity);
    if (rc) return rc;
    char *base = static_cast<char *>(ws);
    float *mult = reinterpret_cast<float *>(base + o_mult);
    int32_t *corr = reinterpret_cast<int32_t *>(base + o_corr);
    int8_t *wpk = reinterpret_cast<int8_t *>(base + o_w);
    if (need_pack) {
        hipLaunchKernelGGL(qfirst_pack_kernel<C>, dim3(unsigned(std::min<size_t>((w_bytes + 255) / 256, 256))), dim3(256), 0,
                           ctx->stream, w, w_scale, bias, wpk, mult, corr, g.K, kb32, q.x_scale, q.y_scale, q.x_zp, q.n_wscale);
        ZANT_LAUNCH_CHECK(ctx);
    }
    const int64_t positions = int64_t(g.N) * (pool ? g.OH / 2 : g.OH) * (pool ? g.OW / 2 : g.OW);
    if (positions * ((g.K + 15) / 16) >= (int64_t(1) << 31)) return 1;  // blocked output units are addressed in 32 bits
    // One resident generation of workgroups walks all the tiles: a workgroup's set-up (the activation table, the
    // weights and tables of its channel block) is paid once per wave slot, not once per two tiles.
    const int yb = y_blocked ? 1 : 0;
    KernelTimer kt(ctx);
#define ZANT_QFIRST_NV(SV, PV, NVV)                                                                                         \
    do {                                                                                                                    \
        static int per_cu = 0;                                                                                              \
        if (!per_cu && hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, qfirst_mfma_kernel<C, SV, PV, NVV>, 256, 0) != hipSuccess) \
            per_cu = 2;                                                                                                     \
        const unsigned blocks = unsigned(std::min<int64_t>(std::max<int64_t>(ceil_div64(positions, 128), 1),              \
                                                           int64_t(ctx->num_cus) * std::max(per_cu, 1)));                   \
        ZANT_KERNEL_NAME(ctx, "qfirst_mfma_kernel<%d,%d,%s,%d>", C, SV, PV ? "true" : "false", NVV);                        \
        hipLaunchKernelGGL((qfirst_mfma_kernel<C, SV, PV, NVV>), dim3(blocks), dim3(256), 0, ctx->stream, x,               \
                           reinterpret_cast<const uint4 *>(wpk), mult, corr, y, g, q, yb, kb32);                           \
    } while (0)
#define ZANT_QFIRST(SV, PV)                                                                                                 \
    do {                                                                                                                    \
        if (g.K <= 16) ZANT_QFIRST_NV(SV, PV, 8);                                                                           \
        else ZANT_QFIRST_NV(SV, PV, 16);                                                                                    \
    } while (0)
    if (pool) ZANT_QFIRST(1, true);
    else if (g.sh == 1) ZANT_QFIRST(1, false);
    else ZANT_QFIRST(2, false);
#undef ZANT_QFIRST
#undef ZANT_QFIRST_NV
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

int run_qconv_smallc(zant_ctx *ctx, const uint8_t *x, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *y,
                     const ConvGeom &g, const QConvArgs &q, bool y_blocked, bool pool, zant_pack_slot *slot) {
    if (qfirst_eligible(g, pool)) {
        switch (g.C) {
        case 1: return launch_qfirst<1>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
        case 2: return launch_qfirst<2>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
        case 3: return launch_qfirst<3>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
        default: return launch_qfirst<4>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
        }
    }
    switch (g.C) {
    case 1: return launch_smallc<1>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
    case 2: return launch_smallc<2>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
    case 3: return launch_smallc<3>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
    default: return launch_smallc<4>(ctx, x, w, w_scale, bias, y, g, q, y_blocked, pool, slot);
    }
}

// ------------------------------------------------------------------------------------------------------------------
// Depthwise 3x3 on the blocked layout (HBM-bound): one thread per output unit (16 channels of one position): nine
// 16-byte loads, one 16-byte store.  A workgroup works on one channel block, so its weights are wave-uniform: they are
// pre-expanded to one dword per (tap, channel) with the weight in that channel's byte lane and zeros elsewhere, and
// acc[ch] += v_dot4_i32_i8(x_dword, w_dword) picks the channel's byte without any unpacking.
// ------------------------------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
qdw_pack_kernel(const int8_t *__restrict__ w, const float *__restrict__ w_scale, const int32_t *__restrict__ bias,
                uint32_t *__restrict__ wm, float *__restrict__ mult, int32_t *__restrict__ corr, int K, int kpad, float x_scale,
                float y_scale, int x_zp, int n_wscale) {
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= kpad) return;
    int sum = 0;
    const int cb = k >> 4, qd = (k >> 2) & 3, j = k & 3;
    for (int t = 0; t < 9; ++t) {
        const int wv = k < K ? int(w[int64_t(k) * 9 + t]) : 0;
        sum += wv;
        wm[((cb * 4 + qd) * 9 + t) * 4 + j] = uint32_t(uint8_t(wv)) << (8 * j);
    }
    corr[k] = k < K ? (bias ? bias[k] : 0) + (128 - x_zp) * sum : 0;
    mult[k] = k < K ? (x_scale * w_scale[n_wscale == 1 ? 0 : k]) / y_scale : 0.0f;
}

__global__ void __launch_bounds__(256)
qdw3x3_blocked_kernel(const uint4 *__restrict__ x, const uint32_t *__restrict__ wm, const float *__restrict__ mult,
                      const int32_t *__restrict__ corr, uint4 *__restrict__ y, ConvGeom g, QConvArgs q, int CB,
                      int blocks_per_cb) {
    __shared__ uint8_t lut[256];
    lut[threadIdx.x] = uint8_t((q.has_act ? qact_apply(uint8_t(threadIdx.x), q.act) : uint8_t(threadIdx.x)) ^ 0x80);
    __syncthreads();
    const int cb = blockIdx.x / blocks_per_cb, blk = blockIdx.x - cb * blocks_per_cb;
    const int64_t per_cb = int64_t(g.N) * g.OH * g.OW;
    const uint32_t pad4 = uint32_t(q.x_zp ^ 0x80) * 0x01010101u;
    const uint32_t *wcb = wm + cb * 144;
    for (int64_t i = int64_t(blk) * 256 + threadIdx.x; i < per_cb; i += int64_t(blocks_per_cb) * 256) {
        const int ow = int(i % g.OW);
        const int oh = int((i / g.OW) % g.OH);
        const int64_t n = i / (int64_t(g.OW) * g.OH);
        const uint4 *xp = x + (n * CB + cb) * int64_t(g.H) * g.W;
        uint4 xv[9];
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int ih = oh * g.sh - g.pt + t / 3, iw = ow * g.sw - g.pl + t % 3;
            xv[t] = (ih >= 0 && ih < g.H && iw >= 0 && iw < g.W) ? xp[ih * g.W + iw] : make_uint4(pad4, pad4, pad4, pad4);
        }
        uint32_t out[4];
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) {
            int acc[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = corr[cb * 16 + qd * 4 + j];
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                const uint32_t xd = qd == 0 ? xv[t].x : qd == 1 ? xv[t].y : qd == 2 ? xv[t].z : xv[t].w;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[j] = __builtin_amdgcn_sdot4(int(xd), int(wcb[(qd * 9 + t) * 4 + j]), acc[j], false);
            }
            uint32_t o = 0;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                o |= uint32_t(lut[sat_u8_rne_finite(float(acc[j]) * mult[cb * 16 + qd * 4 + j], float(q.y_zp))]) << (8 * j);
            out[qd] = o;
        }
        y[((n * CB + cb) * g.OH + oh) * int64_t(g.OW) + ow] = make_uint4(out[0], out[1], out[2], out[3]);
    }
}

// The same on the int8 matrix cores.  A wavefront takes 32 output positions x 32 channels (two channel blocks): lane
// (p, h) loads the nine 16-byte taps of position p in channel block h -- exactly the B operand of
// v_mfma_i32_32x32x32_i8 -- and multiplies them by nine DIAGONAL 32x32 weight matrices (row c holds tap t's weight of
// channel c in column c), built once per workgroup in registers.  1/32 of the multiplies are useful, yet nine MFMAs
// replace 144 dot instructions per lane, which is what bounded the VALU version.  The accumulators come out as 16
// channels of one position per lane, requantised and stored like the dense kernel's blocked epilogue.
// ROWS = 2 (stride 1): a lane computes two vertically adjacent outputs from a 4 x 3 patch -- twelve loads instead of
// eighteen, one index decode, and two independent accumulator chains whose MFMAs interleave.
template <int ROWS>
__global__ void __launch_bounds__(256)
qdw3x3_mfma_kernel(const uint4 *__restrict__ x, const uint32_t *__restrict__ wm, const float *__restrict__ mult,
                   const int32_t *__restrict__ corr, uint8_t *__restrict__ y, ConvGeom g, QConvArgs q, int CB,
                   int blocks_per_pair) {
    __shared__ __attribute__((aligned(256))) uint8_t lut[256];
    lut[threadIdx.x] = uint8_t((q.has_act ? qact_apply(uint8_t(threadIdx.x), q.act) : uint8_t(threadIdx.x)) ^ 0x80);
    __syncthreads();
    const unsigned lut_a = lds_address(lut);  // 256-aligned: a converted byte is the low byte of the entry's address
    const int pair = blockIdx.x / blocks_per_pair;
    int blk = blockIdx.x - pair * blocks_per_pair;
    // Consecutive workgroup ids run on different XCDs, each with an L2 of its own, while consecutive tiles share input rows
    // (a tile's patch overlaps the row group above and below it).  With a multiple of 8 workgroups per pair, XCD j takes
    // the j-th eighth of the workgroup order, so that neighbouring tiles meet in one L2: on 1024 x 96 x 48 x 48 the kernel
    // fetched 322 MB for its 226 MB input with the round-robin order and fetches 230 MB with this one.
    if ((blocks_per_pair & 7) == 0) blk = (blk & 7) * (blocks_per_pair >> 3) + (blk >> 3);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6)), l32 = lane & 31, lh = lane >> 5;
    const int cb = 2 * pair + lh;
    const bool cb_ok = cb < CB;
    i32x4 a[9];
    {
        const int k = pair * 32 + l32, kcb = k >> 4, qd = (k >> 2) & 3, j = k & 3;
        const bool mine = (l32 >> 4) == lh;  // the diagonal element of row l32 lies in this lane's half of the columns
#pragma unroll
        for (int t = 0; t < 9; ++t) {
            const int wv = mine ? int(wm[((kcb * 4 + qd) * 9 + t) * 4 + j]) : 0;
            a[t][0] = qd == 0 ? wv : 0;
            a[t][1] = qd == 1 ? wv : 0;
            a[t][2] = qd == 2 ? wv : 0;
            a[t][3] = qd == 3 ? wv : 0;
        }
    }
    float mv[16];
    i32x16 cvec;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int k = pair * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
        mv[v] = mult[k];
        cvec[v] = corr[k];
    }
    // positions are (image, row group, column): a row group is ROWS output rows
    const int OHG = (g.OH + ROWS - 1) / ROWS;
    const unsigned total = unsigned(g.N) * unsigned(OHG) * unsigned(g.OW);  // < 2^31 (checked by the host)
    const unsigned n_ptiles = (total + 31u) / 32u;
    const unsigned per_img = unsigned(OHG) * unsigned(g.OW);                 // < 2^20 (checked by the host)
    const uint32_t pad4 = uint32_t(q.x_zp ^ 0x80) * 0x01010101u;
    const float zpf = float(q.y_zp);
    const char *xbytes = reinterpret_cast<const char *>(x);  // the whole tensor is < 4 GB (checked by the host)
    const unsigned plane = unsigned(g.H) * unsigned(g.W);
    constexpr int PR = ROWS + 2;  // input rows of the patch (ROWS = 2 implies stride 1)
    // This lane's position in the wave's next tile as (image, row group, column).  A wave's tiles lie a fixed number
    // of positions apart, so the triple advances by that step's own triple with two carries; it is divided out once.
    const unsigned pt_first = unsigned(blk) * 4u + unsigned(wave), pt_step = unsigned(blocks_per_pair) * 4u;
    // The image is carried as its first 16-byte unit in the input and in the output (both tensors are < 4 GB: the host
    // checks), so that no multiplication by the image number is left in the loop.
    const unsigned in_img = unsigned(CB) * plane, out_img = unsigned(CB) * unsigned(g.OH) * unsigned(g.OW);
    const unsigned in_last = unsigned(g.N - 1) * in_img, out_last = unsigned(g.N - 1) * out_img;
    // (lanes past the end of the last tile are told by the image count itself -- the offsets may wrap there -- and take
    // the last image's)
    unsigned wn, w_in, w_out;
    int wohg, wow;
    {
        const unsigned i = pt_first * 32u + unsigned(l32);
        wn = i / per_img;
        const unsigned rem = i - wn * per_img;
        wohg = int(rem / unsigned(g.OW));
        wow = int(rem - unsigned(wohg) * unsigned(g.OW));
        w_in = wn * in_img;
        w_out = wn * out_img;
    }
    const unsigned step = pt_step * 32u;
    const unsigned d_n = step / per_img, step_r = step - d_n * per_img;
    const int d_ohg = int(step_r / unsigned(g.OW)), d_ow = int(step_r - unsigned(d_ohg) * unsigned(g.OW));
    const unsigned d_in = d_n * in_img, d_out = d_n * out_img;
    const unsigned cb_in = unsigned(cb_ok ? cb : 0) * plane;                      // this lane's channel block inside an image
    const unsigned out_plane = unsigned(g.OH) * unsigned(g.OW);
    for (unsigned pt = pt_first; pt < n_ptiles; pt += pt_step) {
        const bool valid = wn < unsigned(g.N);  // (only the last tile has lanes past the end: they compute image N - 1 again)
        const unsigned n_in = valid ? w_in : in_last, n_out = valid ? w_out : out_last;
        const int ohg = wohg, ow = wow;
        {
            wow += d_ow;
            const int c1 = wow >= g.OW ? 1 : 0;
            wow -= c1 ? g.OW : 0;
            wohg += d_ohg + c1;
            const bool c2 = wohg >= OHG;
            wohg -= c2 ? OHG : 0;
            wn += d_n + (c2 ? 1u : 0u);
            w_in += d_in + (c2 ? in_img : 0u);
            w_out += d_out + (c2 ? out_img : 0u);
        }
        const int oh = ohg * ROWS;
        // Every tap is loaded from an address inside the tensor (a tap outside the image reads its clamped neighbour)
        // and replaced by the padding vector afterwards: no divergent control flow around the loads.
        const int ih0 = oh * g.sh - g.pt, iw0 = ow * g.sw - g.pl;  // top-left tap
        const unsigned base = (n_in + cb_in) * 16u;
        bool rv[PR], cvd[3];
        unsigned rowb[PR], colb[3];
#pragma unroll
        for (int k = 0; k < PR; ++k) {
            const int ih = ih0 + k;
            rv[k] = cb_ok && unsigned(ih) < unsigned(g.H);
            rowb[k] = base + __umul24(unsigned(min(max(ih, 0), g.H - 1)), unsigned(g.W) * 16u);  // H, W * 16 < 2^24 (host)
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const int iw = iw0 + k;
            cvd[k] = unsigned(iw) < unsigned(g.W);
            colb[k] = unsigned(min(max(iw, 0), g.W - 1)) * 16u;
        }
        uint4 xv[PR * 3];
#pragma unroll
        for (int t = 0; t < PR * 3; ++t) xv[t] = *reinterpret_cast<const uint4 *>(xbytes + (rowb[t / 3] + colb[t % 3]));
        // Only tiles that touch an image border (or the tail of the channel blocks) replace taps by the padding vector:
        // a wave-uniform branch keeps the selects out of the interior tiles.
        const bool inner = rv[0] && rv[PR - 1] && cvd[0] && cvd[2];
        if (__builtin_amdgcn_ballot_w64(!inner) != 0) {
#pragma unroll
            for (int t = 0; t < PR * 3; ++t) {
                const bool ok = rv[t / 3] && cvd[t % 3];
                xv[t].x = ok ? xv[t].x : pad4; xv[t].y = ok ? xv[t].y : pad4;
                xv[t].z = ok ? xv[t].z : pad4; xv[t].w = ok ? xv[t].w : pad4;
            }
        }
        i32x16 acc[ROWS];
#pragma unroll
        for (int t = 0; t < 9; ++t)
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const uint4 &xt = xv[t + 3 * r];  // output row r reads patch rows r .. r + 2
                i32x4 b;
                b[0] = int(xt.x); b[1] = int(xt.y); b[2] = int(xt.z); b[3] = int(xt.w);
                acc[r] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[t], b, t == 0 ? cvec : acc[r], 0, 0, 0);
            }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            uint32_t d[4];
            if (q.has_act) {
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    uint32_t o = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        o |= requant_lookup(float(acc[r][gq * 4 + e]) * mv[gq * 4 + e], zpf, lut_a) << (8 * e);
                    d[gq] = o;
                }
            } else {
                // no activation: the saturating conversion packs the four bytes of a dword itself
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    uint32_t w4 = 0;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        w4 = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[r][gq * 4 + e]) * mv[gq * 4 + e]) + zpf, unsigned(e), w4);
                    d[gq] = w4 ^ 0x80808080u;
                }
            }
            // lanes p and p + 32 exchange one dword per channel block so that each stores 8 consecutive bytes
            // (the half-wave swap: the lower lane ends up with dword 2b of both lanes, the upper lane with dword 2b + 1)
            const bool row_ok = valid && oh + r < g.OH;
            const unsigned pos = n_out + __umul24(unsigned(oh + r), unsigned(g.OW)) + unsigned(ow);  // unit inside channel block 0
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const auto sw = __builtin_amdgcn_permlane32_swap(d[2 * b], d[2 * b + 1], false, false);
                const int cbo = 2 * pair + b;
                if (row_ok && cbo < CB)
                    *reinterpret_cast<uint2 *>(y + ((pos + unsigned(cbo) * out_plane) * 16u + unsigned(lh) * 8u)) = make_uint2(sw[0], sw[1]);
            }
        }
    }
}

bool dw_eligible(const ConvGeom &g) {
    return g.groups == g.C && g.K == g.C && g.CG == 1 && g.KH == 3 && g.KW == 3 && g.dh == 1 && g.dw == 1;
}

size_t qdw_table_bytes(int C) {
    const int CB = ((C + 31) / 32) * 2;  // the matrix-core kernel works on pairs of channel blocks
    return 2 * align256(size_t(CB) * 64) + size_t(CB) * 144 * 4;
}

// x, y blocked; `tables` holds qdw_table_bytes(C) bytes that are (re)filled when need_pack is set.
int run_qdw_blocked(zant_ctx *ctx, const uint8_t *xb, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *yb,
                    const ConvGeom &g, const QConvArgs &q, void *tables, bool need_pack) {
    const int CB = (g.C + 15) / 16, n_pairs = (CB + 1) / 2, kpad = n_pairs * 32;
    const size_t o_corr = align256(size_t(kpad) * 4), o_w = 2 * o_corr;
    char *base = static_cast<char *>(tables);
    float *mult = reinterpret_cast<float *>(base);
    int32_t *corr = reinterpret_cast<int32_t *>(base + o_corr);
    uint32_t *wm = reinterpret_cast<uint32_t *>(base + o_w);
    if (need_pack) {
        hipLaunchKernelGGL(qdw_pack_kernel, dim3((kpad + 255) / 256), dim3(256), 0, ctx->stream, w, w_scale, bias, wm, mult,
                           corr, g.K, kpad, q.x_scale, q.y_scale, q.x_zp, q.n_wscale);
        ZANT_LAUNCH_CHECK(ctx);
    }
    const int64_t per_cb = int64_t(g.N) * g.OH * g.OW;
    KernelTimer kt(ctx);
    if (per_cb < (int64_t(1) << 31) - 64 && int64_t(g.OH) * g.OW < (1 << 20) &&
        int64_t(g.N) * CB * g.H * g.W * 16 < (int64_t(1) << 32) && int64_t(g.N) * CB * g.OH * g.OW * 16 < (int64_t(1) << 32) &&
        g.H < (1 << 24) && g.W < (1 << 20) && g.OH < (1 << 24) && g.OW < (1 << 24)) {
        ZANT_KERNEL_NAME(ctx, "qdw3x3_mfma_kernel<%d>", (g.sh == 1 && g.sw == 1 && g.OH >= 2) ? 2 : 1);
        // one resident generation of workgroups (three share a CU at this kernel's register count): a workgroup's
        // set-up -- the activation table, the nine diagonal operands, the tables -- is paid once per wave slot
        static int per_cu[2] = {0, 0};
        const int rows2 = (g.sh == 1 && g.sw == 1 && g.OH >= 2) ? 1 : 0;
        if (!per_cu[rows2]) {
            const hipError_t e = rows2 ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[1], qdw3x3_mfma_kernel<2>, 256, 0)
                                       : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[0], qdw3x3_mfma_kernel<1>, 256, 0);
            if (e != hipSuccess || per_cu[rows2] < 1) per_cu[rows2] = 2;
        }
        const int64_t want = std::max<int64_t>(1, (int64_t(ctx->num_cus) * per_cu[rows2] + n_pairs - 1) / n_pairs);
        int blocks_per_pair = int(std::min<int64_t>(std::max<int64_t>(ceil_div64(per_cb, 128), 1), want));
        if (blocks_per_pair > 8) blocks_per_pair &= ~7;  // a multiple of 8: the kernel then gives every XCD a contiguous run of tiles
        if (g.sh == 1 && g.sw == 1 && g.OH >= 2)
            hipLaunchKernelGGL(qdw3x3_mfma_kernel<2>, dim3(unsigned(n_pairs) * blocks_per_pair), dim3(256), 0, ctx->stream,
                               reinterpret_cast<const uint4 *>(xb), wm, mult, corr, yb, g, q, CB, blocks_per_pair);
        else
            hipLaunchKernelGGL(qdw3x3_mfma_kernel<1>, dim3(unsigned(n_pairs) * blocks_per_pair), dim3(256), 0, ctx->stream,
                               reinterpret_cast<const uint4 *>(xb), wm, mult, corr, yb, g, q, CB, blocks_per_pair);
    } else {
        const int64_t want = std::max<int64_t>(1, (int64_t(ctx->num_cus) * 16 + CB - 1) / CB);
        const int blocks_per_cb = int(std::min<int64_t>(std::max<int64_t>(ceil_div64(per_cb, 256), 1), want));
        hipLaunchKernelGGL(qdw3x3_blocked_kernel, dim3(unsigned(CB) * blocks_per_cb), dim3(256), 0, ctx->stream,
                           reinterpret_cast<const uint4 *>(xb), wm, mult, corr, reinterpret_cast<uint4 *>(yb), g, q, CB,
                           blocks_per_cb);
    }
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

}  // namespace

int zant_qpack_dense(zant_ctx *ctx, const int8_t *w, const float *w_scale, int64_t n_wscale, const int32_t *bias, int K, int C,
                     int T, int k_blk, float x_scale, int x_zp, float y_scale, int8_t *wp, float *mult, int32_t *corr,
                     int8_t *padvec) {
    const int n_chunks = (C + QCC - 1) / QCC, n_kblocks = (K + k_blk - 1) / k_blk;
    const int64_t wp_bytes = int64_t(n_chunks) * n_kblocks * T * QCC * k_blk, kpad = int64_t(n_kblocks) * k_blk;
    const unsigned pb = unsigned(std::min<int64_t>(std::max<int64_t>(ceil_div64(wp_bytes, 256), ceil_div64(kpad, 4)), 1024));
    hipLaunchKernelGGL(qpack_kernel, dim3(pb), dim3(256), 0, ctx->stream, w, w_scale, bias, wp, mult, corr, padvec,
                       K, C, T, n_chunks, n_kblocks, k_blk, x_scale, y_scale, x_zp, int(n_wscale), 0, C);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

int zant_qpack_depthwise(zant_ctx *ctx, const int8_t *w, const float *w_scale, int64_t n_wscale, const int32_t *bias, int K,
                         int kpad, float x_scale, int x_zp, float y_scale, uint32_t *wm, float *mult, int32_t *corr) {
    hipLaunchKernelGGL(qdw_pack_kernel, dim3((kpad + 255) / 256), dim3(256), 0, ctx->stream, w, w_scale, bias, wm, mult, corr, K,
                       kpad, x_scale, y_scale, x_zp, int(n_wscale));
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

int zant_to_blocked(zant_ctx *ctx, const uint8_t *x, int64_t N, int64_t C, int64_t HW, uint8_t *xb) {
    if (!ctx) return ZANT_NullPointer;
    if (N <= 0 || C <= 0 || HW <= 0) return ZANT_OK;
    if (!x || !xb) return ZANT_NullPointer;
    const int64_t CB = (C + 15) / 16;
    const int vec_ok = (HW % 4 == 0) && (reinterpret_cast<uintptr_t>(x) % 4 == 0);
    KernelTimer kt(ctx);
    const int64_t quads = N * CB * (HW / 4);  // (16-byte units of the blocked tensor, four at a time)
    if (vec_ok && quads < (int64_t(1) << 29))
        hipLaunchKernelGGL(to_blocked_s8_quads_kernel, dim3(unsigned((quads + 63) / 64)), dim3(256), 0, ctx->stream, x,
                           reinterpret_cast<uint4 *>(xb), unsigned(quads), int(C), unsigned(CB), unsigned(HW / 4));
    else
        hipLaunchKernelGGL(to_blocked_s8_kernel, dim3(to_blocked_grid(ctx, N, CB, HW)), dim3(256), 0, ctx->stream, x,
                           reinterpret_cast<uint4 *>(xb), int(N), int(C), int(CB), HW, vec_ok);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// fuse_pool (internal callers only): ydim is the 2x2/2 max-pooled shape; the first-layer kernel and the matrix-core
// kernel (blocked tensors on both sides) take it.
int zant_qlinearconv_layout_pool(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale, uint8_t x_zp,
                                 const int8_t *w, const int64_t wdim[4], const float *w_scale, int64_t n_wscale,
                                 const int8_t *w_zp, float y_scale, uint8_t y_zp, const int32_t *bias, uint8_t *y,
                                 const int64_t ydim[4], const int64_t stride[2], const int64_t pads[4], const int64_t dil[2],
                                 int64_t group, int act, float act_alpha, float act_scale, uint8_t act_zp, int x_layout,
                                 int y_layout, int fuse_pool, bool query_only, zant_pack_slot *slot) {
    if (!ctx || !xdim || !wdim || !ydim || !stride || !pads || !dil) return ZANT_NullPointer;
    for (int i = 0; i < 4; ++i)
        if (xdim[i] <= 0 || wdim[i] <= 0 || xdim[i] > INT32_MAX || wdim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    if (stride[0] <= 0 || stride[1] <= 0 || dil[0] <= 0 || dil[1] <= 0) return ZANT_WrongStride;
    if (pads[0] < 0 || pads[1] < 0 || pads[2] < 0 || pads[3] < 0) return ZANT_InvalidPadding;
    const int64_t C = xdim[1], K = wdim[0];
    if (group < 1 || C % group || K % group || C / group != wdim[1]) return ZANT_InvalidDimensions;
    if (n_wscale != 1 && n_wscale != K) return ZANT_InputTensorDimensionMismatch;
    if (act < ZANT_ACT_NONE || act > ZANT_ACT_RELU6) return ZANT_InvalidInput;
    const int64_t dkh = (wdim[2] - 1) * dil[0] + 1, dkw = (wdim[3] - 1) * dil[1] + 1;
    const int64_t PH = xdim[2] + pads[0] + pads[2], PW = xdim[3] + pads[1] + pads[3];
    if (PH < dkh || PW < dkw) return ZANT_InvalidDimensions;
    const int64_t OH = (PH - dkh) / stride[0] + 1, OW = (PW - dkw) / stride[1] + 1;
    const int64_t OHo = fuse_pool ? OH / 2 : OH, OWo = fuse_pool ? OW / 2 : OW;
    if (ydim[0] != xdim[0] || ydim[1] != K || ydim[2] != OHo || ydim[3] != OWo) return ZANT_InvalidDimensions;
    // the i32 accumulator must not overflow: |x - zp| <= 255, |w - wzp| <= 255
    if (wdim[1] * wdim[2] * wdim[3] > (int64_t(1) << 31) / (255 * 255) - 1) return ZANT_InvalidDimensions;

    ConvGeom g;
    g.N = int(xdim[0]); g.C = int(C); g.H = int(xdim[2]); g.W = int(xdim[3]);
    g.K = int(K); g.CG = int(wdim[1]); g.KH = int(wdim[2]); g.KW = int(wdim[3]);
    g.OH = int(OH); g.OW = int(OW);
    g.sh = int(stride[0]); g.sw = int(stride[1]); g.dh = int(dil[0]); g.dw = int(dil[1]);
    g.pt = int(pads[0]); g.pl = int(pads[1]); g.groups = int(group);
    const bool xb = x_layout == ZANT_LAYOUT_BLOCKED16, yb = y_layout == ZANT_LAYOUT_BLOCKED16;
    const bool smallc = w_zp == nullptr && !xb && smallc_eligible(g);
    QConvArgs q;
    q.x_scale = x_scale; q.y_scale = y_scale; q.x_zp = x_zp; q.y_zp = y_zp; q.n_wscale = int(n_wscale);
    q.has_act = act != ZANT_ACT_NONE;
    q.act.act = act; q.act.alpha = act_alpha; q.act.in_scale = y_scale; q.act.in_zp = y_zp;
    q.act.out_scale = act_scale; q.act.out_zp = act_zp;

    // Pooling rides in the first-layer kernel (NCHW input) or in the matrix-core kernel (blocked on both sides).
    const bool pool_mfma = fuse_pool && !smallc && xb && yb && w_zp == nullptr && !dw_eligible(g) && OHo >= 1 && OWo >= 1 &&
                           run_qconv_mfma(ctx, nullptr, nullptr, nullptr, nullptr, nullptr, g, q, true, true, nullptr, true, true) == ZANT_OK;
    if (fuse_pool && !pool_mfma && (!smallc || OHo < 1 || OWo < 1)) return 1;
    if (query_only) return ZANT_OK;
    if (!x || !w || !w_scale || !y) return ZANT_NullPointer;

    if (pool_mfma) return run_qconv_mfma(ctx, x, w, w_scale, bias, y, g, q, true, true, slot, true, false);
    if (smallc) return run_qconv_smallc(ctx, x, w, w_scale, bias, y, g, q, yb, fuse_pool != 0, slot);

    const size_t x_blk = zant_blocked_bytes(xdim), y_blk = zant_blocked_bytes(ydim);
    if (w_zp == nullptr && dw_eligible(g)) {
        // the depthwise kernel works blocked -> blocked; NCHW operands pass through conversions in the workspace
        const size_t o_y = xb ? 0 : align256(x_blk), dyn_bytes = o_y + (yb ? 0 : align256(y_blk));
        void *tables = nullptr, *dyn = nullptr;
        bool need_pack = true;
        int parity = 0;
        int rc = zant_pack_region(ctx, slot, qdw_table_bytes(g.C), dyn_bytes, &tables, &dyn, &need_pack, &parity);
        if (rc) return rc;
        char *base = static_cast<char *>(dyn);
        const uint8_t *xin = x;
        if (!xb) {
            rc = zant_to_blocked(ctx, x, g.N, g.C, int64_t(g.H) * g.W, reinterpret_cast<uint8_t *>(base));
            if (rc) return rc;
            xin = reinterpret_cast<uint8_t *>(base);
        }
        uint8_t *yout = yb ? y : reinterpret_cast<uint8_t *>(base + o_y);
        rc = run_qdw_blocked(ctx, xin, w, w_scale, bias, yout, g, q, tables, need_pack);
        if (rc) return rc;
        return yb ? ZANT_OK : zant_from_blocked(ctx, yout, g.N, g.K, int64_t(g.OH) * g.OW, y);
    }
    if (w_zp == nullptr) {  // a non-zero weight zero point makes the correction position dependent: direct kernel
        const int rc = run_qconv_mfma(ctx, x, w, w_scale, bias, y, g, q, xb, yb, slot);
        if (rc <= 0) return rc;
    }
    // direct kernel: NCHW only; blocked operands pass through conversions in the workspace
    const uint8_t *xin = x;
    uint8_t *yout = y;
    if (xb || yb) {
        const size_t x_n = size_t(g.N) * g.C * g.H * g.W, y_n = size_t(g.N) * g.K * g.OH * g.OW;
        void *ws = nullptr;
        int rc = zant_workspace(ctx, align256(x_n) + y_n, &ws);
        if (rc) return rc;
        if (xb) {
            rc = zant_from_blocked(ctx, x, g.N, g.C, int64_t(g.H) * g.W, static_cast<uint8_t *>(ws));
            if (rc) return rc;
            xin = static_cast<uint8_t *>(ws);
        }
        if (yb) yout = static_cast<uint8_t *>(ws) + align256(x_n);
    }
    const int64_t total = int64_t(g.N) * g.K * g.OH * g.OW;
    int64_t blocks = ceil_div64(total, 256);
    if (blocks > int64_t(ctx->num_cus) * 32) blocks = int64_t(ctx->num_cus) * 32;
    {
        KernelTimer kt(ctx);
        hipLaunchKernelGGL(qconv_direct_kernel, dim3(unsigned(blocks)), dim3(256), 0, ctx->stream, xin, w, w_scale, w_zp, bias,
                           yout, g, q);
        ZANT_LAUNCH_CHECK(ctx);
    }
    return yb ? zant_to_blocked(ctx, yout, g.N, g.K, int64_t(g.OH) * g.OW, y) : ZANT_OK;
}

extern "C" int zant_hip_qlinearconv_u8i8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale,
                                         uint8_t x_zp, const int8_t *w, const int64_t wdim[4], const float *w_scale,
                                         int64_t n_wscale, const int8_t *w_zp, float y_scale, uint8_t y_zp,
                                         const int32_t *bias, uint8_t *y, const int64_t ydim[4], const int64_t stride[2],
                                         const int64_t pads[4], const int64_t dil[2], int64_t group, int act,
                                         float act_alpha, float act_scale, uint8_t act_zp) {
    return zant_qlinearconv_layout_pool(ctx, x, xdim, x_scale, x_zp, w, wdim, w_scale, n_wscale, w_zp, y_scale, y_zp, bias, y,
                                        ydim, stride, pads, dil, group, act, act_alpha, act_scale, act_zp, ZANT_LAYOUT_NCHW,
                                        ZANT_LAYOUT_NCHW, 0, false, nullptr);
}
