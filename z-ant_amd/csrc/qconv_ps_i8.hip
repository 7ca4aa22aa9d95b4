// QLinearConv 3x3 / stride 1 on the int8 matrix cores, patch-stationary form.
//
// One workgroup of eight wavefronts (two per SIMD) owns a tile of NB whole images x TH output rows x all columns and
// ALL output channels.  The tile's input patch (with its halo) is brought to LDS once, for every input channel, and
// stays there; only the weights stream through LDS, one slab of 32 input channels x 9 taps x up to 128 output channels
// per step, through a two-slab ring that the copies of step s + 1 fill while the matrix cores work on step s.
// Compared with staging patch chunk and weight slab per (tile, chunk, output-channel block) step this moves each
// activation into LDS once instead of once per output-channel block, needs one barrier per 9 taps x 32 channels, and
// lets the tile be chosen to fill the GPU exactly ("128 x 128 x 28 x 28, 128 filters": half an image per workgroup =
// 256 tiles on 256 CUs).
//
// Wave w computes two 32-channel blocks (pair w mod pairs, pairs = output channels per pass / 64) for the position
// tiles of group w div pairs; the tile's position tiles of 32 are dealt evenly to the groups.  One activation operand
// feeds two MFMAs, which keeps the LDS read traffic per MFMA low.  Copies go through registers (an ordinary load, an
// LDS write two taps later), two units per thread and tap, in the shadow of the MFMAs; the two waves of a SIMD cover
// each other's waits.
// Arithmetic, operand layout (channel-blocked signed activations, [tap][half][channel][16] weights), zero-point folding
// and the requantisation epilogue are those of qconv_mfma_kernel (qconv_i8.hip).
#include <algorithm>
#include <cstring>

#include "quant_common.h"
#include "quant_layout.h"

namespace {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

constexpr int PS_WAVES = 8;           // wavefronts per workgroup: two per SIMD
constexpr int PS_NT = PS_WAVES * 64;  // threads per workgroup
constexpr int PS_RMAX = 2;            // 16-byte units per thread of one 16-channel block of the patch: P1s / PS_NT
constexpr int PS_MTMAX = 4;           // position tiles per wave (x 2 channel blocks x 16 accumulator registers)
constexpr int PS_RING = 36 * 1024;    // bytes of one slab of the weight ring: 9 taps x 4 KB

struct PsGeom {
    int N, H, W, CB;            // input: images, rows, columns, 16-channel blocks
    int K, KB, OH, OW, pt, pl;  // output channels and 16-channel blocks, output rows / columns, top / left padding
    int NB, TH;                 // images and output rows per tile
    int PH, PW, P1, P1s;        // patch rows / columns / positions; positions rounded up to a multiple of PS_NT
    int n_row_tiles, n_tiles;
    int NC;                     // chunks of 32 input channels
    int NKP, KP;                // output-channel passes and channels per pass (64 or 128)
    int npt;                    // position tiles of 32 per tile
    int kpad;                   // NKP * KP
    int tab_rounds;             // copy rounds of the multiplier and correction tables: ceil(kpad / 2 / PS_NT)
    // NCHW output staged through LDS (PS_OUT_NCHW_ST*): the tile's bytes as [channel of the pass][S_pad] rows, then
    // written out as whole runs of a plane.
    int S_pad;                  // bytes of a staging row: a tile's position tiles x 32, rounded up to 8 x an odd number
    int stage_off;              // staging region, in bytes from the weight ring's start
    int stage_alias;            // it lies over the ring, the slot table and the patch (one tile per workgroup, one pass)
    int out_unit;               // bytes per copy of the write-out: 8 or 4
    // Fused 2x2/2 max pool (PS_OUT_POOL): a tile's positions are numbered window by window (4 consecutive positions =
    // the members of one window), the windows in (image, pooled row, pooled column) order; OH, OW, TH are even.
    int pool;
    int W_pad;                  // windows of a staging row: a tile's position tiles x 8, rounded to an odd multiple of 8
};

__device__ __forceinline__ unsigned ps_lds_addr(const void *p) {
    return unsigned(reinterpret_cast<uintptr_t>((lptr_t) const_cast<void *>(p)));
}
// LDS reads the compiler does not see, so that it inserts no waits of its own for them.  The waits take the values as
// in/out operands so their users stay behind them.
__device__ __forceinline__ uint32_t ps_read_u8(unsigned addr) {
    uint32_t v;
    asm volatile("ds_read_u8 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
__device__ __forceinline__ uint32_t ps_read_b32(unsigned addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
__device__ __forceinline__ void ps_wait16(uint32_t (&v)[16]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                   "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15]));
}
// One 128-bit LDS read at an immediate byte offset from a per-lane address.  ps_operand_ready waits until at most
// `pending` younger LDS operations are outstanding (they complete in order; operations of other kinds that share the
// counter only make the wait stricter) and makes the operand visible to its users only behind that wait.
__device__ __forceinline__ void ps_ds_read128(i32x4 &v, unsigned addr, int imm) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(imm));
}
__device__ __forceinline__ void ps_operand_ready(i32x4 &b, int pending) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(b) : "i"(pending));
}
__device__ __forceinline__ void ps_operands_ready(i32x4 &a0, i32x4 &a1, i32x4 &b, int pending) {
    asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a0), "+v"(a1), "+v"(b) : "i"(pending));
}

// Where this thread's patch units of a tile come from: offset (in 16-byte units) of the unit's position in channel
// block 0 of the blocked input, per round, and which rounds read real data (the others hold the padding vector).
struct PsDesc {
    unsigned off[PS_RMAX];
    unsigned ok;
};

__device__ __forceinline__ void ps_describe(PsDesc &d, const PsGeom &p, int tile) {
    const int ig = tile / p.n_row_tiles;
    const int n0 = ig * p.NB, oh0 = (tile - ig * p.n_row_tiles) * p.TH;
    const int patch_hw = p.PH * p.PW;
    const float inv_patch = 1.0f / float(patch_hw), inv_pw = 1.0f / float(p.PW);
    d.ok = 0;
#pragma unroll
    for (int r = 0; r < PS_RMAX; ++r) {
        d.off[r] = 0;
        if (r * PS_NT < p.P1s) {
            const int e = r * PS_NT + int(threadIdx.x);
            const int img = small_div(e, patch_hw, inv_patch), rem = e - img * patch_hw;
            const int ph = small_div(rem, p.PW, inv_pw), pw = rem - ph * p.PW;
            const int ih = oh0 - p.pt + ph, iw = pw - p.pl, n = n0 + img;
            const bool ok = e < p.P1 && n < p.N && ih >= 0 && ih < p.H && iw >= 0 && iw < p.W;
            d.off[r] = ok ? unsigned((n * p.CB * p.H + ih) * p.W + iw) : 0u;
            d.ok |= ok ? 1u << r : 0u;
        }
    }
}

// One 16-byte unit of the patch: round r, half h of channel chunk c of the tile `d` describes.  Units outside the
// image, past the patch or of a channel block the tensor does not have hold the padding vector.  Loaded into registers
// and written to LDS later (ps_patch_store): an ordinary load issues in a few cycles, where a direct global->LDS copy
// holds the issuing wave for a couple of hundred.
__device__ __forceinline__ u32x4 ps_patch_load(const PsDesc &d, const int8_t *__restrict__ xb, const int8_t *__restrict__ padvec,
                                               const PsGeom &p, int c, int r, int h) {
    const int cb = 2 * c + h;
    const bool ok = ((d.ok >> r) & 1u) && cb < p.CB;
    const int8_t *src = ok ? xb + (size_t(d.off[r]) + size_t(cb) * unsigned(p.H * p.W)) * 16 : padvec;
    return *reinterpret_cast<const u32x4 *>(src);
}
__device__ __forceinline__ void ps_patch_store(char *patch, const PsGeom &p, int c, int r, int h, const u32x4 &v) {
    *reinterpret_cast<u32x4 *>(patch + ((2 * c + h) * p.P1s + r * PS_NT + int(threadIdx.x)) * 16) = v;
}

// The whole patch of one tile straight from an NCHW u8 tensor whose channel count is a multiple of 16 and whose rows are
// whole, aligned dwords (the host checks).  An item is 4 consecutive columns of one input row in
// one block of 16 channels: 16 dword loads (one per channel plane; a wave's 64 items are consecutive dwords of a plane,
// so every load instruction fetches 256 contiguous bytes), a 4 x 4 byte transpose per group of four channels, value ^
// 0x80, and four 16-byte units written to their patch positions.  Positions outside the image (halo columns, rows above
// or below, images past the batch) receive the padding vector in every channel block, as do blocks past the last one.
__device__ __forceinline__ void ps_patch_from_nchw(const int8_t *__restrict__ xn, const int8_t *__restrict__ padvec, char *patch,
                                                   const PsGeom &p, int tile) {
    const int ig = tile / p.n_row_tiles;
    const int n0 = ig * p.NB, oh0 = (tile - ig * p.n_row_tiles) * p.TH;
    const u32x4 pad = *reinterpret_cast<const u32x4 *>(padvec);
    const int CBp = 2 * p.NC, patch_hw = p.PH * p.PW;
    const float inv_patch = 1.0f / float(patch_hw), inv_pw = 1.0f / float(p.PW);
    for (int e = int(threadIdx.x); e < p.P1; e += PS_NT) {
        const int img = small_div(e, patch_hw, inv_patch), rem = e - img * patch_hw;
        const int ph = small_div(rem, p.PW, inv_pw), pw = rem - ph * p.PW;
        const int ih = oh0 - p.pt + ph, iw = pw - p.pl;
        if (n0 + img >= p.N || ih < 0 || ih >= p.H || iw < 0 || iw >= p.W)
            for (int cb = 0; cb < CBp; ++cb) *reinterpret_cast<u32x4 *>(patch + (cb * p.P1s + e) * 16) = pad;
    }
    const int WQ = p.W >> 2, row_items = p.PH * WQ, n_items = p.NB * CBp * row_items;
    const float inv_row_items = 1.0f / float(row_items), inv_wq = 1.0f / float(WQ), inv_cbp = 1.0f / float(CBp);
    const unsigned plane = unsigned(p.H * p.W);
    for (int it = int(threadIdx.x); it < n_items; it += PS_NT) {
        const int ic = small_div(it, row_items, inv_row_items), r2 = it - ic * row_items;  // (image, channel block), (row, quad)
        const int img = small_div(ic, CBp, inv_cbp), cb = ic - img * CBp;
        const int ph = small_div(r2, WQ, inv_wq), k = r2 - ph * WQ;
        const int ih = oh0 - p.pt + ph, n = n0 + img;
        if (n >= p.N || ih < 0 || ih >= p.H) continue;
        char *dst = patch + (cb * p.P1s + (img * p.PH + ph) * p.PW + 4 * k + p.pl) * 16;
        if (cb >= p.CB) {
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) *reinterpret_cast<u32x4 *>(dst + qd * 16) = pad;
            continue;
        }
        const int8_t *src = xn + (size_t(unsigned((n * p.CB + cb) * 16)) * plane + unsigned(ih * p.W + 4 * k));
        uint32_t d[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) d[j] = *reinterpret_cast<const uint32_t *>(src + size_t(j) * plane);
        u32x4 o[4];
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {  // channels 4 g4 .. 4 g4 + 3 -> dword g4 of the four units
            const uint32_t lo01 = __builtin_amdgcn_perm(d[4 * g4 + 1], d[4 * g4], 0x05010400u), hi01 = __builtin_amdgcn_perm(d[4 * g4 + 1], d[4 * g4], 0x07030602u);
            const uint32_t lo23 = __builtin_amdgcn_perm(d[4 * g4 + 3], d[4 * g4 + 2], 0x05010400u), hi23 = __builtin_amdgcn_perm(d[4 * g4 + 3], d[4 * g4 + 2], 0x07030602u);
            o[0][g4] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u) ^ 0x80808080u;
            o[1][g4] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u) ^ 0x80808080u;
            o[2][g4] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u) ^ 0x80808080u;
            o[3][g4] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u) ^ 0x80808080u;
        }
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) *reinterpret_cast<u32x4 *>(dst + qd * 16) = o[qd];
    }
}

// What a thread copies while its wave multiplies: up to 4 units of a patch chunk (of this tile, or chunk 0 of the next)
// and its share of the NEXT step's weight slab: unit wunit of the taps wtap0, wtap0 + wtaps, ...
struct PsStream {
    const int8_t *wsrc;      // this thread's unit in tap 0 of the next step's slab (taps tap_bytes apart)
    char *wdst;              // the same place in the ring slab the next step reads (taps 4 KB apart)
    int tap_bytes;
    int wtap0, wtaps;        // first tap this thread copies, and the stride of its taps
    int pcur;                // the step copies a patch chunk
    char *patch;             // patch base
    int pchunk;              // channel chunk this step's patch copies fill
};

constexpr int PS_PCMAX = 2 * PS_RMAX;  // patch units per thread and chunk
constexpr int PS_WUMAX = 5;            // weight units per thread and step: ceil(9 taps / 2 thread groups)

// The matrix-core work of one step: 9 taps x 32 input channels for this wave's MT position tiles x 2 channel blocks.
// wr: LDS address of this lane's weight operand of tap 0 of the wave's first channel block (the second block 512 bytes
// on, taps 4 KB apart); xbase[i] + chunk_off: LDS address of position slot i's patch entry for tap (0, 0) in this step's
// channel chunk and this lane's half; PW16: bytes of a patch row.  last_slot: position slot MT - 1 holds a tile of
// the wave's group (tiles are dealt evenly, so a wave is normally at most one short; slots below the last are always
// multiplied: an empty one reads a valid address and its sums are dropped).
// The activation operand of slot i for the NEXT tap is read into the same registers right behind slot i's two MFMAs of
// this tap: a rolling pipeline one tap deep in which every read has 2 * MT MFMAs to land and each MFMA pair waits only
// for its own operand.  Filter columns are immediate offsets, filter rows an address increment.
// The copies of PsStream ride along: two units loaded behind the first MFMA pair of each of taps 0..4 and written to
// LDS two taps later.
// FIRST: the step opens a pass: its first tap starts the accumulators from zero (an inline constant of the MFMA).
// SWAP: positions are the MFMA's rows and channels its columns (a lane then holds 16 positions of ONE channel) instead of
// the other way round (16 channels of one position).
template <int MT, bool FIRST, bool SWAP>
__device__ __forceinline__ void ps_mfma_step(unsigned wr, const unsigned (&xbase)[MT], unsigned chunk_off, unsigned PW16, const PsStream &st,
                                             const PsDesc &d, const int8_t *__restrict__ xb, const int8_t *__restrict__ padvec,
                                             const PsGeom &p, i32x16 (&acc)[2][MT], bool last_slot) {
    i32x4 a[2][2], b[MT];  // a[buffer][channel block]
    u32x4 stg[3][2];       // units on their way from global memory to LDS, by tap modulo 3
    unsigned xr[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) xr[i] = xbase[i] + chunk_off;
    ps_ds_read128(a[0][0], wr, 0);
    ps_ds_read128(a[0][1], wr, 512);
#pragma unroll
    for (int i = 0; i < MT; ++i) ps_ds_read128(b[i], xr[i], 0);
    // unit j of the thread's copy list: j < PS_PCMAX: patch unit (round j >> 1, half j & 1); else weight unit j - PS_PCMAX
    auto unit_load = [&](int j, u32x4 &v) {
        if (j < PS_PCMAX) {
            if (st.pcur && (j >> 1) * PS_NT < p.P1s) v = ps_patch_load(d, xb, padvec, p, st.pchunk, j >> 1, j & 1);
        } else if (j < PS_PCMAX + PS_WUMAX) {
            const int tp = st.wtap0 + (j - PS_PCMAX) * st.wtaps;
            if (tp < 9) v = *reinterpret_cast<const u32x4 *>(st.wsrc + tp * st.tap_bytes);
        }
    };
    auto unit_store = [&](int j, const u32x4 &v) {
        if (j < PS_PCMAX) {
            if (st.pcur && (j >> 1) * PS_NT < p.P1s) ps_patch_store(st.patch, p, st.pchunk, j >> 1, j & 1, v);
        } else if (j < PS_PCMAX + PS_WUMAX) {
            const int tp = st.wtap0 + (j - PS_PCMAX) * st.wtaps;
            if (tp < 9) *reinterpret_cast<u32x4 *>(st.wdst + tp * 4096) = v;
        }
    };
    // which position slot of a tap the loads / stores ride behind: loads early, stores late, so that a unit has more
    // than two taps to arrive
    const int i_load = 0, i_store = MT - 1;
#pragma unroll
    for (int t = 0; t < 9; ++t) {
        const int cur = t & 1, nxt = cur ^ 1;
        const int kw1 = (t + 1) % 3;  // filter column of the next tap
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            // younger than this operand: the rest of this tap's, and what was issued for the next tap so far
            // (two weight operands and the activation operands of the slots before this one)
            const int pending = t == 8 ? MT - 1 - i : (i == 0 ? MT - 1 : MT + 1);
            if (i == 0) ps_operands_ready(a[cur][0], a[cur][1], b[i], pending);
            else ps_operand_ready(b[i], pending);
            __builtin_amdgcn_s_setprio(1);
            // (a wave whose last position slot holds no tile of its group skips that slot's MFMAs: wave-uniform)
            if (i < MT - 1 || last_slot)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                if (FIRST && t == 0) {
                    const i32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    acc[j][i] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(b[i], a[cur][j], zero, 0, 0, 0)
                                     : __builtin_amdgcn_mfma_i32_32x32x32_i8(a[cur][j], b[i], zero, 0, 0, 0);
                } else {
                    acc[j][i] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(b[i], a[cur][j], acc[j][i], 0, 0, 0)
                                     : __builtin_amdgcn_mfma_i32_32x32x32_i8(a[cur][j], b[i], acc[j][i], 0, 0, 0);
                }
            }
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            if (i == 0 && t < 8) {
                ps_ds_read128(a[nxt][0], wr, (t + 1) * 4096);
                ps_ds_read128(a[nxt][1], wr, (t + 1) * 4096 + 512);
            }
            if (i == i_load && 2 * t < PS_PCMAX + PS_WUMAX) {
                unit_load(2 * t, stg[t % 3][0]);
                unit_load(2 * t + 1, stg[t % 3][1]);
            }
            if (i == i_store && t >= 2 && 2 * (t - 2) < PS_PCMAX + PS_WUMAX) {
                unit_store(2 * (t - 2), stg[(t - 2) % 3][0]);
                unit_store(2 * (t - 2) + 1, stg[(t - 2) % 3][1]);
            }
            if (t < 8) {
                if (kw1 == 0) xr[i] += PW16;  // the next tap starts a filter row
                ps_ds_read128(b[i], xr[i], kw1 * 16);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// OUT: how the output bytes are formed and stored.
enum { PS_OUT_NCHW_LUT = 0, PS_OUT_BLOCKED_LUT = 1, PS_OUT_BLOCKED = 2, PS_OUT_NCHW = 3, PS_OUT_NCHW_ST = 4, PS_OUT_NCHW_ST_LUT = 5,
       PS_OUT_POOL = 6 };

// Write-out of a staged NCHW tile: rows of the staging region (one per image and channel, `row_bytes` real bytes each)
// go to their runs of the output planes in units of U bytes, consecutive threads on consecutive units.
template <typename U>
__device__ __forceinline__ void ps_write_out(const char *stage, uint8_t *__restrict__ y, const PsGeom &p, int kh, int imgs_here,
                                             int row_bytes, unsigned g_origin, int plane) {
    const int upr = row_bytes / int(sizeof(U)), n_rows = imgs_here * kh, n_units = n_rows * upr;
    const float inv_upr = 1.0f / float(upr), inv_kh = 1.0f / float(kh);
    const int per_img = p.TH * p.OW;
#pragma unroll 4
    for (int u = int(threadIdx.x); u < n_units; u += PS_NT) {
        const int row = small_div(u, upr, inv_upr), off = u - row * upr;
        int img = 0, kk = row;
        if (p.NB > 1) {
            img = small_div(row, kh, inv_kh);
            kk = row - img * kh;
        }
        const U v = *reinterpret_cast<const U *>(stage + kk * p.S_pad + img * per_img + off * int(sizeof(U)));
        *reinterpret_cast<U *>(y + (g_origin + unsigned(img * p.K + kk) * unsigned(plane) + unsigned(off * int(sizeof(U))))) = v;
    }
}

// tabs: the per-channel requantisation multipliers (kpad floats) followed by the integer corrections (kpad ints).
// XN: the input is the caller's NCHW u8 tensor: a tile's whole patch is read and regrouped into 16-channel units by the
// workgroup itself before the tile's first step (ps_patch_from_nchw), instead of streaming chunk by chunk out of a
// blocked copy that a kernel of its own would have to write first.
template <int MT, int OUT, bool XN>
__global__ void __launch_bounds__(PS_NT)
qconv_ps_kernel(const int8_t *__restrict__ xb, const int8_t *__restrict__ wp, const char *__restrict__ tabs,
                const int8_t *__restrict__ padvec, uint8_t *__restrict__ y, PsGeom p, QConvArgs q) {
    constexpr bool pooled = OUT == PS_OUT_POOL;  // blocked output of the 2x2/2 max-pooled result, through the byte table
    constexpr bool y_blocked = OUT == PS_OUT_BLOCKED_LUT || OUT == PS_OUT_BLOCKED || pooled;
    constexpr bool use_lut = OUT == PS_OUT_BLOCKED_LUT || OUT == PS_OUT_NCHW_LUT || OUT == PS_OUT_NCHW_ST_LUT || pooled;
    constexpr bool staged = OUT == PS_OUT_NCHW_ST || OUT == PS_OUT_NCHW_ST_LUT;
    constexpr bool swapped = staged || pooled;  // positions are the accumulators' rows (registers), channels their lanes
    extern __shared__ __attribute__((aligned(256))) char ps_lds_raw[];
    // LDS: [256-byte activation table, 256-aligned][multipliers, corrections][weight ring: 2 slabs][slot table]
    //      [patch: 2*NC blocks x P1s x 16]
    const unsigned lut_a = (ps_lds_addr(ps_lds_raw) + 255u) & ~255u;
    char *lds = ps_lds_raw + (lut_a - ps_lds_addr(ps_lds_raw));
    uint8_t *lut = reinterpret_cast<uint8_t *>(lds);
    char *tab_l = lds + 256;
    char *wring = tab_l + p.tab_rounds * PS_NT * 16;
    int *postab = reinterpret_cast<int *>(wring + 2 * PS_RING);  // [MT][PS_NT]: where each lane's position slots lie
    char *patch = reinterpret_cast<char *>(postab + MT * PS_NT);

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, lh = lane >> 5;
    // wave -> (pair of channel blocks, group of position tiles): KP = 128: two pairs x four groups; KP = 64: one pair x
    // eight groups.  Waves w and w + 4 share a SIMD; with two pairs they hold groups g and g + 2 of one pair.
    const int pairs = p.KP >> 6, NG = PS_WAVES / pairs;
    const int cp = wave % pairs, grp = wave / pairs;
    // position tiles of this wave's group: the tile's npt tiles dealt evenly, the first (npt mod NG) groups one more
    const int base = p.npt / NG, rem = p.npt - base * NG;
    const int mt = base + (grp < rem ? 1 : 0), pt0 = grp * base + min(grp, rem);

    // The activation table first, the table copies after it: an LDS write behind an asynchronous copy waits for it.
    if (use_lut && tid < 256) {
        const uint8_t v = uint8_t(tid);
        lut[tid] = uint8_t((q.has_act ? qact_apply(v, q.act) : v) ^ (y_blocked ? 0x80 : 0));
    }
    const unsigned mult_a = ps_lds_addr(tab_l), corr_a = mult_a + unsigned(p.kpad) * 4u;
    const unsigned postab_a = ps_lds_addr(postab) + unsigned(tid) * 4u;

    const int NS = p.NKP * p.NC;           // steps per tile: (pass, chunk)
    const int tap_bytes = 2 * p.KP * 16;   // packed weights of one tap: [half][KP][16]
    const unsigned PW16 = unsigned(p.PW * 16);
    // The weight ring: two slabs (the step being multiplied, the step being copied) of 9 taps x 4 KB, each tap laid out
    // as in the packed weights.  The threads split a slab: unit wunit of every wtaps-th tap from wtap0.
    const int upt = tap_bytes >> 4;        // 16-byte units per tap: 256 or 128
    PsStream st;
    st.tap_bytes = tap_bytes; st.patch = patch;
    st.wtaps = PS_NT / upt; st.wtap0 = __builtin_amdgcn_readfirstlane(tid / upt);  // wave-uniform: upt is a multiple of 64
    const int wunit = tid - st.wtap0 * upt;
    const unsigned wr0 = ps_lds_addr(wring) + unsigned(lh * p.KP + 2 * cp * 32 + l32) * 16u;  // this lane's operand, tap 0

    int tile = int(blockIdx.x);
    if (tile >= p.n_tiles) return;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the activation table is written
    // the two tables: rounds of 16-byte units straight into LDS; lanes past the end repeat the last unit into padding
    for (int r = 0; r < p.tab_rounds; ++r) {
        const int u = min(r * PS_NT + tid, p.kpad / 2 - 1);
        __builtin_amdgcn_global_load_lds((gptr_t)(tabs + u * 16), (lptr_t)(tab_l + (r * PS_NT + wave * 64) * 16), 16, 0, 0);
    }
    // The first tile's first patch chunk and the weights of step 0 at once.  Everything later is copied by the steps
    // themselves, two units per tap, so that the copy stream never stops.
    PsDesc desc;
    if constexpr (XN) {
        desc.ok = 0;
#pragma unroll
        for (int r = 0; r < PS_RMAX; ++r) desc.off[r] = 0;
    } else {
        ps_describe(desc, p, tile);
    }
    u32x4 pv[PS_RMAX][2], wv[PS_WUMAX];
    if constexpr (!XN) {
#pragma unroll
        for (int r = 0; r < PS_RMAX; ++r)
            if (r * PS_NT < p.P1s) {
                pv[r][0] = ps_patch_load(desc, xb, padvec, p, 0, r, 0);
                pv[r][1] = ps_patch_load(desc, xb, padvec, p, 0, r, 1);
            }
    }
#pragma unroll
    for (int k = 0; k < PS_WUMAX; ++k) {
        const int tp = st.wtap0 + k * st.wtaps;
        if (tp < 9) wv[k] = *reinterpret_cast<const u32x4 *>(wp + wunit * 16 + tp * tap_bytes);
    }
    __builtin_amdgcn_sched_barrier(0);

    // While those loads are in flight: position slot i of this lane: image, row, column inside the tile
    // (image << 20 | row << 10 | column, -1 beyond the tile; kept in LDS for the epilogues) and the LDS address of the
    // slot's patch entry in channel block `lh`.
    unsigned xbase[MT];
    {
        const int per_img = p.TH * p.OW;
        const float inv_per_img = 1.0f / float(per_img), inv_ow = 1.0f / float(p.OW);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int pp = (pt0 + i) * 32 + l32;
            int img, r, c;
            if constexpr (pooled) {
                // window pp / 4 in (image, pooled row, pooled column) order, member pp % 4 = (row, column) inside it
                const int wi = pp >> 2, per_img_w = per_img >> 2, ow2 = p.OW >> 1;
                img = small_div(wi, per_img_w, 4.0f * inv_per_img);
                const int r2 = wi - img * per_img_w;
                const int wr = small_div(r2, ow2, 2.0f * inv_ow);
                r = 2 * wr + ((pp >> 1) & 1);
                c = 2 * (r2 - wr * ow2) + (pp & 1);
            } else {
                img = small_div(pp, per_img, inv_per_img);
                const int r2 = pp - img * per_img;
                r = small_div(r2, p.OW, inv_ow);
                c = r2 - r * p.OW;
            }
            const bool in_tile = i < mt && img < p.NB;
            const int lds_off = in_tile ? (img * p.PH + r) * p.PW + c : 0;
            xbase[i] = ps_lds_addr(patch) + unsigned(lh * p.P1s + lds_off) * 16u;
            postab[i * PS_NT + tid] = in_tile ? (img << 20) | (r << 10) | c : -1;
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (!XN) {
#pragma unroll
        for (int r = 0; r < PS_RMAX; ++r)
            if (r * PS_NT < p.P1s) {
                ps_patch_store(patch, p, 0, r, 0, pv[r][0]);
                ps_patch_store(patch, p, 0, r, 1, pv[r][1]);
            }
    } else {
        ps_patch_from_nchw(xb, padvec, patch, p, tile);
    }
#pragma unroll
    for (int k = 0; k < PS_WUMAX; ++k) {
        const int tp = st.wtap0 + k * st.wtaps;
        if (tp < 9) *reinterpret_cast<u32x4 *>(wring + wunit * 16 + tp * 4096) = wv[k];
    }
    __builtin_amdgcn_sched_barrier(0);

    i32x16 acc[2][MT];
    const bool last_slot = mt == MT;  // wave-uniform: the wave's last position slot holds a tile of its group
    int gs = 0;  // steps done by this workgroup; its parity selects the ring slab a step reads
    while (true) {
        const int next_tile = tile + int(gridDim.x);
        int s = 0;
        for (int kp = 0; kp < p.NKP; ++kp) {
            // One step = (pass kp, chunk c).  At its boundary this thread's copies (LDS writes, and the table copies of
            // the first tile) are done, and everybody has left the previous step.
            auto boundary = [&]() {
                if (gs == 0) __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
                else __builtin_amdgcn_s_waitcnt(0xC07F);           // lgkmcnt(0): output stores may still be on their way
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            };
            // what step s copies: the next step's weights (the first step's after the last), and a patch chunk
            auto plan_copies = [&](int c) {
                const int s1 = s + 1 == NS ? 0 : s + 1;
                st.wsrc = wp + size_t(s1) * 9 * tap_bytes + wunit * 16;
                st.wdst = wring + ((gs + 1) & 1) * PS_RING + wunit * 16;
                st.pcur = 0;
                st.pchunk = 0;
                if constexpr (XN) {
                    // the whole patch is in place before the tile's first step
                } else if (kp == 0 && c + 1 < p.NC) {
                    st.pcur = 1; st.pchunk = c + 1;
                } else if (s + 1 == NS && p.NC > 1 && next_tile < p.n_tiles) {
                    ps_describe(desc, p, next_tile);  // chunk 0 of the next tile: nobody reads that region any more
                    st.pcur = 1;
                }
            };
            {
                boundary();
                plan_copies(0);
                // slots past this wave's tiles multiply patch entry 0; their results are dropped
                ps_mfma_step<MT, true, swapped>(wr0 + unsigned((gs & 1) * PS_RING), xbase, 0u, PW16, st, desc, xb, padvec, p, acc, last_slot);
                ++s; ++gs;
            }
            for (int c = 1; c < p.NC; ++c, ++s, ++gs) {
                boundary();
                plan_copies(c);
                ps_mfma_step<MT, false, swapped>(wr0 + unsigned((gs & 1) * PS_RING), xbase, unsigned(2 * c * p.P1s * 16), PW16, st, desc,
                                        xb, padvec, p, acc, last_slot);
            }

            // ---- end of pass kp: requantisation (+ fused activation), stores ----
            if (!XN && s == NS && p.NC == 1 && next_tile < p.n_tiles) {
                // a single channel chunk cannot be refilled while it is read: the next tile's patch goes in at once,
                // after everybody has left the matrix-core loop, and lands under this epilogue
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                ps_describe(desc, p, next_tile);
#pragma unroll
                for (int r = 0; r < PS_RMAX; ++r)
                    if (r * PS_NT < p.P1s) {
                        ps_patch_store(patch, p, 0, r, 0, ps_patch_load(desc, xb, padvec, p, 0, r, 0));
                        ps_patch_store(patch, p, 0, r, 1, ps_patch_load(desc, xb, padvec, p, 0, r, 1));
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (pooled) {
                // A lane holds 16 positions of ONE channel per accumulator tuple, and registers 4g..4g+3 are the four
                // members of one pooling window.  Requantisation and the activation are monotone in the accumulator
                // (non-decreasing for a multiplier >= 0, non-increasing below), so the pooled byte is the requantised
                // maximum (minimum) of the four sums: one value in four goes through the float sequence.  A 4 x 4 byte
                // transpose across each quad of lanes (= four channels) turns a lane's four window bytes into four
                // channel bytes of one window: a dword of the staging rows [16-channel block][window][16 bytes], which
                // the workgroup then writes out as whole 16-byte units of the pooled blocked tensor.
                const int ig = tile / p.n_row_tiles;
                const int n0 = ig * p.NB, oh0 = (tile - ig * p.n_row_tiles) * p.TH;
                const int rows_here = min(p.TH, p.OH - oh0), imgs_here = min(p.NB, p.N - n0);
                const float zpf = float(q.y_zp);
                char *stage = wring + p.stage_off;
                uint32_t lq = uint32_t(lane);
                asm volatile("" : "+v"(lq));
                uint32_t sel1, sel2;  // sel1 = lane & 1 ? 0x03070105 : 0x06020400, sel2 = lane & 2 ? 0x03020706 : 0x05040100
                asm volatile("v_bfe_i32 %0, %2, 0, 1\n\tv_bfe_i32 %1, %2, 1, 1\n\t"
                             "v_and_b32 %0, 0x05050505, %0\n\tv_and_b32 %1, 0x06060606, %1\n\t"
                             "v_xor_b32 %0, 0x06020400, %0\n\tv_xor_b32 %1, 0x05040100, %1"
                             : "=&v"(sel1), "=&v"(sel2) : "v"(lq));
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int kk = (2 * cp + j) * 32 + l32;  // this lane's channel inside the pass
                    uint32_t mr = ps_read_b32(mult_a + unsigned(kp * p.KP + kk) * 4u), cr = ps_read_b32(corr_a + unsigned(kp * p.KP + kk) * 4u);
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(mr), "+v"(cr));
                    const float mv = __uint_as_float(mr);
                    const int cv = int(cr);
                    const bool up = mv >= 0.0f;
                    // after the transpose this lane holds window (lane & 3) of each group of four windows... of ITS quad's
                    // four channels: the dword at [block kk / 16][window][channel (kk & 12)]
                    char *row = stage + (((kk >> 4) * p.W_pad + pt0 * 8 + int(lq & 3) * 2 + lh) * 16 + (l32 & 12));
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        __builtin_amdgcn_sched_barrier(0);  // one position tile at a time
                        if (i >= mt) continue;              // (wave-uniform) an empty slot's windows belong to another wave
                        uint32_t ob[4];
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq) {
                            const int a0 = acc[j][i][gq * 4], a1 = acc[j][i][gq * 4 + 1], a2 = acc[j][i][gq * 4 + 2], a3 = acc[j][i][gq * 4 + 3];
                            const int hi = max(max(a0, a1), max(a2, a3)), lo = min(min(a0, a1), min(a2, a3));
                            const int sum = (up ? hi : lo) + cv;
                            ob[gq] = ps_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(sum) * mv) + zpf, 0u, lut_a));
                        }
                        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ob[0]), "+v"(ob[1]), "+v"(ob[2]), "+v"(ob[3]));
                        const uint32_t d0 = ob[0] | (ob[1] << 8) | (ob[2] << 16) | (ob[3] << 24);  // byte g: window 2g + lh... of the tile
                        const uint32_t x1 = uint32_t(__builtin_amdgcn_update_dpp(0, int(d0), 0xB1, 0xf, 0xf, false));  // lane ^ 1
                        const uint32_t t1 = __builtin_amdgcn_perm(x1, d0, sel1);
                        const uint32_t x2 = uint32_t(__builtin_amdgcn_update_dpp(0, int(t1), 0x4E, 0xf, 0xf, false));  // lane ^ 2
                        const uint32_t o4 = __builtin_amdgcn_perm(x2, t1, sel2);
                        *reinterpret_cast<uint32_t *>(row + i * 128) = o4;
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                {
                    // write-out: 16-byte units, rows = (image, 16-channel block), a row's windows one run of the pooled plane
                    const int ow2 = p.OW >> 1, per_img_w = (p.TH >> 1) * ow2, here_w = (rows_here >> 1) * ow2;
                    const int kb0 = kp * (p.KP >> 4), kbh = min(p.KP >> 4, p.KB - kb0);
                    const int n_rows = imgs_here * kbh, n_units = n_rows * here_w;
                    const int plane_p = (p.OH >> 1) * ow2;
                    const float inv_w = 1.0f / float(here_w), inv_kbh = 1.0f / float(kbh);
                    const unsigned g_origin = unsigned((n0 * p.KB + kb0) * plane_p + (oh0 >> 1) * ow2);
#pragma unroll 2
                    for (int u = tid; u < n_units; u += PS_NT) {
                        const int rw = small_div(u, here_w, inv_w), off = u - rw * here_w;
                        int img = 0, kbl = rw;
                        if (p.NB > 1) {
                            img = small_div(rw, kbh, inv_kbh);
                            kbl = rw - img * kbh;
                        }
                        const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + (kbl * p.W_pad + img * per_img_w + off) * 16);
                        __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(y) + (g_origin + unsigned((img * p.KB + kbl) * plane_p + off)));
                    }
                }
                // the next pass or tile writes these rows again: not before everybody has read them
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            } else if constexpr (staged) {
                // A lane holds 16 positions of ONE channel per accumulator tuple (registers 4g..4g+3: four consecutive
                // positions of the tile's flattened (image, row, column) order): one multiplier and one correction per
                // lane, a dword of four positions per group with no exchange between lanes.  The dwords go to the
                // staging rows [channel][position]; the workgroup then writes each row's bytes to its plane as one run.
                const int ig = tile / p.n_row_tiles;
                const int n0 = ig * p.NB, oh0 = (tile - ig * p.n_row_tiles) * p.TH;
                const int rows_here = min(p.TH, p.OH - oh0), imgs_here = min(p.NB, p.N - n0);
                const int plane = p.OH * p.OW;
                const float zpf = float(q.y_zp);
                char *stage = wring + p.stage_off;
                if (p.stage_alias) {  // everybody has left the matrix-core loop: ring, slot table and patch are free
                    __builtin_amdgcn_s_waitcnt(0xC07F);
                    __builtin_amdgcn_s_barrier();
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int kk = (2 * cp + j) * 32 + l32;  // this lane's channel inside the pass
                    uint32_t mr = ps_read_b32(mult_a + unsigned(kp * p.KP + kk) * 4u), cr = ps_read_b32(corr_a + unsigned(kp * p.KP + kk) * 4u);
                    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(mr), "+v"(cr));
                    const float mv = __uint_as_float(mr);
                    const int cv = int(cr);
                    char *row = stage + kk * p.S_pad + (pt0 * 32 + lh * 4);
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        __builtin_amdgcn_sched_barrier(0);  // one position tile at a time
                        if (i >= mt) continue;              // (wave-uniform) an empty slot's positions belong to another wave
#pragma unroll
                        for (int gq = 0; gq < 4; ++gq) {
                            uint32_t w4 = 0;
                            if constexpr (use_lut) {
                                uint32_t ob[4];
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    ob[e] = ps_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[j][i][gq * 4 + e] + cv) * mv) + zpf, 0u, lut_a));
                                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ob[0]), "+v"(ob[1]), "+v"(ob[2]), "+v"(ob[3]));
                                w4 = ob[0] | (ob[1] << 8) | (ob[2] << 16) | (ob[3] << 24);
                            } else {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    w4 = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(acc[j][i][gq * 4 + e] + cv) * mv) + zpf, unsigned(e), w4);
                            }
                            *reinterpret_cast<uint32_t *>(row + i * 32 + gq * 8) = w4;
                        }
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                const int kh = min(p.KP, p.K - kp * p.KP);
                const unsigned g_origin = unsigned((n0 * p.K + kp * p.KP) * plane + oh0 * p.OW);
                if (p.out_unit == 8) ps_write_out<uint2>(stage, y, p, kh, imgs_here, rows_here * p.OW, g_origin, plane);
                else ps_write_out<uint32_t>(stage, y, p, kh, imgs_here, rows_here * p.OW, g_origin, plane);
                if (!p.stage_alias) {  // the next pass or tile writes these rows again: not before everybody has read them
                    __builtin_amdgcn_s_waitcnt(0xC07F);
                    __builtin_amdgcn_s_barrier();
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                const int ig = tile / p.n_row_tiles;
                const int n0 = ig * p.NB, oh0 = (tile - ig * p.n_row_tiles) * p.TH;
                const int rows_here = min(p.TH, p.OH - oh0), imgs_here = min(p.NB, p.N - n0);
                const int plane = p.OH * p.OW;
                const float zpf = float(q.y_zp);
                const unsigned img_stride = unsigned((y_blocked ? p.KB : p.K) * plane);
                // NCHW output in dwords of four positions: rows, planes and tile rows of whole quads, an aligned base
                const bool quad_rows = !y_blocked && (p.OW & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 3) == 0;
                // where this lane's position slots lie
                uint32_t praw[MT];
#pragma unroll
                for (int i = 0; i < MT; ++i) praw[i] = ps_read_b32(postab_a + unsigned(i * PS_NT * 4));
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int kblk = kp * p.KP + (2 * cp + j) * 32;  // first channel of this 32-channel block
                    const int kbase = kblk + lh * 4;
                    // multipliers and integer corrections (bias and zero-point term) of this lane's 16 channels
                    uint32_t mraw[16], craw[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) mraw[v] = ps_read_b32(mult_a + unsigned(kbase + (v >> 2) * 8 + (v & 3)) * 4u);
#pragma unroll
                    for (int v = 0; v < 16; ++v) craw[v] = ps_read_b32(corr_a + unsigned(kbase + (v >> 2) * 8 + (v & 3)) * 4u);
                    ps_wait16(mraw);
                    ps_wait16(craw);
                    if (j == 0) {
#pragma unroll
                        for (int i = 0; i < MT; ++i) asm volatile("" : "+v"(praw[i]));  // behind the wait above
                    }
                    float mv[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) mv[v] = __uint_as_float(mraw[v]);
                    const int cb0 = kblk >> 4;
                    // scalar part of the output offset (16-byte units of the blocked tensor / elements of the NCHW one)
                    const unsigned origin = y_blocked ? unsigned((n0 * p.KB + cb0) * plane + oh0 * p.OW)
                                                      : unsigned((n0 * p.K + kbase) * plane + oh0 * p.OW);
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        __builtin_amdgcn_sched_barrier(0);  // one position tile at a time
                        if (i == MT - 1 && !last_slot) continue;  // no tile in the wave's last slot (wave-uniform)
                        const int pos = int(praw[i]);
                        const int img = pos >> 20, r = (pos >> 10) & 1023, cc = pos & 1023;
                        const bool ok = pos >= 0 && img < imgs_here && r < rows_here;
                        const unsigned rel = __umul24(unsigned(img), img_stride) + __umul24(unsigned(r), unsigned(p.OW)) + unsigned(cc);
                        int av[16];  // this tile's sums with the corrections added
#pragma unroll
                        for (int v = 0; v < 16; ++v) av[v] = acc[j][i][v] + int(craw[v]);
                        // four dwords of four consecutive channels each, of one position (signed bytes for the blocked layout)
                        uint32_t d[4];
                        if constexpr (use_lut) {
                            uint32_t ob[16];
#pragma unroll
                            for (int v = 0; v < 16; ++v)
                                ob[v] = ps_read_u8(__builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(av[v]) * mv[v]) + zpf, 0u, lut_a));
                            ps_wait16(ob);
#pragma unroll
                            for (int gq = 0; gq < 4; ++gq)
                                d[gq] = ob[gq * 4] | (ob[gq * 4 + 1] << 8) | (ob[gq * 4 + 2] << 16) | (ob[gq * 4 + 3] << 24);
                        } else {
#pragma unroll
                            for (int gq = 0; gq < 4; ++gq) {
                                uint32_t w4 = 0;
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    w4 = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(float(av[gq * 4 + e]) * mv[gq * 4 + e]) + zpf, unsigned(e), w4);
                                d[gq] = y_blocked ? w4 ^ 0x80808080u : w4;
                            }
                        }
                        if constexpr (y_blocked) {
                            // [N][KB][OH][OW][16] signed.  A lane holds 4 groups of 4 consecutive channels of one position.
                            // Lanes l and l + 32 hold the two interleaved halves of the wave's two 16-channel blocks: the
                            // half-wave swap leaves the lower lane with all 16 bytes of the first block and the upper lane
                            // with those of the second, so each lane stores one whole 16-byte unit and a half wave 512
                            // contiguous bytes.
                            const auto s0 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
                            const auto s1 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
                            u32x4 out;
                            out[0] = s0[0]; out[1] = s0[1]; out[2] = s1[0]; out[3] = s1[1];
                            if (ok && cb0 + lh < p.KB)
                                __builtin_nontemporal_store(out, reinterpret_cast<u32x4 *>(y) + (origin + rel + unsigned(lh * plane)));
                        } else {
                            if (quad_rows) {
                                // Four lanes of a quad hold four consecutive positions of one row; a 4 x 4 byte transpose
                                // across them (two lane exchanges and two byte permutes per group of four channels) leaves
                                // lane q of the quad with channel q's four position bytes: a dword store per group where
                                // there were four byte stores.  (Plain stores: the cache gathers the 32-byte pieces of a
                                // line that successive position tiles write; non-temporal ones were slower, and a further
                                // transpose to one 16-byte store per lane gained nothing.)
                                // Everything derived from the lane number is made here, per tile, behind an opaque copy:
                                // held across the main loop it would not fit this kernel's registers.
                                uint32_t lq = uint32_t(lane);
                                asm volatile("" : "+v"(lq));
                                // sel1 = lane & 1 ? 0x03070105 : 0x06020400, sel2 = lane & 2 ? 0x03020706 : 0x05040100, without a
                                // register per constant
                                uint32_t sel1, sel2;
                                asm volatile("v_bfe_i32 %0, %2, 0, 1\n\tv_bfe_i32 %1, %2, 1, 1\n\t"
                                             "v_and_b32 %0, 0x05050505, %0\n\tv_and_b32 %1, 0x06060606, %1\n\t"
                                             "v_xor_b32 %0, 0x06020400, %0\n\tv_xor_b32 %1, 0x05040100, %1"
                                             : "=&v"(sel1), "=&v"(sel2) : "v"(lq));
                                const unsigned lq3 = lq & 3;
#pragma unroll
                                for (int gq = 0; gq < 4; ++gq) {
                                    const uint32_t d0 = d[gq];
                                    const uint32_t x1 = uint32_t(__builtin_amdgcn_update_dpp(0, int(d0), 0xB1, 0xf, 0xf, false));  // lane ^ 1
                                    const uint32_t t1 = __builtin_amdgcn_perm(x1, d0, sel1);
                                    const uint32_t x2 = uint32_t(__builtin_amdgcn_update_dpp(0, int(t1), 0x4E, 0xf, 0xf, false));  // lane ^ 2
                                    const uint32_t o4 = __builtin_amdgcn_perm(x2, t1, sel2);
                                    const int dk = gq * 8 + int(lq3);
                                    if (ok && kbase + dk < p.K)
                                        *reinterpret_cast<uint32_t *>(y + (origin + rel - lq3 + unsigned(dk * plane))) = o4;
                                }
                            } else if (ok) {
                                uint8_t *yp = y + (origin + rel);
#pragma unroll
                                for (int v = 0; v < 16; ++v) {
                                    const int dk = (v >> 2) * 8 + (v & 3);
                                    if (kbase + dk < p.K) yp[dk * plane] = uint8_t(d[v >> 2] >> ((v & 3) * 8));
                                }
                            }
                        }
                    }
                }
            }
        }
        tile = next_tile;
        if (tile >= p.n_tiles) break;
        if constexpr (XN) {
            // everybody has left the patch (and a staging region behind it): the next tile's goes in; the step boundary
            // that follows waits for these writes
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            ps_patch_from_nchw(xb, padvec, patch, p, tile);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Packs OIHW int8 weights into [pass][chunk of 32 input channels][tap][half][KP][16] (zero padded): the order in
// which the kernel's steps consume them, so that the weight stream is one run of addresses.  Also writes the
// per-channel requantisation multiplier, the integer correction (bias + (128 - x_zp) * sum of weights) and the 16-byte
// padding vector (x_zp - 128 in every lane).
__global__ void __launch_bounds__(256)
ps_pack_kernel(const int8_t *__restrict__ w, const float *__restrict__ w_scale, const int32_t *__restrict__ bias,
               int8_t *__restrict__ wp, float *__restrict__ mult, int32_t *__restrict__ corr, int8_t *__restrict__ padvec,
               int K, int C, int NC, int NKP, int KP, float x_scale, float y_scale, int x_zp, int n_wscale) {
    // (fewer than 2^31 packed bytes: the host checks; KP is 64 or 128)
    const unsigned total = unsigned(NKP) * unsigned(NC) * 9u * 32u * unsigned(KP);
    const unsigned step = gridDim.x * blockDim.x;
    const unsigned gid = blockIdx.x * blockDim.x + threadIdx.x;
    const int kp_shift = KP == 128 ? 7 : 6;
    if (gid < 16) padvec[gid] = int8_t(x_zp - 128);
    for (unsigned i = gid; i < total; i += step) {
        unsigned r = i;
        const int j = int(r & 15u); r >>= 4;
        const int kk = int(r & unsigned(KP - 1)); r >>= kp_shift;
        const int half = int(r & 1u); r >>= 1;
        const unsigned r9 = r / 9u;
        const int tap = int(r - r9 * 9u);
        const unsigned kp = r9 / unsigned(NC);
        const int chunk = int(r9 - kp * unsigned(NC));
        const int k = int(kp) * KP + kk, c = chunk * 32 + half * 16 + j;
        wp[i] = (k < K && c < C) ? w[(int64_t(k) * C + c) * 9 + tap] : int8_t(0);
    }
    // per output channel: one wavefront sums the channel's weights, as dwords where the rows are whole aligned dwords
    // (four signed bytes summed by one dot product with ones), every load of a round issued before the first add
    const int kpad = NKP * KP;
    const int lane = threadIdx.x & 63;
    const unsigned wave = gid >> 6, n_waves = step >> 6;
    const int row = C * 9;
    const bool dwords = (row & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 3) == 0;
    for (unsigned k = wave; k < unsigned(kpad); k += n_waves) {
        int sum = 0;
        if (k < unsigned(K)) {
            const int8_t *wk = w + int64_t(k) * row;
            if (dwords) {
                const int *wk4 = reinterpret_cast<const int *>(wk);
                const int n4 = row >> 2;
                for (int e0 = 0; e0 < n4; e0 += 8 * 64) {
                    int v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int e = e0 + u * 64 + lane;
                        v[u] = e < n4 ? wk4[e] : 0;
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u) sum = __builtin_amdgcn_sdot4(v[u], 0x01010101, sum, false);
                }
            } else {
                for (int e = lane; e < row; e += 64) sum += int(wk[e]);
            }
        }
        for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        if (lane == 0) {
            corr[k] = k < unsigned(K) ? (bias ? bias[k] : 0) + (128 - x_zp) * sum : 0;
            mult[k] = k < unsigned(K) ? (x_scale * w_scale[n_wscale == 1 ? 0 : k]) / y_scale : 0.0f;
        }
    }
}

size_t ps_align256(size_t v) { return (v + 255) & ~size_t(255); }

// Picks the tile (NB images x TH rows) with the smallest estimated time: rounds of tiles over the CUs times the MFMA
// count of the busiest SIMD of a tile, plus a fixed cost per tile for its fill and epilogue.
bool ps_plan(const ConvGeom &g, int num_cus, bool pool, PsGeom *out, size_t *lds_bytes, int *MT) {
    if (g.groups != 1 || g.KH != 3 || g.KW != 3 || g.sh != 1 || g.sw != 1 || g.dh != 1 || g.dw != 1) return false;
    if (g.pt > 1 || g.pl > 1) return false;
    if (g.C < 32 || g.K < 33) return false;
    // with the fused pool: whole windows only, and one output-channel pass (measured against the tiled kernel on
    // 512 x 128 x 6 x 6 -> 256 channels, two passes over 36-position images: 25.7 us here, 23.5 us there; from 16 -> 32
    // channels at 48 x 48, half of every MFMA multiplying padding: 39 against 26; 32 -> 64 at 24 x 24 and 64 -> 128 at
    // 12 x 12: 17.8 against 19.5 and 14.0 against 18.1)
    if (pool && ((g.OH & 1) || (g.OW & 1) || g.K > 128)) return false;
    if (g.OH > 1023 || g.OW > 1023) return false;
    const int CB = (g.C + 15) / 16;
    if (int64_t(g.N) * CB * g.H * g.W >= (int64_t(1) << 27)) return false;  // 16-byte units addressed with 32-bit offsets
    PsGeom p{};
    p.pool = pool ? 1 : 0;
    p.N = g.N; p.H = g.H; p.W = g.W; p.CB = CB; p.K = g.K; p.KB = (g.K + 15) / 16; p.OH = g.OH; p.OW = g.OW; p.pt = g.pt; p.pl = g.pl;
    p.NC = (g.C + 31) / 32;
    p.KP = g.K > 64 ? 128 : 64;
    p.NKP = (g.K + p.KP - 1) / p.KP;
    p.kpad = p.NKP * p.KP;
    p.tab_rounds = (p.kpad / 2 + PS_NT - 1) / PS_NT;
    const int pairs = p.KP / 64, NG = PS_WAVES / pairs;
    const int max_pos = NG * PS_MTMAX * 32;
    // output offsets are formed in 32 bits, per-image strides with 24-bit multiplies
    const int64_t plane = int64_t(g.OH) * g.OW;
    if (int64_t(p.KB) * plane >= (1 << 24) || int64_t(g.N) * p.KB * plane >= (int64_t(1) << 28)) return false;
    if (int64_t(g.K) * plane >= (1 << 24) || int64_t(g.N) * g.K * plane >= (int64_t(1) << 31)) return false;
    const size_t fixed = 256 + 256 + size_t(p.tab_rounds) * PS_NT * 16 + 2 * size_t(PS_RING);  // + slot table and patch
    const size_t cap = 160 * 1024;
    double best = 0;
    bool found = false;
    p.PW = g.OW + 2;
    auto consider = [&](int NB, int TH) {
        if (pool && (TH & 1)) return;
        PsGeom t = p;
        t.NB = NB; t.TH = TH;
        const int S = NB * TH * g.OW;
        if (S > max_pos || S < 1) return;
        t.PH = TH + 2;
        t.P1 = NB * t.PH * t.PW;
        t.P1s = (t.P1 + PS_NT - 1) / PS_NT * PS_NT;
        if (t.P1s / PS_NT > PS_RMAX || NB > 2047) return;
        t.npt = (S + 31) / 32;
        // (two position slots per wave at least: the one-slot instantiation needs more registers than it has, and a
        // kernel whose LDS reads are hidden from the compiler must not spill)
        const int per_wave = std::max(2, (t.npt + NG - 1) / NG);
        size_t lds = fixed + size_t(per_wave) * PS_NT * 4 + size_t(2 * t.NC) * t.P1s * 16;
        if (pool) {  // the staging rows of the pooled bytes: [16-channel block of a pass][window][16], behind the patch
            t.W_pad = (t.npt | 1) * 8;  // an odd number of position tiles: the two blocks of a store fall on different banks
            t.stage_off = int(2 * PS_RING + size_t(per_wave) * PS_NT * 4 + size_t(2 * t.NC) * t.P1s * 16);
            lds += size_t(t.W_pad) * t.KP;
        }
        if (lds > cap) return;
        t.n_row_tiles = (g.OH + TH - 1) / TH;
        const int64_t nt = int64_t((g.N + NB - 1) / NB) * t.n_row_tiles;
        if (nt >= (int64_t(1) << 30)) return;
        t.n_tiles = int(nt);
        // MFMAs of the busiest SIMD (waves w and w + 4) per tile
        const int base = t.npt / NG, rem = t.npt % NG;
        auto tiles_of = [&](int grp) { return base + (grp < rem ? 1 : 0); };
        int busiest_tiles = 0;
        for (int w = 0; w < 4; ++w) busiest_tiles = std::max(busiest_tiles, tiles_of(w / pairs) + tiles_of((w + 4) / pairs));
        const double mfma = 2.0 * busiest_tiles * t.NKP * t.NC * 9 * 32.0;
        const double rounds = double((t.n_tiles + num_cus - 1) / num_cus);
        const double tile_cycles = mfma + 4000.0 + double(S) * p.kpad / 256.0 * (pool ? 3.0 : 7.0);  // + fill, + epilogue VALU
        const double score = 1.0 / (rounds * tile_cycles);
        if (!found || score > best * 1.01) {
            best = score; found = true; *out = t; *lds_bytes = lds; *MT = per_wave;
        }
    };
    const int per_img = g.OH * g.OW;
    if (per_img <= max_pos)
        for (int NB = 1; NB <= std::min(g.N, max_pos / per_img); ++NB) consider(NB, g.OH);
    for (int TH = 1; TH <= g.OH; ++TH) consider(1, TH);
    return found;
}

template <int MT, int OUT, bool XN>
void ps_launch_one(zant_ctx *ctx, int grid, size_t lds, const int8_t *xb, const int8_t *wp, const char *tabs,
                   const int8_t *padvec, uint8_t *y, const PsGeom &p, const QConvArgs &q) {
    // (the kernel has no static LDS: the whole 160 KB of a compute unit may be asked for as dynamic LDS)
    if (!zant_raise_lds_limit(ctx, reinterpret_cast<const void *>(&qconv_ps_kernel<MT, OUT, XN>), 160 * 1024)) return;
    ZANT_KERNEL_NAME(ctx, "qconv_ps_kernel<%d,%d,%s>", MT, OUT, XN ? "true" : "false");
    hipLaunchKernelGGL((qconv_ps_kernel<MT, OUT, XN>), dim3(grid), dim3(PS_NT), lds, ctx->stream, xb, wp, tabs, padvec, y, p, q);
}

template <int MT, int OUT>
void ps_launch_out(zant_ctx *ctx, int grid, size_t lds, const int8_t *xb, const int8_t *wp, const char *tabs,
                   const int8_t *padvec, uint8_t *y, const PsGeom &p, const QConvArgs &q, bool x_nchw) {
    // an NCHW input comes from a caller of the C ABI, whose output is NCHW too
    constexpr bool nchw_out = OUT == PS_OUT_NCHW_LUT || OUT == PS_OUT_NCHW || OUT == PS_OUT_NCHW_ST || OUT == PS_OUT_NCHW_ST_LUT;
    if constexpr (nchw_out) {
        if (x_nchw) return ps_launch_one<MT, OUT, true>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q);
    }
    ps_launch_one<MT, OUT, false>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q);
}

template <int MT>
void ps_launch(zant_ctx *ctx, int grid, size_t lds, const int8_t *xb, const int8_t *wp, const char *tabs,
               const int8_t *padvec, uint8_t *y, const PsGeom &p, const QConvArgs &q, int yb, bool x_nchw) {
    if (!yb && p.out_unit && q.has_act) ps_launch_out<MT, PS_OUT_NCHW_ST_LUT>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
    else if (!yb && p.out_unit) ps_launch_out<MT, PS_OUT_NCHW_ST>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
    else if (!yb && q.has_act) ps_launch_out<MT, PS_OUT_NCHW_LUT>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
    else if (!yb) ps_launch_out<MT, PS_OUT_NCHW>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
    else if (p.pool) ps_launch_out<MT, PS_OUT_POOL>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
    else if (q.has_act) ps_launch_out<MT, PS_OUT_BLOCKED_LUT>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
    else ps_launch_out<MT, PS_OUT_BLOCKED>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, x_nchw);
}

}  // namespace

// The patch-stationary matrix-core path; ZANT_OK when it ran (or, with plan_only, would run), 1 when the shape is left
// to the other kernels.
int zant_qconv_ps(zant_ctx *ctx, const uint8_t *x, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *y,
                  const ConvGeom &g, const QConvArgs &q, bool x_blocked, bool y_blocked, zant_pack_slot *slot, bool plan_only,
                  bool pool) {
    PsGeom p;
    size_t lds = 0;
    int MT = 0;
    // a fused 2x2/2 max pool: blocked output, and an activation that keeps the order of its inputs (the pool is taken on
    // the accumulators)
    if (pool && (!y_blocked || (q.has_act && !(q.act.alpha >= 0.0f && q.act.in_scale > 0.0f && q.act.out_scale > 0.0f)))) return 1;
    // the tile search depends on the geometry only: a node or plan that calls again with the same one reuses its result
    struct PlanKey { ConvGeom g; int pool, cus, kind; } pkey;
    struct PlanVal { PsGeom p; size_t lds; int MT; } pval;
    std::memset(&pkey, 0, sizeof(pkey));
    pkey.g = g; pkey.pool = pool; pkey.cus = ctx->num_cus; pkey.kind = 0x50535f50;  // "PS_P"
    if (!plan_only && zant_plan_cached(slot, pkey, &pval)) {
        p = pval.p; lds = pval.lds; MT = pval.MT;
    } else {
        if (!ps_plan(g, ctx->num_cus, pool, &p, &lds, &MT)) return 1;
        if (!plan_only && MT >= 2 && MT <= PS_MTMAX) {
            std::memset(&pval, 0, sizeof(pval));
            pval.p = p; pval.lds = lds; pval.MT = MT;
            zant_plan_remember(slot, pkey, pval);
        }
    }
    if (MT < 2 || MT > PS_MTMAX) return 1;
    if (size_t(p.NKP) * p.NC * 9 * 32 * p.KP >= (size_t(1) << 31)) return 1;  // the packing kernel indexes in 32 bits
    if (plan_only) return ZANT_OK;
    const size_t wp_bytes = size_t(p.NKP) * p.NC * 9 * 32 * p.KP;
    // an NCHW input the kernel can regroup by itself needs no blocked copy
    const bool x_direct = !x_blocked && !y_blocked && g.C % 16 == 0 && g.W % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 4 == 0 &&
                          int64_t(g.N) * g.C * g.H * g.W < (int64_t(1) << 31);
    const size_t xb_bytes = x_blocked || x_direct ? 0 : size_t(g.N) * p.CB * g.H * g.W * 16;
    // [tile counters (unused) | padding vector | multipliers, corrections (one contiguous table) | packed weights]
    const size_t o_pad = 256, o_mult = 512, o_corr = o_mult + size_t(p.kpad) * 4,
                 o_wp = o_mult + ps_align256(size_t(p.kpad) * 8), static_bytes = o_wp + ps_align256(wp_bytes);
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
    if (need_pack) {
        const unsigned pb = unsigned(std::min<int64_t>(std::max<int64_t>(ceil_div64(int64_t(wp_bytes), 256), ceil_div64(p.kpad, 4)), 1024));
        hipLaunchKernelGGL(ps_pack_kernel, dim3(pb), dim3(256), 0, ctx->stream, w, w_scale, bias, wp, mult, corr, padvec, g.K, g.C,
                           p.NC, p.NKP, p.KP, q.x_scale, q.y_scale, q.x_zp, q.n_wscale);
        ZANT_LAUNCH_CHECK(ctx);
    }
    const int8_t *xb = reinterpret_cast<const int8_t *>(x);
    if (!x_blocked && !x_direct) {
        rc = zant_to_blocked(ctx, x, g.N, g.C, int64_t(g.H) * g.W, static_cast<uint8_t *>(dyn));
        if (rc) return rc;
        xb = static_cast<const int8_t *>(dyn);
    }
    const int grid = std::min(p.n_tiles, ctx->num_cus);
    // NCHW output: staged through LDS and written as whole runs of a plane when the runs are made of aligned 8- or
    // 4-byte units and the tile's bytes have room: a region of their own behind the patch, or -- one tile per workgroup,
    // one pass -- the ring, slot table and patch, which are dead by then.
    p.out_unit = 0; p.stage_alias = 0; p.S_pad = 0;
    if (!pool) p.stage_off = 0;
    if (!y_blocked) {
        const int per_img = p.TH * p.OW, plane = p.OH * p.OW;
        auto unit_ok = [&](int u) {
            return per_img % u == 0 && plane % u == 0 && (p.OH % p.TH == 0 || p.OW % u == 0) && reinterpret_cast<uintptr_t>(y) % u == 0;
        };
        const int unit = unit_ok(8) ? 8 : unit_ok(4) ? 4 : 0;
        // a staging row holds the tile's positions rounded up to whole position tiles (the last one is written whole);
        // 8 x an odd number of bytes: the 32 channels of a store then fall on 32 different even banks
        const int spad = ((p.npt * 32 / 8) | 1) * 8;
        const size_t need = size_t(spad) * p.KP, behind_ring = size_t(MT) * PS_NT * 4 + size_t(2 * p.NC) * p.P1s * 16;
        if (unit && lds + need <= size_t(160) * 1024) {
            p.out_unit = unit; p.S_pad = spad; p.stage_off = int(2 * PS_RING + behind_ring); lds += need;
        } else if (unit && p.n_tiles <= grid && p.NKP == 1 && need <= 2 * PS_RING + behind_ring) {
            p.out_unit = unit; p.S_pad = spad; p.stage_alias = 1;
        }
    }
    KernelTimer kt(ctx);
    const int yb = y_blocked ? 1 : 0;
    const char *tabs = base + o_mult;
    switch (MT) {
    case 2: ps_launch<2>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, yb, x_direct); break;
    case 3: ps_launch<3>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, yb, x_direct); break;
    default: ps_launch<4>(ctx, grid, lds, xb, wp, tabs, padvec, y, p, q, yb, x_direct); break;
    }
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
