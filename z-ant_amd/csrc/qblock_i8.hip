// MobileNetV2's inverted residual block as ONE kernel on the int8 matrix cores:
//   1x1 expansion (+ activation) -> depthwise 3x3, pads 1, stride 1 or 2 (+ activation) -> 1x1 projection
//   (-> QLinearAdd with the block input).
// Run layer by layer, the expanded tensors (6x the block input) cross HBM four times and every small layer pays a
// kernel launch; here they live only in LDS and a block is one launch.  The arithmetic of each stage is exactly that
// of the stand-alone kernels (exact int32 accumulation, the one f32 requantisation sequence, the activation as a
// 256-entry table), so the fused block is bit-identical to running the three QLinearConv nodes one after another.
//
// A workgroup (4 wavefronts) walks tiles of NB images x TH output rows.  Per tile:
//   A  the input patch ((TH-1)*stride+3 rows, W+2 columns, halo included) is copied into LDS, channel-blocked;
//   B  expansion: wave w takes (32 patch positions) x (32 expanded channels) pairs, one v_mfma_i32_32x32x32_i8 per 32
//      input channels, requantises and writes the bytes (value ^ 0x80) to the expanded patch in LDS; patch positions
//      outside the image receive the depthwise zero point instead (they are its padding);
//   D  depthwise + projection: wave w takes 32 output positions; per 32 expanded channels nine MFMAs with DIAGONAL
//      weight matrices (row c = tap weight of channel c in column c) compute the depthwise sums of 32 positions x 32
//      channels, the requantised bytes are exchanged between lanes p and p+32 so that each lane holds 16 consecutive
//      channels of its position -- the B operand of the projection MFMA -- and the projection accumulates over the
//      expanded channels in registers.  The result is requantised (and added to the block input) and stored.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <initializer_list>
#include <type_traits>

#include "quant_common.h"
#include "quant_layout.h"

namespace {

typedef int i32x16 __attribute__((ext_vector_type(16)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

struct QBlockArgs {
    int N, H, W, OH, OW, stride;
    int CBin, Cin32, Ce32, CBo;        // input channel blocks (16) / chunks (32); expanded chunks; output blocks
    int Co;                            // output channels (the rest of the last block is padding)
    int NB, TH, PH, PW, P, Ppad, Q;    // tile: images, output rows, patch rows / columns / positions, output positions
    int n_row_tiles, n_tiles;
    int o_xl, o_e, o_w1, o_w2, o_wdw, o_tab, o_ptab;  // LDS byte offsets
    int packed_units;                  // 16-byte units of weights and tables: the LDS bytes from o_w1 to o_ptab
    int split;                         // stage D deals (position tile, channel chunk) units to the waves (few position tiles)
    float zp1f, zp2f, zp3f;            // zero points of the three convolutions' own outputs
    QAct act1, act2;
    int has_act1, has_act2;
    uint32_t pad_e4;                   // the depthwise input zero point ^ 0x80 in every byte
    int half_last;                     // the last chunk of expanded channels holds at most 16 real ones
    int has_res, fast_div;             // fast_div: the scales allow the unscaled division sequence
    float ry_rcp;                      // refined reciprocal of ry_scale
    float ra_scale, rb_scale, ry_scale;  // residual add: a = projection output, b = block input, y = sum
    int ra_zp, rb_zp, ry_zp;
};

__device__ __forceinline__ i32x4 as_i32x4(const uint4 &v) {
    i32x4 r;
    r[0] = int(v.x); r[1] = int(v.y); r[2] = int(v.z); r[3] = int(v.w);
    return r;
}

// One block for the tiles of this workgroup; `lds` is the workgroup's dynamic LDS (256-byte aligned: the activation
// tables need it).
template <int CO32, int MQ, bool PF, bool SPLIT>
__device__ __forceinline__ void qblock_body(const uint4 *__restrict__ x, uint8_t *__restrict__ y, const uint4 *__restrict__ packed,
                                            const QBlockArgs &a, char *lds) {
    uint8_t *lut1 = reinterpret_cast<uint8_t *>(lds), *lut2 = lut1 + 256;
    uint4 *XL = reinterpret_cast<uint4 *>(lds + a.o_xl);   // [Cin32*2][Ppad] units of 16 channels
    uint4 *E = reinterpret_cast<uint4 *>(lds + a.o_e);     // [Ce32*2][Ppad]
    uint4 *W1 = reinterpret_cast<uint4 *>(lds + a.o_w1);   // [Cin32][Ce32][2][32] units
    uint4 *W2 = reinterpret_cast<uint4 *>(lds + a.o_w2);   // [Ce32][CO32][2][32] units
    uint32_t *WDW = reinterpret_cast<uint32_t *>(lds + a.o_wdw);  // [Ce/4][9][4] dwords
    const int Ce = a.Ce32 * 32;
    float *m1 = reinterpret_cast<float *>(lds + a.o_tab);
    int *c1 = reinterpret_cast<int *>(m1 + Ce);
    float *m2 = reinterpret_cast<float *>(c1 + Ce);
    int *c2 = reinterpret_cast<int *>(m2 + Ce);
    float *m3 = reinterpret_cast<float *>(c2 + Ce);
    int *c3 = reinterpret_cast<int *>(m3 + CO32 * 32);
    int *ptab = reinterpret_cast<int *>(lds + a.o_ptab);   // [Ppad] patch row; bit 31: a halo column or past the patch

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), l32 = lane & 31, lh = lane >> 5;
    const unsigned lut1_a = lds_address(lut1), lut2_a = lds_address(lut2);

    // ---- once per workgroup: tables and weights into LDS ----
    {
        const uint8_t b = uint8_t(tid);
        lut1[tid] = uint8_t((a.has_act1 ? qact_apply(b, a.act1) : b) ^ 0x80);
        lut2[tid] = uint8_t((a.has_act2 ? qact_apply(b, a.act2) : b) ^ 0x80);
    }
    // weights and requantisation tables: `packed` holds them in the order and spacing of their LDS region, so they are
    // one copy, eight 16-byte units per thread in flight at a time.  The first eight are loaded here and written to LDS
    // behind the first tile's input patch, whose loads thereby travel with them.
    i32x4 *wdst = reinterpret_cast<i32x4 *>(lds + a.o_w1);
    i32x4 w0[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) w0[r] = *reinterpret_cast<const i32x4 *>(packed + min(r * 256 + tid, a.packed_units - 1));
    {
        const int patch = a.PH * a.PW;
        const float inv_patch = 1.0f / float(patch), inv_pw = 1.0f / float(a.PW);
        for (int p = tid; p < a.Ppad; p += 256) {
            const int pp = min(p, a.P - 1);
            const int img = small_div(pp, patch, inv_patch), rem = pp - img * patch;
            const int ph = small_div(rem, a.PW, inv_pw), pw = rem - ph * a.PW;
            ptab[p] = ph | ((p >= a.P || pw == 0 || pw == a.PW - 1) ? int(0x80000000u) : 0);
        }
    }

    const float inv_p = 1.0f / float(a.P), inv_nptiles = 1.0f / float(a.Ppad >> 5);
    const float inv_tile_img = 1.0f / float(a.TH * a.OW), inv_ow = 1.0f / float(a.OW);
    const int n_ptiles = a.Ppad >> 5, nq_tiles = (a.Q + 31) >> 5;
    // the diagonal element of row l32 lies in this lane's half of the columns; which dword of the 16-byte operand
    const bool diag_mine = (l32 >> 4) == lh;
    const int diag_q = (l32 >> 2) & 3;
    const uint32_t dm0 = diag_mine && diag_q == 0 ? 0xffffffffu : 0u, dm1 = diag_mine && diag_q == 1 ? 0xffffffffu : 0u,
                   dm2 = diag_mine && diag_q == 2 ? 0xffffffffu : 0u, dm3 = diag_mine && diag_q == 3 ? 0xffffffffu : 0u;

    // ---- A: input patch -> LDS (positions outside the image are left as they are: C overwrites what they yield).  The
    // first tile's patch is copied before the loop; every later one is loaded into registers before stage B of the tile
    // in front of it and written to LDS after that stage (the input patch is dead once B is done), so its global
    // latency passes under B.  Patches of more than QB_PF units per thread are copied in place instead. ----
    constexpr int QB_PF = 4;
    const int patch_hw = a.PH * a.PW;
    const float inv_patch_hw = 1.0f / float(patch_hw), inv_pw_ = 1.0f / float(a.PW);
    const int a_units = a.CBin * a.P;
    const bool prefetch = PF && a_units <= QB_PF * 256;  // PF is off for the instantiations without registers to spare
    auto patch_unit = [&](int tile_, int u, int &dst) -> const uint4 * {  // source of unit u of a tile's patch, or null
        const int ig_ = tile_ / a.n_row_tiles, rt_ = tile_ - ig_ * a.n_row_tiles;
        const int cb = small_div(u, a.P, inv_p), p = u - cb * a.P;
        const int img = small_div(p, patch_hw, inv_patch_hw), rem = p - img * patch_hw;   // (not from the position table: the
        const int ph = small_div(rem, a.PW, inv_pw_), pw = rem - ph * a.PW;               // first patch is fetched before it exists)
        const int n = ig_ * a.NB + img, ih = rt_ * a.TH * a.stride - 1 + ph, iw = pw - 1;
        dst = cb * a.Ppad + p;
        if (n < a.N && ih >= 0 && ih < a.H && iw >= 0 && iw < a.W) return x + ((int64_t(n) * a.CBin + cb) * a.H + ih) * int64_t(a.W) + iw;
        return nullptr;
    };
    auto copy_patch = [&](int tile_) {  // four loads in flight per thread, then their four LDS writes
        for (int u0 = tid; u0 < a_units; u0 += 4 * 256) {
            i32x4 v[4];  // (a native vector type: arrays of it are kept in registers)
            int dst[4];
            bool ok[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int u = min(u0 + r * 256, a_units - 1);
                const uint4 *src = patch_unit(tile_, u, dst[r]);
                ok[r] = src != nullptr && u0 + r * 256 < a_units;
                v[r] = *reinterpret_cast<const i32x4 *>(ok[r] ? src : x);
            }
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (ok[r]) *reinterpret_cast<i32x4 *>(XL + dst[r]) = v[r];
        }
    };
    if (int(blockIdx.x) < a.n_tiles) copy_patch(blockIdx.x);
#pragma unroll
    for (int r = 0; r < 8; ++r)
        if (r * 256 + tid < a.packed_units) wdst[r * 256 + tid] = w0[r];
    for (int i0 = 8 * 256; i0 < a.packed_units; i0 += 8 * 256) {
        i32x4 v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) v[r] = *reinterpret_cast<const i32x4 *>(packed + min(i0 + r * 256 + tid, a.packed_units - 1));
#pragma unroll
        for (int r = 0; r < 8; ++r)
            if (i0 + r * 256 + tid < a.packed_units) wdst[i0 + r * 256 + tid] = v[r];
    }
    __syncthreads();

    for (int tile = blockIdx.x; tile < a.n_tiles; tile += gridDim.x) {
        const int ig = tile / a.n_row_tiles, rt = tile - ig * a.n_row_tiles;
        const int n0 = ig * a.NB, oh0 = rt * a.TH, ih0 = oh0 * a.stride - 1;
        const int next_tile = tile + int(gridDim.x);
        const bool has_next = next_tile < a.n_tiles;
        i32x4 nxt[QB_PF];
        int nxt_dst[QB_PF];
        unsigned nxt_ok = 0;
        if (PF && prefetch && has_next) {
#pragma unroll
            for (int r = 0; r < QB_PF; ++r) {
                nxt_dst[r] = 0;
                if (r * 256 < a_units) {
                    // every lane loads (from the tensor's first unit when it has nothing to fetch): no divergent branch
                    // around the load, so nothing waits for it before the values are written to LDS
                    const int u = min(r * 256 + tid, a_units - 1);
                    const uint4 *src = patch_unit(next_tile, u, nxt_dst[r]);
                    const bool ok = src != nullptr && r * 256 + tid < a_units;
                    nxt[r] = *reinterpret_cast<const i32x4 *>(ok ? src : x);
                    nxt_ok |= ok ? 1u << r : 0u;
                }
            }
        }

        // ---- B: expansion.  A wave keeps one block of 32 expanded channels (its multipliers, corrections and, for one
        // chunk of input channels, its weights) in registers and walks the position tiles with it. ----
        {
            // (channel block, position tile) units in channel-block-major order, split evenly over the four waves
            // (a block whose second half is padding costs about 4/5 of a full one: half the requantisation)
            const int full_units = (a.half_last ? a.Ce32 - 1 : a.Ce32) * n_ptiles, half_units = a.half_last ? n_ptiles : 0;
            const int cost = full_units * 5 + half_units * 4;
            auto unit_at = [&](int c) { return c <= full_units * 5 ? c / 5 : full_units + (c - full_units * 5) / 4; };
            const int u_begin = unit_at((cost * wave) >> 2), u_end = wave == 3 ? full_units + half_units : unit_at((cost * (wave + 1)) >> 2);
            int kb = small_div(u_begin, n_ptiles, inv_nptiles), ptile = u_begin - kb * n_ptiles;
            for (int u = u_begin; u < u_end;) {
                const int kch = kb * 32 + lh * 4;
                i32x16 cvec;
                float mv[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    cvec[v] = c1[kch + (v >> 2) * 8 + (v & 3)];
                    mv[v] = m1[kch + (v >> 2) * 8 + (v & 3)];
                }
                const i32x4 wa0 = as_i32x4(W1[kb * 64 + lh * 32 + l32]);
                const bool half = a.half_last && kb == a.Ce32 - 1;
                // this lane's operand of input chunk 0 and the 16-byte unit it writes: lane (p, 0) the block of expanded
                // channels 32 kb .. + 15 of its position, lane (p, 1) the block of channels 32 kb + 16 .. + 31
                const unsigned x_addr = lds_address(XL) + unsigned(lh * a.Ppad + l32) * 16u;
                const unsigned e_addr = lds_address(E) + unsigned((2 * kb + lh) * a.Ppad + l32) * 16u;
                // Two position tiles at a time (then a single one): the second tile's operand read, MFMA and table lookups
                // travel under the first one's arithmetic.  A position of the depthwise convolution's padding -- a halo
                // column, a row outside the image -- receives that convolution's zero point instead of its expansion.
                auto units = [&](auto nu_tag) {
                    constexpr int NU = decltype(nu_tag)::value;
                    bool padp[NU];
#pragma unroll
                    for (int j = 0; j < NU; ++j) {
                        const int e = ptab[(ptile + j) * 32 + l32];
                        padp[j] = e < 0 || unsigned(ih0 + (e & 0xffff)) >= unsigned(a.H);
                    }
                    i32x4 xb[NU];
#pragma unroll
                    for (int j = 0; j < NU; ++j) qb_read128(xb[j], x_addr + unsigned(ptile + j) * 512u, 0);
                    i32x16 acc[NU];
#pragma unroll
                    for (int j = 0; j < NU; ++j) {
                        qb_ready(xb[j], NU - 1 - j);
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa0, xb[j], cvec, 0, 0, 0);
                    }
                    for (int chunk = 1; chunk < a.Cin32; ++chunk) {
                        const i32x4 wc = as_i32x4(W1[(chunk * a.Ce32 + kb) * 64 + lh * 32 + l32]);
#pragma unroll
                        for (int j = 0; j < NU; ++j)
                            acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wc, as_i32x4(XL[(2 * chunk + lh) * a.Ppad + (ptile + j) * 32 + l32]),
                                                                           acc[j], 0, 0, 0);
                    }
                    // a last block with at most 16 real channels: accumulator rows 16..31 (values 8..15) are padding
                    uint32_t d[NU][4];
                    if (half) qb_requant_lookup_n<2, NU>(acc, mv, a.zp1f, lut1_a, d);
                    else qb_requant_lookup_n<4, NU>(acc, mv, a.zp1f, lut1_a, d);
#pragma unroll
                    for (int j = 0; j < NU; ++j) {
                        // the half-wave swap leaves the lower lane with the 16 bytes of the first block of 16 channels and
                        // the upper lane with those of the second: one 16-byte write per lane
                        const auto s0 = __builtin_amdgcn_permlane32_swap(d[j][0], d[j][2], false, false);
                        const auto s1 = __builtin_amdgcn_permlane32_swap(d[j][1], d[j][3], false, false);
                        i32x4 out;
                        out[0] = padp[j] ? int(a.pad_e4) : int(s0[0]); out[1] = padp[j] ? int(a.pad_e4) : int(s0[1]);
                        out[2] = padp[j] ? int(a.pad_e4) : int(s1[0]); out[3] = padp[j] ? int(a.pad_e4) : int(s1[1]);
                        if (!half || !lh)
                            *reinterpret_cast<__attribute__((address_space(3))) i32x4 *>(e_addr + unsigned(ptile + j) * 512u) = out;
                    }
                    ptile += NU;
                    u += NU;
                };
                while (ptile + 1 < n_ptiles && u + 1 < u_end) units(std::integral_constant<int, 2>());
                if (ptile < n_ptiles && u < u_end) units(std::integral_constant<int, 1>());
                ptile = 0;
                ++kb;
            }
        }
        __syncthreads();

        // ---- the next tile's input patch goes to LDS (the current one is dead; stage D reads the expanded patch only) ----
        if (has_next) {
            if (PF && prefetch) {
#pragma unroll
                for (int r = 0; r < QB_PF; ++r)
                    if ((nxt_ok >> r) & 1u) *reinterpret_cast<i32x4 *>(XL + nxt_dst[r]) = nxt[r];
            } else {
                copy_patch(next_tile);
            }
        }

        // ---- D: depthwise 3x3 + projection.  A wave takes MQ tiles of 32 output positions at a time; per chunk of 32
        // expanded channels the nine diagonal operands and the requantisation tables are set up once for all of them. ----
        // With few position tiles per workgroup tile (late, small feature maps) that split leaves waves idle while others
        // walk every chunk: then (SPLIT) every wave holds all MQ = nq_tiles position tiles, the (position tile, chunk)
        // units are dealt evenly to the four waves in position-tile-major order, and the waves' partial projection sums
        // are added up in LDS (integer addition: the order does not matter) before wave j requantises position tile j.
        const int q_per_wave = SPLIT ? nq_tiles : (nq_tiles + 3) >> 2;
        const int q_end = SPLIT ? nq_tiles : min(nq_tiles, (wave + 1) * q_per_wave);
        const int n_units = nq_tiles * a.Ce32, u_begin = (n_units * wave) >> 2, u_end = (n_units * (wave + 1)) >> 2;
        for (int q0 = SPLIT ? 0 : wave * q_per_wave; q0 < q_end; q0 += MQ) {
            int p0[MQ], qimg[MQ], qr[MQ], qc[MQ];
            bool qvalid[MQ];
#pragma unroll
            for (int j = 0; j < MQ; ++j) {
                const int q = (q0 + j) * 32 + l32;
                qvalid[j] = q0 + j < q_end && q < a.Q;
                const int qq = qvalid[j] ? q : 0;
                qimg[j] = small_div(qq, a.TH * a.OW, inv_tile_img);
                const int rem = qq - qimg[j] * a.TH * a.OW;
                qr[j] = small_div(rem, a.OW, inv_ow);
                qc[j] = rem - qr[j] * a.OW;
                p0[j] = (qimg[j] * a.PH + qr[j] * a.stride) * a.PW + qc[j] * a.stride;  // top-left tap in the patch
            }
            i32x16 acc3[MQ][CO32];
#pragma unroll
            for (int kb3 = 0; kb3 < CO32; ++kb3)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int cv = SPLIT ? 0 : c3[kb3 * 32 + lh * 4 + (v >> 2) * 8 + (v & 3)];  // split: added after the sum
#pragma unroll
                    for (int j = 0; j < MQ; ++j) acc3[j][kb3][v] = cv;
                }
            for (int ch = 0; ch < a.Ce32; ++ch) {
                if (SPLIT) {  // does any position tile's unit of this chunk belong to this wave?
                    bool any = false;
#pragma unroll
                    for (int j = 0; j < MQ; ++j) any |= j * a.Ce32 + ch >= u_begin && j * a.Ce32 + ch < u_end;
                    if (!any) continue;
                }
                const int kch = ch * 32 + lh * 4;
                const bool half = a.half_last && ch == a.Ce32 - 1;
                i32x16 cvec;
                float mv[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    cvec[v] = c2[kch + (v >> 2) * 8 + (v & 3)];
                    mv[v] = m2[kch + (v >> 2) * 8 + (v & 3)];
                }
                const uint32_t *wk = WDW + ((ch * 32 + l32) >> 2) * 36 + (l32 & 3);
                i32x4 wa[9];
#pragma unroll
                for (int t = 0; t < 9; ++t) {
                    const uint32_t wd = wk[t * 4];
                    wa[t][0] = int(wd & dm0); wa[t][1] = int(wd & dm1); wa[t][2] = int(wd & dm2); wa[t][3] = int(wd & dm3);
                }
                i32x4 w2a[CO32];
#pragma unroll
                for (int kb3 = 0; kb3 < CO32; ++kb3) w2a[kb3] = as_i32x4(W2[(ch * CO32 + kb3) * 64 + lh * 32 + l32]);
                // The nine taps of a position tile are issued as one batch and consumed by the MFMAs as they arrive; the
                // taps of the next tile are issued before this tile's requantisation, so they travel under its arithmetic.
                const unsigned e_ch = lds_address(E) + unsigned((2 * ch + lh) * a.Ppad) * 16u;
                const unsigned row_b = unsigned(a.PW) * 16u;
                i32x4 tap[9];
                auto issue_taps = [&](int j) {
                    const unsigned r0 = e_ch + unsigned(p0[j]) * 16u, r1 = r0 + row_b, r2 = r1 + row_b;
                    qb_read128(tap[0], r0, 0); qb_read128(tap[1], r0, 16); qb_read128(tap[2], r0, 32);
                    qb_read128(tap[3], r1, 0); qb_read128(tap[4], r1, 16); qb_read128(tap[5], r1, 32);
                    qb_read128(tap[6], r2, 0); qb_read128(tap[7], r2, 16); qb_read128(tap[8], r2, 32);
                };
                if (!SPLIT) issue_taps(0);
#pragma unroll
                for (int j = 0; j < MQ; ++j) {
                    if (SPLIT) {
                        if (j * a.Ce32 + ch < u_begin || j * a.Ce32 + ch >= u_end) continue;
                        issue_taps(j);
                    }
                    qb_ready(tap[0], 8);
                    i32x16 acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[0], tap[0], cvec, 0, 0, 0);
#pragma unroll
                    for (int t = 1; t < 9; ++t) {
                        qb_ready(tap[t], 8 - t);
                        acc2 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wa[t], tap[t], acc2, 0, 0, 0);
                    }
                    if (j + 1 < MQ && !SPLIT) issue_taps(j + 1);
                    uint32_t d[4];
                    if (half) qb_requant_lookup<2>(acc2, mv, a.zp2f, lut2_a, d);
                    else qb_requant_lookup<4>(acc2, mv, a.zp2f, lut2_a, d);
                    // lane (p, 0) gathers channels 0..15 of the chunk, lane (p, 1) channels 16..31
                    const auto s0 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
                    i32x4 db;
                    db[0] = int(s0[0]); db[1] = int(s0[1]); db[2] = int(s1[0]); db[3] = int(s1[1]);
#pragma unroll
                    for (int kb3 = 0; kb3 < CO32; ++kb3)
                        acc3[j][kb3] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w2a[kb3], db, acc3[j][kb3], 0, 0, 0);
                }
            }
            if (SPLIT) {
                // the expanded patch is dead once every wave has left the chunk loop: its first bytes hold the sums,
                // [position tile][output block][accumulator register][lane]
                int *R = reinterpret_cast<int *>(E);
                __syncthreads();
                for (int i = tid; i < MQ * CO32 * 16 * 64; i += 256) R[i] = 0;
                __syncthreads();
#pragma unroll
                for (int j = 0; j < MQ; ++j) {
                    if (u_begin >= (j + 1) * a.Ce32 || u_end <= j * a.Ce32 || u_begin >= u_end) continue;  // no unit of tile j
#pragma unroll
                    for (int kb3 = 0; kb3 < CO32; ++kb3)
#pragma unroll
                        for (int v = 0; v < 16; ++v) atomicAdd(R + ((j * CO32 + kb3) * 16 + v) * 64 + lane, acc3[j][kb3][v]);
                }
                __syncthreads();
#pragma unroll
                for (int j = 0; j < MQ; ++j) {
                    if (j != wave) continue;
#pragma unroll
                    for (int kb3 = 0; kb3 < CO32; ++kb3)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            acc3[j][kb3][v] = R[((j * CO32 + kb3) * 16 + v) * 64 + lane] + c3[kb3 * 32 + lh * 4 + (v >> 2) * 8 + (v & 3)];
                }
            }
            auto store_tiles = [&](auto res_tag, auto fast_tag) {
                constexpr bool RES = decltype(res_tag)::value, FAST = decltype(fast_tag)::value;
                // byte offset of this lane's four channels in block 0 of its position (the host checks that the blocked
                // tensors stay below 2^31 bytes); a block of 16 channels further on is one plane further
                unsigned ybase[MQ];
                bool ok[MQ];
                const unsigned plane16 = unsigned(a.OH * a.OW) * 16u;
#pragma unroll
                for (int j = 0; j < MQ; ++j) {
                    const int n = n0 + qimg[j], oh = oh0 + qr[j];
                    ok[j] = qvalid[j] && n < a.N && oh < a.OH && (!SPLIT || j == wave);
                    ybase[j] = ((unsigned(n) * unsigned(a.CBo) * unsigned(a.OH) + unsigned(oh)) * unsigned(a.OW) + unsigned(qc[j])) * 16u + unsigned(lh) * 4u;
                }
                // the residual's bytes of every (tile, group) first, as one batch of loads
                uint32_t xr[MQ][CO32 * 4];
                if (RES) {
#pragma unroll
                    for (int j = 0; j < MQ; ++j)
#pragma unroll
                        for (int g = 0; g < CO32 * 4; ++g) {
                            xr[j][g] = 0;
                            if (ok[j] && g * 8 < a.Co)
                                xr[j][g] = *reinterpret_cast<const uint32_t *>(reinterpret_cast<const char *>(x) + (ybase[j] + unsigned(g >> 1) * plane16 + unsigned(g & 1) * 8u));
                        }
                }
#pragma unroll
                for (int kb3 = 0; kb3 < CO32; ++kb3) {
#pragma unroll
                    for (int gq = 0; gq < 4; ++gq) {
                        const int cbq = kb3 * 2 + (gq >> 1);
                        if (cbq >= a.CBo) continue;
                        const unsigned goff = unsigned(cbq) * plane16 + unsigned(gq & 1) * 8u;
                        // eight output channels per group: a group past the last real channel is padding of the blocked
                        // layout (no kernel reads it against a non-zero weight): no arithmetic, zeros stored
                        if (kb3 * 32 + gq * 8 >= a.Co) {
#pragma unroll
                            for (int j = 0; j < MQ; ++j)
                                if (ok[j]) *reinterpret_cast<uint32_t *>(y + (ybase[j] + goff)) = 0u;
                            continue;
                        }
                        float mq[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) mq[e] = m3[kb3 * 32 + gq * 8 + lh * 4 + e];
#pragma unroll
                        for (int j = 0; j < MQ; ++j) {
                            uint32_t o = 0;
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const float r = __builtin_rintf(float(acc3[j][kb3][gq * 4 + e]) * mq[e]) + a.zp3f;
                                if (RES) {
                                    // the projection's own output byte as a float (the saturation is the clamp), then the
                                    // quantised add in dequantised space; every step is the stand-alone kernels' arithmetic
                                    const float va = __builtin_amdgcn_fmed3f(r, 0.0f, 255.0f);
                                    const float fa = (va - float(a.ra_zp)) * a.ra_scale;
                                    const float fb = (float(((xr[j][kb3 * 4 + gq] ^ 0x80808080u) >> (8 * e)) & 0xffu) - float(a.rb_zp)) * a.rb_scale;
                                    // finite operands: the saturating conversion replaces the clamp
                                    const float qv = FAST ? div_by(fa + fb, a.ry_scale, a.ry_rcp, 1) : (fa + fb) / a.ry_scale;
                                    o = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_rintf(qv) + float(a.ry_zp), e, o);
                                } else {
                                    o = __builtin_amdgcn_cvt_pk_u8_f32(r, e, o);
                                }
                            }
                            if (ok[j]) *reinterpret_cast<uint32_t *>(y + (ybase[j] + goff)) = o ^ 0x80808080u;
                        }
                    }
                }
            };
            if (!a.has_res) store_tiles(std::false_type(), std::false_type());
            else if (a.fast_div) store_tiles(std::true_type(), std::true_type());
            else store_tiles(std::true_type(), std::false_type());
        }
        __syncthreads();  // the next tile overwrites the patches
    }
}

template <int CO32, int MQ, bool PF, bool SPLIT>
__global__ void __launch_bounds__(256, 2)  // 256 registers per lane for every instantiation: over that, values would be
                                           // parked in accumulator registers, which the hand-issued LDS reads do not survive
qblock_kernel(const uint4 *__restrict__ x, uint8_t *__restrict__ y, const uint4 *__restrict__ packed, QBlockArgs a) {
    extern __shared__ __attribute__((aligned(256))) char lds[];
    qblock_body<CO32, MQ, PF, SPLIT>(x, y, packed, a, lds);
}

// Several blocks in a row as ONE launch.  Every block of a chain works on tiles of the same NB whole images, one tile
// per workgroup, so the images a workgroup reads in block b + 1 are exactly those it wrote in block b: no workgroup ever
// waits for another one, and a barrier of the workgroup (whose release waits for its stores; the vector L1 is shared by
// the wavefronts of a compute unit) orders its own writes before its own reads.  What a chain saves is the launch,
// the drain and the cold start of every block but the first; the arithmetic is that of the single blocks.
// Workgroups run through the chain at their own pace, so one may be writing block b + 1's output while another still reads
// block b's input: the caller must give every tensor of a chain storage of its own (a planner that lets a later tensor
// reuse an earlier one's memory, as is right for separate launches, would let images overwrite each other here).
constexpr int QB_CHAIN_MAX = 10;
struct QBlockLink {
    const uint4 *x;
    uint8_t *y;
    const uint4 *packed;
    QBlockArgs a;
};
struct QBlockChain {
    int n;
    QBlockLink link[QB_CHAIN_MAX];
};

template <int CO32, int MQ>
__global__ void __launch_bounds__(256, 2)
qblock_chain_kernel(QBlockChain c) {
    extern __shared__ __attribute__((aligned(256))) char lds[];
    for (int b = 0; b < c.n; ++b) {
        const QBlockLink &l = c.link[b];
        if (l.a.split) qblock_body<CO32, MQ, false, true>(l.x, l.y, l.packed, l.a, lds);
        else qblock_body<CO32, MQ, false, false>(l.x, l.y, l.packed, l.a, lds);
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): this wave's stores of the block's output have arrived
        __syncthreads();
    }
}

size_t align256(size_t v) { return (v + 255) & ~size_t(255); }
size_t align16(size_t v) { return (v + 15) & ~size_t(15); }

bool conv1x1(const zant_qconv_desc *d) { return d && d->K > 0 && d->C > 0 && (d->n_wscale == 1 || d->n_wscale == d->K); }

// What a launch needs of one block: its kernel arguments, LDS bytes, instantiation and packed weights.
struct QBlockPrep {
    QBlockArgs a;
    size_t lds_bytes;
    int CO32, MQv;
    const uint4 *packed;
};

// Plans a block's tile, (re)packs its weights and tables into `slot` (or the context workspace) and fills the kernel
// arguments.  force_nb > 0: tiles of exactly that many whole images, or 1.  plan_only: no packing, no pointers needed.
int qblock_prepare(zant_ctx *ctx, const int64_t xdim[4], const zant_qconv_desc *expand, const zant_qconv_desc *dw, int64_t dw_stride,
                   const zant_qconv_desc *project, int residual, float add_scale, int add_zp, const int64_t ydim[4], bool plan_only,
                   zant_pack_slot *slot, int force_nb, QBlockPrep *out) {
    if (!ctx || !xdim || !ydim || !expand || !dw || !project) return ZANT_NullPointer;
    if (!conv1x1(expand) || !conv1x1(dw) || !conv1x1(project)) return 1;
    const int64_t N = xdim[0], Cin = xdim[1], H = xdim[2], W = xdim[3];
    const int64_t Ce = expand->K, Co = project->K;
    if (N <= 0 || H <= 0 || W <= 0 || expand->C != Cin || dw->C != Ce || dw->K != Ce || project->C != Ce) return 1;
    if (dw_stride != 1 && dw_stride != 2) return 1;
    const int64_t OH = (H + 2 - 3) / dw_stride + 1, OW = (W + 2 - 3) / dw_stride + 1;
    if (ydim[0] != N || ydim[1] != Co || ydim[2] != OH || ydim[3] != OW) return 1;
    if (residual && (Co != Cin || OH != H || OW != W)) return 1;
    if (Cin > 512 || Ce > 2048 || Co > 128 || W + 2 > 1023 || N > INT32_MAX / 2) return 1;
    if (N * ((Cin + 15) / 16) * H * W >= (int64_t(1) << 27) || N * ((Co + 15) / 16) * OH * OW >= (int64_t(1) << 27)) return 1;

    QBlockArgs a;
    a.N = int(N); a.H = int(H); a.W = int(W); a.OH = int(OH); a.OW = int(OW); a.stride = int(dw_stride);
    a.CBin = int((Cin + 15) / 16); a.Cin32 = int((Cin + 31) / 32); a.Ce32 = int((Ce + 31) / 32); a.CBo = int((Co + 15) / 16); a.Co = int(Co);
    const int CO32 = int((Co + 31) / 32), CeP = a.Ce32 * 32;
    a.PW = int(W) + 2;
    // LDS: fixed part, then per patch position the input and expanded bytes and one table entry
    const size_t w1_bytes = size_t(a.Cin32) * a.Ce32 * 1024, w2_bytes = size_t(a.Ce32) * CO32 * 1024;
    const size_t wdw_bytes = size_t(CeP) * 9 * 4, tab_bytes = (size_t(CeP) * 4 + size_t(CO32) * 32 * 2) * 4;
    if (CO32 > 4) return 1;
    // Tile = NB whole images, or TH output rows of one image.  Among the shapes that fit -- in half a CU's LDS first, so
    // that two workgroups share a CU -- the one with the fewest wave instructions per image by a model of the kernel's
    // stages: B works on (32 positions x 32 expanded channels) units split over 4 waves, D on tiles of 32 output
    // positions, MQ at a time per wave; partly filled units and the halo rows cost as much as full ones.
    const int mq_cap = CO32 == 1 ? 4 : CO32 == 2 ? 2 : 1;
    const int64_t p_img = ((OH - 1) * dw_stride + 3) * a.PW;
    auto lds_for = [&](int64_t P) {
        const int64_t Ppad = (P + 31) & ~int64_t(31);
        return size_t(512) + size_t(a.Cin32 * 2 + a.Ce32 * 2) * size_t(Ppad) * 16 + w1_bytes + w2_bytes + wdw_bytes + tab_bytes +
               size_t(Ppad) * 4;
    };
    auto tile_cost = [&](int64_t P, int64_t Q) {
        const int64_t b_units = int64_t(a.Ce32) * ((P + 31) / 32), nq = (Q + 31) / 32, qpw = (nq + 3) / 4;
        const int64_t rounds = (qpw + mq_cap - 1) / mq_cap, mq = (qpw + rounds - 1) / rounds;
        const double epi = residual ? 350.0 : 150.0;
        return double((b_units + 3) / 4) * 150.0 + double(rounds) * (a.Ce32 * (100.0 + mq * 170.0) + mq * epi) +
               double(P) * (a.CBin + a.Ce32 * 2) / 256.0 * 15.0 + 300.0;
    };
    bool found = false;
    size_t cap_used = 0;
    double best_time = 0.0;
    // the tile search below depends on the shapes only: a node or plan that calls again with the same ones reuses it
    struct PlanKey { int64_t x[4], y[4], Ce, stride; int residual, force_nb, cus, kind; } pkey;
    struct PlanVal { QBlockArgs a; size_t cap_used; } pval;
    std::memset(&pkey, 0, sizeof(pkey));
    for (int i = 0; i < 4; ++i) { pkey.x[i] = xdim[i]; pkey.y[i] = ydim[i]; }
    pkey.Ce = Ce; pkey.stride = dw_stride; pkey.residual = residual ? 1 : 0; pkey.force_nb = force_nb; pkey.cus = ctx->num_cus;
    pkey.kind = 0x51424c4b;  // "QBLK"
    const bool cached = zant_plan_cached(slot, pkey, &pval);
    if (cached) { a = pval.a; cap_used = pval.cap_used; found = true; }
    // 76 KB: what two workgroups per CU leave each other after the allocation granularity.  Both sizes are planned and
    // the cheaper taken: two workgroups on a CU run at half speed each but overlap each other's barriers and latencies,
    // which the estimate credits with a factor 1.5 against the single large workgroup.
    for (size_t cap : {size_t(76 * 1024), size_t(160 * 1024)}) {
        if (cached) break;
        const bool two = cap <= 80 * 1024;
        const int64_t slots = int64_t(ctx->num_cus) * (two ? 2 : 1);
        double best = 0.0;
        int bNB = 0, bTH = 0;
        if (lds_for(p_img) <= cap) {
            for (int64_t nb = 1; nb <= std::min<int64_t>(N, 2047) && lds_for(nb * p_img) <= cap; ++nb) {
                if (force_nb > 0 && nb != force_nb) continue;
                const int64_t tiles = (N + nb - 1) / nb, waves = (tiles + slots - 1) / slots;
                const double c = tile_cost(nb * p_img, nb * OH * OW) * double(waves);  // time of the busiest workgroup slot
                if (!bNB || c < best * 0.98) { best = c; bNB = int(nb); bTH = int(OH); }
            }
        } else if (force_nb <= 0) {
            for (int64_t th = 1; th <= OH; ++th) {
                const int64_t P = ((th - 1) * dw_stride + 3) * a.PW;
                if (lds_for(P) > cap) break;
                const int64_t nrt = (OH + th - 1) / th;
                if ((OH + nrt - 1) / nrt != th) continue;  // only evened-out row tiles
                const int64_t tiles = N * nrt, waves = (tiles + slots - 1) / slots;
                const double c = tile_cost(P, th * OW) * double(waves);
                if (!bNB || c < best * 0.98) { best = c; bNB = 1; bTH = int(th); }
            }
        }
        if (!bNB) continue;
        const double time = best * (two ? 2.0 : 1.5);
        if (found && time >= best_time) continue;
        QBlockArgs t = a;
        t.NB = bNB; t.TH = bTH;
        t.PH = (bTH - 1) * int(dw_stride) + 3;
        if (t.PH > 1023) continue;
        t.P = bNB * t.PH * t.PW;
        t.Ppad = (t.P + 31) & ~31;
        t.Q = bNB * bTH * int(OW);
        t.n_row_tiles = int((OH + bTH - 1) / bTH);
        const int64_t n_tiles = ((N + bNB - 1) / bNB) * t.n_row_tiles;
        if (n_tiles > INT32_MAX || t.P >= (1 << 20) || t.Q >= (1 << 20)) continue;
        t.n_tiles = int(n_tiles);
        size_t o = 512;
        t.o_xl = int(o); o += size_t(t.Cin32) * 2 * t.Ppad * 16;
        t.o_e = int(o); o += size_t(t.Ce32) * 2 * t.Ppad * 16;
        t.o_w1 = int(o); o += w1_bytes;
        t.o_w2 = int(o); o += w2_bytes;
        t.o_wdw = int(o); o += wdw_bytes;
        t.o_tab = int(o); o += tab_bytes;
        t.o_ptab = int(o); o += size_t(t.Ppad) * 4;
        if (o > cap) continue;
        a = t;
        cap_used = o;
        best_time = time;
        found = true;
    }
    if (!found) return 1;
    if (!cached) {
        std::memset(&pval, 0, sizeof(pval));
        pval.a = a;
        pval.cap_used = cap_used;
        zant_plan_remember(slot, pkey, pval);
    }
    // position tiles a wave handles together in stage D: what its share of the tile needs, within the register budget
    {
        const int nq_tiles = (a.Q + 31) / 32;
        const int q_per_wave = (nq_tiles + 3) / 4;
        const int rounds = (q_per_wave + mq_cap - 1) / mq_cap;
        // fewer position tiles than waves: the waves share them chunk by chunk (their sums meet in the expanded patch's LDS)
        a.split = CO32 <= 2 && nq_tiles < 4 && nq_tiles <= mq_cap && a.Ce32 >= 2 &&
                  size_t(nq_tiles) * CO32 * 4096 <= size_t(a.Ce32) * 2 * a.Ppad * 16;
        out->MQv = a.split ? nq_tiles : std::max(1, (q_per_wave + rounds - 1) / rounds);
        out->CO32 = CO32;
        out->lds_bytes = cap_used;
    }
    if (plan_only) {
        out->a = a;
        out->packed = nullptr;
        return ZANT_OK;
    }
    if (!expand->w || !expand->w_scale || !dw->w || !dw->w_scale || !project->w || !project->w_scale)
        return ZANT_NullPointer;

    // packed weights and tables of the three convolutions
    const size_t kp1 = size_t(CeP), kp3 = size_t(CO32) * 32;
    // in the order and spacing of the kernel's LDS region [o_w1, o_ptab): weights of the expansion, of the projection, of
    // the depthwise convolution, then the tables m1 c1 m2 c2 (CeP entries each) m3 c3 (kp3 entries each)
    const size_t o_w1p = 256, o_w2p = o_w1p + w1_bytes, o_wm = o_w2p + w2_bytes, o_m1 = o_wm + wdw_bytes, o_c1 = o_m1 + kp1 * 4,
                 o_m2 = o_c1 + kp1 * 4, o_c2 = o_m2 + kp1 * 4, o_m3 = o_c2 + kp1 * 4, o_c3 = o_m3 + kp3 * 4,
                 static_bytes = align256(o_c3 + kp3 * 4);
    if (o_c3 + kp3 * 4 - o_w1p != w1_bytes + w2_bytes + wdw_bytes + tab_bytes || size_t(a.o_ptab - a.o_w1) != o_c3 + kp3 * 4 - o_w1p)
        return ZANT_InvalidInput;  // the two layouts must stay in step
    void *ws = nullptr, *dyn = nullptr;
    bool need_pack = true;
    int parity = 0;
    int rc = zant_pack_region(ctx, slot, static_bytes, 0, &ws, &dyn, &need_pack, &parity);
    if (rc) return rc;
    char *base = static_cast<char *>(ws);
    int8_t *w1p = reinterpret_cast<int8_t *>(base + o_w1p), *w2p = reinterpret_cast<int8_t *>(base + o_w2p);
    float *m1 = reinterpret_cast<float *>(base + o_m1), *m2 = reinterpret_cast<float *>(base + o_m2),
          *m3 = reinterpret_cast<float *>(base + o_m3);
    int32_t *c1 = reinterpret_cast<int32_t *>(base + o_c1), *c2 = reinterpret_cast<int32_t *>(base + o_c2),
            *c3 = reinterpret_cast<int32_t *>(base + o_c3);
    uint32_t *wmk = reinterpret_cast<uint32_t *>(base + o_wm);
    if (need_pack) {
        int8_t *padvec = reinterpret_cast<int8_t *>(base + 16);
        rc = zant_qpack_dense(ctx, expand->w, expand->w_scale, expand->n_wscale, expand->bias, int(Ce), int(Cin), 1, 32,
                              expand->x_scale, expand->x_zp, expand->y_scale, w1p, m1, c1, padvec);
        if (rc) return rc;
        rc = zant_qpack_depthwise(ctx, dw->w, dw->w_scale, dw->n_wscale, dw->bias, int(Ce), CeP, dw->x_scale, dw->x_zp,
                                  dw->y_scale, wmk, m2, c2);
        if (rc) return rc;
        rc = zant_qpack_dense(ctx, project->w, project->w_scale, project->n_wscale, project->bias, int(Co), int(Ce), 1, 32,
                              project->x_scale, project->x_zp, project->y_scale, w2p, m3, c3, padvec + 16);
        if (rc) return rc;
    }

    a.zp1f = float(expand->y_zp); a.zp2f = float(dw->y_zp); a.zp3f = float(project->y_zp);
    a.has_act1 = expand->act != ZANT_ACT_NONE;
    a.act1.act = expand->act; a.act1.alpha = expand->act_alpha; a.act1.in_scale = expand->y_scale; a.act1.in_zp = expand->y_zp;
    a.act1.out_scale = expand->act_scale; a.act1.out_zp = uint8_t(expand->act_zp);
    a.has_act2 = dw->act != ZANT_ACT_NONE;
    a.act2.act = dw->act; a.act2.alpha = dw->act_alpha; a.act2.in_scale = dw->y_scale; a.act2.in_zp = dw->y_zp;
    a.act2.out_scale = dw->act_scale; a.act2.out_zp = uint8_t(dw->act_zp);
    a.pad_e4 = uint32_t((dw->x_zp ^ 0x80) & 0xff) * 0x01010101u;
    a.half_last = (Ce % 32 != 0 && Ce % 32 <= 16) ? 1 : 0;
    a.has_res = residual ? 1 : 0;
    a.ra_scale = project->y_scale; a.ra_zp = project->y_zp;
    a.rb_scale = expand->x_scale; a.rb_zp = expand->x_zp;
    a.ry_scale = add_scale; a.ry_zp = add_zp;
    a.fast_div = residual && zant_fast_div_ok(a.ra_scale, a.rb_scale, add_scale);
    a.ry_rcp = a.fast_div ? zant_refined_rcp(add_scale) : 0.0f;

    a.packed_units = int((a.o_ptab - a.o_w1) / 16);
    out->a = a;
    out->packed = reinterpret_cast<const uint4 *>(base + o_w1p);
    return ZANT_OK;
}

}  // namespace

int zant_qblock_blocked(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], const zant_qconv_desc *expand,
                        const zant_qconv_desc *dw, int64_t dw_stride, const zant_qconv_desc *project, int residual,
                        float add_scale, int add_zp, uint8_t *y, const int64_t ydim[4], bool query_only, zant_pack_slot *slot) {
    QBlockPrep prep;
    if (!query_only && (!x || !y)) return ZANT_NullPointer;
    const int rc = qblock_prepare(ctx, xdim, expand, dw, dw_stride, project, residual, add_scale, add_zp, ydim, query_only, slot, 0, &prep);
    if (rc || query_only) return rc;
    const QBlockArgs &a = prep.a;
    const size_t cap_used = prep.lds_bytes;
    const int CO32 = prep.CO32, MQv = prep.MQv;
    const uint4 *packed = prep.packed;
    const int per_cu = cap_used <= 76 * 1024 ? 2 : 1;
    const int grid = int(std::min<int64_t>(a.n_tiles, int64_t(ctx->num_cus) * per_cu));
    KernelTimer kt(ctx);
#define ZANT_QBLOCK_LAUNCH(CO, M, P, S)                                                                                          \
    do {                                                                                                                    \
        if (!zant_raise_lds_limit(ctx, reinterpret_cast<const void *>(&qblock_kernel<CO, M, P, S>), 160 * 1024)) break;         \
        ZANT_KERNEL_NAME(ctx, "qblock_kernel<%d,%d,%s,%s>", CO, M, P ? "true" : "false", S ? "true" : "false");                                          \
        hipLaunchKernelGGL((qblock_kernel<CO, M, P, S>), dim3(grid), dim3(256), cap_used, ctx->stream,                           \
                           reinterpret_cast<const uint4 *>(x), y, packed, a);       \
    } while (0)
    switch ((a.split ? 100 : 0) + CO32 * 10 + MQv) {
    case 11: ZANT_QBLOCK_LAUNCH(1, 1, true, false); break;
    case 12: ZANT_QBLOCK_LAUNCH(1, 2, true, false); break;
    case 13: ZANT_QBLOCK_LAUNCH(1, 3, false, false); break;
    case 14: ZANT_QBLOCK_LAUNCH(1, 4, false, false); break;
    case 21: ZANT_QBLOCK_LAUNCH(2, 1, true, false); break;
    case 22: ZANT_QBLOCK_LAUNCH(2, 2, false, false); break;
    case 31: ZANT_QBLOCK_LAUNCH(3, 1, true, false); break;
    case 111: ZANT_QBLOCK_LAUNCH(1, 1, true, true); break;
    case 112: ZANT_QBLOCK_LAUNCH(1, 2, true, true); break;
    case 113: ZANT_QBLOCK_LAUNCH(1, 3, false, true); break;
    case 121: ZANT_QBLOCK_LAUNCH(2, 1, true, true); break;
    case 122: ZANT_QBLOCK_LAUNCH(2, 2, false, true); break;
    default: ZANT_QBLOCK_LAUNCH(4, 1, true, false); break;
    }
#undef ZANT_QBLOCK_LAUNCH
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// Blocks calls[0 .. n) as one launch (qblock_chain_kernel): ZANT_OK when they ran (with query_only: would run), 1 when
// they do not form a chain -- the caller then runs them one by one.  A chain needs whole-image tiles of one size, one
// tile per workgroup, one instantiation of the stage D register tiling for all its blocks, and each block's input to be
// the block before's output.
int zant_qblock_chain(zant_ctx *ctx, int n, const zant_qblock_call *calls, bool query_only) {
    if (!ctx || !calls) return ZANT_NullPointer;
    if (n < 2 || n > QB_CHAIN_MAX) return 1;
    QBlockChain chain;
    chain.n = n;
    size_t lds = 0;
    int CO32 = 0, MQv = 0, NB = 0, n_tiles = 0;
    for (int b = 0; b < n; ++b) {
        const zant_qblock_call &c = calls[b];
        if (!query_only && (!c.x || !c.y || (b > 0 && c.x != calls[b - 1].y))) return b > 0 && c.x && c.y ? 1 : ZANT_NullPointer;
        QBlockPrep prep;
        const int rc = qblock_prepare(ctx, c.xdim, c.expand, c.dw, c.dw_stride, c.project, c.residual, c.add_scale, c.add_zp, c.ydim,
                                      query_only, c.slot, NB, &prep);
        if (rc) return rc;
        if (prep.a.n_row_tiles != 1) return 1;
        if (b == 0) { CO32 = prep.CO32; MQv = prep.MQv; NB = prep.a.NB; n_tiles = prep.a.n_tiles; }
        else if (prep.CO32 != CO32 || prep.MQv != MQv || prep.a.NB != NB || prep.a.n_tiles != n_tiles) return 1;
        lds = std::max(lds, prep.lds_bytes);
        chain.link[b].x = reinterpret_cast<const uint4 *>(c.x);
        chain.link[b].y = c.y;
        chain.link[b].packed = prep.packed;
        chain.link[b].a = prep.a;
    }
    const int per_cu = lds <= 76 * 1024 ? 2 : 1;
    if (n_tiles > ctx->num_cus * per_cu) return 1;  // one tile per workgroup, all of them resident
    const int key = CO32 * 10 + MQv;
    if (key != 11 && key != 12 && key != 13 && key != 21 && key != 22) return 1;
    if (query_only) return ZANT_OK;
    KernelTimer kt(ctx);
#define ZANT_QCHAIN_LAUNCH(CO, M)                                                                                      \
    do {                                                                                                               \
        if (!zant_raise_lds_limit(ctx, reinterpret_cast<const void *>(&qblock_chain_kernel<CO, M>), 160 * 1024)) break; \
        ZANT_KERNEL_NAME(ctx, "qblock_chain_kernel<%d,%d> x %d", CO, M, n);                                            \
        hipLaunchKernelGGL((qblock_chain_kernel<CO, M>), dim3(n_tiles), dim3(256), lds, ctx->stream, chain);          \
    } while (0)
    switch (key) {
    case 11: ZANT_QCHAIN_LAUNCH(1, 1); break;
    case 12: ZANT_QCHAIN_LAUNCH(1, 2); break;
    case 13: ZANT_QCHAIN_LAUNCH(1, 3); break;
    case 21: ZANT_QCHAIN_LAUNCH(2, 1); break;
    default: ZANT_QCHAIN_LAUNCH(2, 2); break;
    }
#undef ZANT_QCHAIN_LAUNCH
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
