// Tiling shared by the implicit-GEMM convolution kernels (f32 and int8).
//
// A tile is NB whole images x TH whole output rows x all OW columns, for one block of output
// channels.  Per chunk of input channels a tile stages a patch of P1 = NB*PH*PW input positions.
// Both kernels use 32 bytes of LDS per patch position and chunk (8 f32 channels or 32 int8 channels)
// and T*32*K_BLK bytes per weight slab, so one planner serves both.
#pragma once
#include "common.h"

struct TileGeom {
    int NB, TH;          // images per workgroup tile, output rows per tile
    int PH, PW, P1;      // staged patch rows / cols, positions per chunk (NB*PH*PW)
    int P1s;             // P1 rounded up to a multiple of 4
    int n_row_tiles;     // ceil(OH / TH)
    int n_chunks;        // ceil(C / channels per chunk)
    int n_kblocks;       // ceil(K / K_BLK)
    int n_sblocks;       // spatial tiles
    int n_tiles;         // n_sblocks * n_kblocks
    int POW;             // fused 2x2/2 max pool: pooled columns (OW / 2); 0 = no pooling
    int x_c4;            // f32 kernel: the input is stored [N][C/4][H][W][4] (set by the launcher, not the planner)
};

struct TilePlan {
    int MT, WM, WN;
    TileGeom t;
    size_t lds_bytes;
    double eff;          // useful fraction of the MFMA columns
    double score;        // eff weighted by how much of the GPU the tiles fill (what plans are ranked by)
};

// Tile id -> first image, first output row, output-channel block.  XCD-aware: consecutive
// workgroups sit on different XCDs, so each XCD gets a contiguous run of spatial tiles (halo rows
// then hit that XCD's own L2).
__device__ __forceinline__ void decode_tile(const TileGeom &t, int tile, int &n0, int &oh0, int &kb) {
    kb = tile % t.n_kblocks;
    int sb = tile / t.n_kblocks;
    if ((t.n_sblocks & 7) == 0) sb = (sb & 7) * (t.n_sblocks >> 3) + (sb >> 3);
    const int ig = sb / t.n_row_tiles;
    n0 = ig * t.NB;
    oh0 = (sb - ig * t.n_row_tiles) * t.TH;
}

// Best tile shape for WM x WN waves (WN*32 output channels per workgroup) among MT = mt_max..1 whose
// two staging buffers, patch table and scheduler slots fit in `lds_cap` bytes.
// chunk_channels: input channels per chunk; elem_bytes: bytes per input element.
// pool: the kernel's epilogue max-pools 2x2/2 (floor).  The MFMA column slots are then counted in POOLED positions:
// tile registers 4j..4j+3 of a lane hold the four members of one window, so MT is a multiple of 4, TH is even and
// a tile covers NB images x TH/2 pooled rows x OW/2 pooled columns.
// target_tiles > 0 (= 2 x CUs, the workgroup slots of the GPU): plans are ranked by an estimate of the kernel time,
// the larger of (a) the MFMA time of the busiest workgroup slot -- which penalises padding lanes and layers too small
// to give every slot a tile -- and (b) the time to copy every tile's operands from L2 into LDS at ~6 TB/s: the int8
// matrix cores outrun that copy stream for all but the largest tiles, so operand reuse per staged byte decides.
// mfma_cycles_per_tap: matrix-core cycles per wave, filter tap and position tile of one chunk.
// copy_threads > 0: the kernel pads the patch region to one 32-byte slot and the weight slab to one 16-byte unit per
// copying thread and round, and keeps 8 bytes of requantisation table per output channel in LDS; the footprint and the
// staging estimate then count those padded sizes.
// n_buffers: staging buffers that must fit (2 = double buffering; more for a deeper copy ring).
// extra_bytes_per_pos: LDS the kernel keeps per patch position beyond the 8 bytes counted here (may be negative).
// max_nb, max_patch_dim: limits of the kernel's packed patch table (images per tile; patch rows and columns).
inline bool zant_plan_conv_tiles(const ConvGeom &g, int WM, int WN, int mt_max, int chunk_channels, size_t elem_bytes,
                                 size_t lds_cap, TilePlan *best, bool pool = false, int target_tiles = 0,
                                 int mfma_cycles_per_tap = 32, int copy_threads = 0, int n_buffers = 2,
                                 int extra_bytes_per_pos = 0, int max_nb = 1 << 15, int max_patch_dim = 1 << 16) {
    const int T = g.KH * g.KW;
    const int K_BLK = WN * 32;
    bool found = false;
    for (int mt = mt_max; mt >= 1; --mt) {
        if (pool && (mt & 3)) continue;
        const int S = pool ? WM * (mt / 4) * 32 : WM * mt * 32;      // position slots (pooled positions when pooling)
        const int rows = pool ? g.OH / 2 : g.OH, cols = pool ? g.OW / 2 : g.OW;
        if (rows < 1 || cols < 1) continue;
        const int per_img = rows * cols;
        TileGeom t;
        t.x_c4 = 0;
        t.POW = pool ? cols : 0;
        int th;  // rows (pooled rows) per tile
        if (per_img <= S) {
            t.NB = S / per_img; th = rows;
            if (t.NB > g.N) t.NB = g.N;
        } else {
            t.NB = 1; th = S / cols;
            if (th < 1) continue;
        }
        t.n_row_tiles = (rows + th - 1) / th;
        th = (rows + t.n_row_tiles - 1) / t.n_row_tiles;  // even out the rows over the row tiles
        t.TH = pool ? 2 * th : th;
        t.PH = (t.TH - 1) * g.sh + (g.KH - 1) * g.dh + 1;
        t.PW = (g.OW - 1) * g.sw + (g.KW - 1) * g.dw + 1;
        t.P1 = t.NB * t.PH * t.PW;
        t.P1s = copy_threads > 0 ? (t.P1 + copy_threads - 1) / copy_threads * copy_threads : (t.P1 + 3) & ~3;
        if (t.PH >= max_patch_dim || t.PW >= max_patch_dim || t.NB >= max_nb) continue;  // packed into one int of the patch table
        if (int64_t(t.NB) * g.C * g.H * g.W * int64_t(elem_bytes) >= (int64_t(1) << 31)) continue;  // 32-bit offsets per image group
        t.n_chunks = (g.C + chunk_channels - 1) / chunk_channels;
        t.n_kblocks = (g.K + K_BLK - 1) / K_BLK;
        t.n_sblocks = ((g.N + t.NB - 1) / t.NB) * t.n_row_tiles;
        const int64_t n_tiles = int64_t(t.n_sblocks) * t.n_kblocks;
        if (n_tiles >= (int64_t(1) << 30)) continue;
        t.n_tiles = int(n_tiles);
        size_t w_slab = size_t(T) * 32 * K_BLK, fixed = size_t(t.P1s) * 8 + 8;  // fixed: patch table, scheduler slots
        if (copy_threads > 0) {
            const size_t round = size_t(copy_threads) * 16;
            w_slab = (w_slab + round - 1) / round * round;
            fixed = size_t(t.P1s) * 8 + 512 + size_t(t.n_kblocks) * K_BLK * 8;
        }
        fixed = size_t(int64_t(fixed) + int64_t(extra_bytes_per_pos) * t.P1s);  // the kernel's own per-position tables
        const size_t lds = n_buffers * (w_slab + size_t(32) * t.P1s) + fixed;  // the staging buffers
        if (lds > lds_cap) continue;
        const double eff = double(g.N) * rows * cols / (double(t.n_sblocks) * S);
        double score = eff;
        if (target_tiles > 0) {
            const double rounds = double((t.n_tiles + target_tiles - 1) / target_tiles);
            const double mfma = rounds * 2.0 * t.n_chunks * mt * T * mfma_cycles_per_tap;                 // cycles
            const double stage = double(t.n_tiles) * t.n_chunks * (double(w_slab) + 32.0 * t.P1s) / 7000.0;  // cycles at the measured L2 -> LDS copy rate (17 TB/s and up)
            score = 1.0e6 / (mfma > stage ? mfma : stage);
        }
        if (!found || score > best->score * 1.02) {  // larger tiles win ties: fewer tiles, more operand reuse
            best->MT = mt; best->WM = WM; best->WN = WN; best->t = t; best->lds_bytes = lds; best->eff = eff;
            best->score = score;
            found = true;
        }
    }
    return found;
}

// LDS bank conflicts of the operand reads of a tile plan, as a function of the patch row pitch.  A lane reads the
// 16-byte unit of its position slot; the LDS serves 16 such units per cycle when they lie in 16 different groups of four
// banks (unit index mod 16), and takes one more cycle for every further distinct unit of a group.  Consecutive lanes
// take consecutive positions of the (pooled) output, so the units a pass touches are spaced by the stride, by two
// columns with a fused pool, by a patch row at a row change and by a patch image at an image change: on small maps a
// pitch of 8 or 16 units puts whole columns of the tile into the same banks.  Returns the average number of cycles per
// 16-lane pass (1 = conflict-free) for patch rows of `pw` units.
inline double zant_patch_read_cycles(const TilePlan &p, const ConvGeom &g, bool pool, int pw) {
    const TileGeom &t = p.t;
    const int per_img = t.TH * g.OW, per_img_p = pool ? (t.TH / 2) * t.POW : 1;
    long total = 0, passes = 0;
    for (int wm = 0; wm < p.WM; ++wm)
        for (int i = 0; i < p.MT; ++i)
            for (int half = 0; half < 2; ++half) {
                int unit[16], n_unit = 0, load[16] = {0};
                for (int l = half * 16; l < half * 16 + 16; ++l) {
                    int img, r, c;
                    if (pool) {
                        const int pp = (wm * (p.MT / 4) + i / 4) * 32 + l;
                        img = pp / per_img_p;
                        const int rem = pp - img * per_img_p, pr = rem / t.POW;
                        r = 2 * pr + ((i & 3) >> 1);
                        c = 2 * (rem - pr * t.POW) + (i & 1);
                    } else {
                        const int q = (wm * p.MT + i) * 32 + l;
                        img = q / per_img;
                        const int rem = q - img * per_img;
                        r = rem / g.OW;
                        c = rem - r * g.OW;
                    }
                    const int u = (img < t.NB && r < t.TH) ? (img * t.PH + r * g.sh) * pw + c * g.sw : 0;
                    bool seen = false;
                    for (int k = 0; k < n_unit; ++k) seen |= unit[k] == u;
                    if (!seen) { unit[n_unit++] = u; ++load[u & 15]; }
                }
                int worst = 1;
                for (int b = 0; b < 16; ++b) worst = load[b] > worst ? load[b] : worst;
                total += worst;
                ++passes;
            }
    return double(total) / double(passes);
}

