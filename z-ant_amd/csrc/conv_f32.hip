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
#include <algorithm>
#include <mutex>

#include "conv_tile.h"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

constexpr int CC = 8;  // input channels staged per chunk (4 MFMA k-steps per filter tap)


// Packs OIHW weights into [chunk][kblock][tap][half][K_BLK][4] (zero padded):
// element (half, k, j) holds W[k][chunk*8 + half*4 + j][tap].  A chunk's slab is one contiguous
// 16-byte aligned run, and one 128-bit LDS read per lane fetches the A operands of 4 k-steps.
// Thread 0 also resets the tile counter the persistent convolution workgroups draw from.
__global__ void pack_weights_f32_kernel(const float *__restrict__ w, float *__restrict__ wp, int K, int C, int T,
                                        int n_chunks, int n_kblocks, int k_blk, int *__restrict__ tile_counter,
                                        int counter_init) {
    const int64_t total = int64_t(n_chunks) * n_kblocks * T * CC * k_blk;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    if (blockIdx.x == 0 && threadIdx.x == 0) *tile_counter = counter_init;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        int64_t r = i;
        const int j = int(r & 3); r >>= 2;
        const int kk = int(r % k_blk); r /= k_blk;
        const int half = int(r & 1); r >>= 1;
        const int tap = int(r % T); r /= T;
        const int kb = int(r % n_kblocks); r /= n_kblocks;
        const int chunk = int(r);
        const int k = kb * k_blk + kk, c = chunk * CC + half * 4 + j;
        wp[i] = (k < K && c < C) ? w[(int64_t(k) * C + c) * T + tap] : 0.0f;
    }
}

// LDS byte address of a pointer into the workgroup's shared memory.
__device__ __forceinline__ unsigned lds_addr_of(const void *p) {
    return unsigned(reinterpret_cast<uintptr_t>((lptr_t) const_cast<void *>(p)));
}
// Starts a 32-bit LDS read without the compiler's knowledge (it inserts no waits of its own for it) ...
__device__ __forceinline__ int lds_read32_async(unsigned addr) {
    int v;
    asm volatile("ds_read_b32 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
// ... and this waits for every outstanding LDS operation; the values are in/out operands so that their users stay
// behind the wait.
__device__ __forceinline__ void lds_wait_all(int &a, int &b, int &c, int &d) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// max without the NaN-quieting pass the compiler puts in front of fmaxf (an MFMA result is never a signalling NaN); a NaN
// operand yields the other one, like fmaxf
__device__ __forceinline__ float vmax(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float vmax3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// S: window-packed tiles of the pooled kernel, window slots per tile.  Every kernel: the tiles from `tail_start` on
// (tail_n of them, the last partial round) are handed out one per workgroup, to workgroups 0 .. tail_n-1.
struct PackGeom { int S, tail_start, tail_n; };

// A few zero words that padding lanes of the asynchronous global->LDS copies read from.
__device__ __align__(16) float g_zero_words[4] = {0.f, 0.f, 0.f, 0.f};

// One (tile, chunk) step of the pipeline: start the asynchronous global->LDS copies of the NEXT step
// into `dma` and run the matrix cores over THIS step's operands in `cmp`.
//
// The three LDS regions are passed as __restrict__ pointers on purpose: `dma`, `cmp` and `ttab` never
// overlap within a step, and saying so is what lets the compiler leave the copies in flight across
// the LDS reads of this step instead of draining them (vmcnt(0)) before the first one.
template <int MT, int WM, int WN, int KV, int TT>
__device__ __forceinline__ void conv_step(float *__restrict__ dma, const float *__restrict__ cmp,
                                          const int *__restrict__ ttab, const float *__restrict__ x,
                                          const float *__restrict__ wp, const ConvGeom &g, const TileGeom &t,
                                          bool do_issue, int n0, int kb, int ichunk, int p1, const int (&lds_off)[MT],
                                          f32x16 (&acc)[MT]) {
    constexpr int NT = WM * WN * 64;
    constexpr int K_BLK = WN * 32;
    constexpr int PPI = NT / 4;  // patch positions covered by one staging instruction of the workgroup
    const int T = TT > 0 ? TT : g.KH * g.KW;
    const int w_chunk = T * CC * K_BLK;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction; says so to the compiler (LDS
                                                                // copy destinations then stay in scalar registers)
    const int wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;

    if (do_issue) {
        float *xl = dma + w_chunk;
        // weight slab: contiguous 16-byte units, lane-consecutive in LDS
        const float *wsrc = wp + (int64_t(ichunk) * t.n_kblocks + kb) * w_chunk;
        const int units = w_chunk >> 2;
        for (int u0 = 0; u0 < units; u0 += NT) {
            const int u = u0 + tid;
            if (u < units)
                __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + u * 4), (lptr_t)(dma + (u0 + wave * 64) * 4), 16, 0, 0);
        }
        // input patch: lane -> (position, channel j of a half); zero words for padding.  The tile's table gives each
        // position's element offset inside the image group (or -1), so a copy costs an add, a compare and the selects:
        // whatever is decided here per step is paid in matrix-pipe time.
        const int64_t x_plane = int64_t(g.H) * g.W;
        const unsigned ttab_addr = lds_addr_of(ttab);
        if (t.x_c4) {
            // Quad-blocked input ([N][C/4][H][W][4]): the four channels of a chunk half at one position are 16 contiguous
            // bytes, which is also how the patch sits in LDS -- one copy per position and half, a quarter of the copy
            // instructions of the NCHW form below (a wave pays ~130 cycles for each, whatever its size).
            const float *q0 = x + int64_t(n0) * g.C * x_plane + int64_t(ichunk * (CC / 4)) * x_plane * 4;
            const float *q1 = q0 + x_plane * 4;
            const bool h_ok1 = ichunk * CC + 4 < g.C;
            for (int p0 = 0; p0 < p1; p0 += 2 * NT) {
                int e[2], pad0 = 0, pad1 = 0;
#pragma unroll
                for (int u = 0; u < 2; ++u) e[u] = lds_read32_async(ttab_addr + unsigned(min(p0 + u * NT + tid, p1 - 1)) * 4u);
                lds_wait_all(e[0], e[1], pad0, pad1);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    if (p0 + u * NT + tid < p1) {
                        const bool ok = e[u] >= 0;
                        const float *sp0 = ok ? q0 + unsigned(e[u]) : g_zero_words;
                        const float *sp1 = (ok && h_ok1) ? q1 + unsigned(e[u]) : g_zero_words;
                        __builtin_amdgcn_global_load_lds((gptr_t)sp0, (lptr_t)(xl + (p0 + u * NT + wave * 64) * 4), 16, 0, 0);
                        __builtin_amdgcn_global_load_lds((gptr_t)sp1, (lptr_t)(xl + (t.P1s + p0 + u * NT + wave * 64) * 4), 16, 0, 0);
                    }
                }
            }
        } else {
        const int j = tid & 3;
        const float *b0 = x + (int64_t(n0) * g.C + ichunk * CC) * x_plane;  // wave-uniform: channel ichunk*CC of image n0
        const float *b1 = b0 + 4 * x_plane;
        const bool c_ok0 = ichunk * CC + j < g.C, c_ok1 = ichunk * CC + 4 + j < g.C;
        const int jplane = j * int(x_plane);  // NB * C * H * W * 4 < 2^31 is checked on the host
        // The table lives in LDS.  The compiler drains every outstanding asynchronous copy before an LDS read
        // it issues itself in this loop (one round trip to L2 per iteration, which made staging cost ~18 % of a
        // step), so the table is read with hand-written ds_read_b32, one iteration ahead of its use.
        for (int p0 = 0; p0 < p1; p0 += 4 * PPI) {
            // four table entries per round; nothing read this way stays in flight across a loop edge (a register
            // copy there would run before the data has landed)
            int e[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                e[u] = lds_read32_async(ttab_addr + unsigned(min(p0 + u * PPI + (tid >> 2), p1 - 1)) * 4u);
            lds_wait_all(e[0], e[1], e[2], e[3]);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int pos = p0 + u * PPI + (tid >> 2);
                if (pos < p1) {
                    const bool ok = e[u] >= 0;
                    const unsigned vo = unsigned(e[u] + jplane);
                    const float *sp0 = (ok && c_ok0) ? b0 + vo : g_zero_words;
                    const float *sp1 = (ok && c_ok1) ? b1 + vo : g_zero_words;
                    __builtin_amdgcn_global_load_lds((gptr_t)sp0, (lptr_t)(xl + (p0 + u * PPI + wave * 16) * 4), 4, 0, 0);
                    __builtin_amdgcn_global_load_lds((gptr_t)sp1, (lptr_t)(xl + (t.P1s + p0 + u * PPI + wave * 16) * 4), 4, 0, 0);
                }
            }
        }
        }
    }

    // keep the copy-issue code and the MFMA loop apart: interleaving them only adds register pressure
    __builtin_amdgcn_sched_barrier(0);

    typedef float vkv __attribute__((ext_vector_type(KV)));
    constexpr int SUBS = 4 / KV;  // LDS reads per tap and operand
    const float *wlf = cmp + (lh * K_BLK + wn * 32 + l32) * 4;
    const float *xlf = cmp + w_chunk + lh * t.P1s * 4;
    vkv a0, a1, b0[MT], b1[MT];
    int lkh = 0, lkw = 0, ltap = 0, lsub = 0;  // what the next load_grp() call fetches
    auto load_grp = [&](vkv &a, vkv (&b)[MT]) {
        const int off = (lkh * g.dh * t.PW + lkw * g.dw) * 4 + lsub * KV;
        a = *reinterpret_cast<const vkv *>(wlf + ltap * 2 * K_BLK * 4 + lsub * KV);
#pragma unroll
        for (int i = 0; i < MT; ++i) b[i] = *reinterpret_cast<const vkv *>(xlf + lds_off[i] * 4 + off);
        if (++lsub == SUBS) {
            lsub = 0;
            ++ltap;
            if (++lkw == g.KW) { lkw = 0; ++lkh; }
        }
    };
    // MFMAs of k-steps [j0, j1) of a group.  Raised priority for the burst: of the two waves sharing a
    // SIMD, the one that reaches its burst first keeps the matrix core and the other fetches operands
    // meanwhile, instead of both interleaving bursts and then both stalling together.
    auto mfma_part = [&](const vkv &a, const vkv (&b)[MT], int j0, int j1) {
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int j = 0; j < KV; ++j)
            if (j >= j0 && j < j1) {
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[j], b[i][j], acc[i], 0, 0, 0);
            }
        __builtin_amdgcn_s_setprio(0);
    };
    // One group: the next group's operand reads are issued in the middle of this group's MFMAs, so
    // they have half a burst to land before anything waits on them.
    auto run_grp = [&](const vkv &a, const vkv (&b)[MT], vkv &an, vkv (&bn)[MT], bool more) {
        mfma_part(a, b, 0, KV / 2);
        if (more) load_grp(an, bn);
        mfma_part(a, b, KV / 2, KV);
    };
    if (TT > 0) {
        constexpr int N_GRP = (TT > 0 ? TT : 1) * SUBS;
        load_grp(a0, b0);
#pragma unroll
        for (int gp = 0; gp < N_GRP; gp += 2) {
            run_grp(a0, b0, a1, b1, gp + 1 < N_GRP);
            if (gp + 1 < N_GRP) run_grp(a1, b1, a0, b0, gp + 2 < N_GRP);
        }
    } else {
        const int n_grp = T * SUBS;
        load_grp(a0, b0);
        for (int gp = 0; gp < n_grp; gp += 2) {
            run_grp(a0, b0, a1, b1, gp + 1 < n_grp);
            if (gp + 1 < n_grp) run_grp(a1, b1, a0, b0, gp + 2 < n_grp);
        }
    }
}

// Persistent implicit-GEMM convolution.
//   MT: 32-position MFMA tiles per wave; WM x WN waves per workgroup (positions x output channels);
//   KV: k-steps fetched per LDS read (4 = 128-bit reads; 2 = 64-bit reads, fewer registers for MT = 8);
//   TT: filter taps KH*KW when known at compile time (the tap loop is then fully unrolled, which lets
//       the compiler count outstanding LDS reads exactly instead of draining them at a loop edge), 0 = any.
// LDS holds two staging buffers, each [weights: T][2][K_BLK][4] + [patch: 2][P1s][4]: the 8 channels
// of a chunk are split in two halves (one per MFMA k index) and the 4 channels of a half sit next to
// each other, so ONE 128-bit LDS read per lane feeds 4 MFMA k-steps.  Global->LDS copies are
// asynchronous (global_load_lds, no VGPR round trip) and run one (tile, chunk) step ahead of the
// matrix cores, across tile boundaries as well: while a tile's bias/ReLU epilogue stores drain, the
// first chunk of the workgroup's next tile is already landing.  Tiles are drawn from an atomic counter.
//
// PACK (with POOL, whole pooled images smaller than a tile's window slots): a tile is not a group of whole images but S
// consecutive pooling windows of the batch's flat window sequence, wherever in an image they start, so no slot is empty
// (25 windows per image fill 50 of 64 slots otherwise).  The patch holds every image the run of windows touches (t.NB =
// the most that can be); a lane's window, its patch offset and its output position change from tile to tile and come
// from a per-workgroup table indexed by the window's number inside the staged images.
template <int MT, int WM, int WN, int KV, int TT, bool POOL = false, bool PACK = false>
__global__ void __launch_bounds__(WM *WN * 64, 2)
conv_f32_mfma_kernel(const float *__restrict__ x, const float *__restrict__ wp, const float *__restrict__ bias,
                     float *__restrict__ y, ConvGeom g, TileGeom t, int relu, int *__restrict__ tile_counters, int parity,
                     PackGeom pk) {
    static_assert(!PACK || POOL, "window packing belongs to the fused pool");
    constexpr int NT = WM * WN * 64;
    constexpr int K_BLK = WN * 32;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int T = TT > 0 ? TT : g.KH * g.KW;
    const int w_chunk = T * CC * K_BLK;          // floats per (chunk, kblock) weight slab
    const int buf_floats = w_chunk + CC * t.P1s;  // one staging buffer
    float *buf0 = lds, *buf1 = lds + buf_floats;
    int *ptab = reinterpret_cast<int *>(lds + 2 * buf_floats);     // [P1s]: img << 24 | patch row << 12 | patch column
    int *ttab0 = ptab + (PACK ? 0 : t.P1s);                        // [2][P1s]: per tile, a position's element offset in
    int *ttab1 = ttab0 + t.P1s;                                    //   the image group, -1 where the patch is padding
    int *sched = ttab1 + t.P1s;                                    // [2]: tile ids handed out by thread 0; [2]: tail tile taken
    float *bias_l = reinterpret_cast<float *>(sched + 4);          // [n_kblocks * K_BLK]: the bias, zero past K
    int *wtab = reinterpret_cast<int *>(bias_l + t.n_kblocks * K_BLK);  // PACK: [NB * windows per image][2]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction; says so to the compiler (LDS
                                                                // copy destinations then stay in scalar registers)
    const int wm = wave % WM, wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;
    const int64_t x_img = int64_t(g.C) * g.H * g.W;
    const int per_img = t.TH * g.OW;
    const int patch_hw = t.PH * t.PW;

    // ---- once per workgroup: the tile-independent part of the patch geometry ----
    // (PACK keeps no such table: its larger patches need the room, and a tile's table costs two divisions per entry)
    if constexpr (!PACK)
    for (int e = tid; e < t.P1; e += NT) {
        const int img = e / patch_hw, rem = e - img * patch_hw;
        const int ph = rem / t.PW, pw = rem - ph * t.PW;
        ptab[e] = (img << 24) | (ph << 12) | pw;  // NB < 256, PH and PW < 4096: the planner's limits
    }
    // With a fused 2x2/2 max pool the lane's tile registers 4j .. 4j+3 are the four members of ONE pooling window
    // (pooled position (wm*MT/4 + j)*32 + l32), so the pool is a register-wise max in the epilogue.
    const int per_img_p = POOL ? (t.TH / 2) * t.POW : 1;
    int lds_off[MT];  // float4 index of each of this lane's output positions inside a patch half
    if constexpr (PACK) {
        // window w of the staged images -> { patch unit of its first member, image << 20 | pooled row << 10 | column }
        for (int w = tid; w < t.NB * per_img_p; w += NT) {
            const int img = w / per_img_p, rem = w - img * per_img_p;
            const int pr = rem / t.POW, pc = rem - pr * t.POW;
            wtab[2 * w] = (img * t.PH + 2 * pr * g.sh) * t.PW + 2 * pc * g.sw;
            wtab[2 * w + 1] = (img << 20) | (pr << 10) | pc;
        }
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        int img, r, c;
        if (PACK) {
            img = r = c = 0;  // set per tile
        } else if (POOL) {
            const int pp = (wm * (MT / 4) + i / 4) * 32 + l32;
            img = pp / per_img_p;
            const int rem = pp - img * per_img_p, pr = rem / t.POW;
            r = 2 * pr + ((i & 3) >> 1);
            c = 2 * (rem - pr * t.POW) + (i & 1);
        } else {
            const int p = (wm * MT + i) * 32 + l32;
            img = p / per_img;
            const int rem = p - img * per_img;
            r = rem / g.OW; c = rem - r * g.OW;
        }
        lds_off[i] = (img < t.NB && r < t.TH) ? (img * t.PH + r * g.sh) * t.PW + c * g.sw : 0;
    }
    // The bias goes to LDS once: read per tile from global memory, its 16 scattered loads sat in every epilogue with
    // their full latency exposed (the accumulators are done, nothing else is left to do).
    for (int k = tid; k < t.n_kblocks * K_BLK; k += NT) bias_l[k] = (bias != nullptr && k < g.K) ? bias[k] : 0.0f;
    // pooled position slot j of this lane inside a tile: image << 20 | pooled row << 10 | pooled column
    int pool_pos[POOL ? MT / 4 : 1];
    if constexpr (PACK) {
#pragma unroll
        for (int j = 0; j < MT / 4; ++j) pool_pos[j] = 0;  // set per tile
    } else if constexpr (POOL) {
#pragma unroll
        for (int j = 0; j < MT / 4; ++j) {
            const int pp = (wm * (MT / 4) + j) * 32 + l32;
            const int img = pp / per_img_p, rem = pp - img * per_img_p;
            const int pr = rem / t.POW, pc = rem - pr * t.POW;
            pool_pos[j] = (min(img, 1023) << 20) | (min(pr, 1023) << 10) | min(pc, 1023);
        }
    } else {
        pool_pos[0] = 0;
    }
    // likewise the unpooled position slots: image << 24 | row << 12 | column (NB < 256, rows and columns < 4096: the
    // planner's limits)
    int out_pos[POOL ? 1 : MT];
    if constexpr (!POOL) {
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int p = (wm * MT + i) * 32 + l32;
            const int img = p / per_img, rem = p - img * per_img;
            const int r = rem / g.OW, c = rem - r * g.OW;
            out_pos[i] = (min(img, 255) << 24) | (min(r, 4095) << 12) | min(c, 4095);
        }
    } else {
        out_pos[0] = 0;
    }
    if (tid == 0) {
        sched[0] = blockIdx.x + gridDim.x;  // the second tile is static, later ones come from the counter
        sched[2] = 0;
    }
    // Two counters take turns: this launch draws from tile_counters[parity] and re-arms the other one for the next
    // launch of the same operator, so that packed weights and counters can be kept across calls without a reset pass.
    if (tid == 0 && blockIdx.x == 0) tile_counters[parity ^ 1] = 2 * int(gridDim.x);
    __syncthreads();

    // A tile's table: which patch positions exist for this tile (rows above / below the image and images past the
    // batch do not) and where they are.  Built once per tile by the whole workgroup, read by every step's copies.
    auto fill_ttab = [&](int *tt, int n0, int oh0, int p1) {
        const int ih0 = oh0 * g.sh - g.pt;
        const int imgs_here = min(t.NB, g.N - n0);
        for (int e = tid; e < p1; e += NT) {
            int img, ih, iw;
            if constexpr (PACK) {
                img = e / patch_hw;
                const int rem = e - img * patch_hw, ph = rem / t.PW;
                ih = ih0 + ph;
                iw = rem - ph * t.PW - g.pl;
            } else {
                const int v = ptab[e];
                img = int(unsigned(v) >> 24); ih = ih0 + ((v >> 12) & 0xfff); iw = (v & 0xfff) - g.pl;
            }
            const bool ok = iw >= 0 && iw < g.W && ih >= 0 && ih < g.H && img < imgs_here;
            // (quad-blocked input: four floats per position inside a quad's plane)
            tt[e] = ok ? img * int(x_img) + (ih * g.W + iw) * (t.x_c4 ? 4 : 1) : -1;  // NB*C*H*W*4 < 2^31 is checked on the host
        }
    };

    int cur = blockIdx.x;
    if (cur >= t.n_tiles) return;
    f32x16 acc[MT];
    // Tiles are decoded once, when their id is known, and the id is made wave-uniform first: decoded per step from the
    // LDS slot (a vector register) the divisions ran in the vector unit, some sixty instructions per step.
    int cn0, coh0, ckb, nn0 = 0, noh0 = 0, nkb = 0;
    int cp1 = t.P1, np1 = t.P1;  // patch positions staged for the tile (PACK: only the images its windows touch)
    int noff = 0;                // PACK: the tile's first window inside its first image
    auto decode = [&](int tile, int &n0, int &oh0, int &kb, int &off, int &p1) {
        if constexpr (PACK) {
            kb = tile % t.n_kblocks;
            int sb = tile / t.n_kblocks;
            if ((t.n_sblocks & 7) == 0) sb = (sb & 7) * (t.n_sblocks >> 3) + (sb >> 3);  // a contiguous run per XCD
            const int w0 = sb * pk.S;  // N * windows per image + S < 2^31 is checked on the host
            n0 = w0 / per_img_p;
            off = w0 - n0 * per_img_p;
            oh0 = 0;
            p1 = min((off + pk.S - 1) / per_img_p + 1, g.N - n0) * patch_hw;
        } else {
            decode_tile(t, tile, n0, oh0, kb);
            off = 0;
            p1 = t.P1;
        }
    };
    // PACK: the lane's window slots of a tile starting `off` windows into its first image
    auto set_slots = [&](int off) {
        if constexpr (PACK) {
#pragma unroll
            for (int j = 0; j < MT / 4; ++j) {
                const int wl = off + (wm * (MT / 4) + j) * 32 + l32;  // < NB * per_img_p: NB is the longest run's span
                const int base = wtab[2 * wl];
                pool_pos[j] = wtab[2 * wl + 1];
#pragma unroll
                for (int i = 0; i < 4; ++i) lds_off[4 * j + i] = base + (i >> 1) * g.sh * t.PW + (i & 1) * g.sw;
            }
        }
    };
    {
        int coff;
        decode(cur, cn0, coh0, ckb, coff, cp1);
        set_slots(coff);
    }
    fill_ttab(ttab0, cn0, coh0, cp1);
    __syncthreads();
    // prologue: copies of the first step, with nothing to compute yet
    {
        const float *wsrc = wp + int64_t(ckb) * w_chunk;
        const int units = w_chunk >> 2;
        for (int u0 = 0; u0 < units; u0 += NT) {
            const int u = u0 + tid;
            if (u < units)
                __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + u * 4), (lptr_t)(buf0 + (u0 + wave * 64) * 4), 16, 0, 0);
        }
        const int64_t x_plane = int64_t(g.H) * g.W;
        const float *xb = x + int64_t(cn0) * x_img;
        const int j = tid & 3;
        float *xl = buf0 + w_chunk;
        if (t.x_c4) {
            for (int p0 = 0; p0 < cp1; p0 += NT) {
                const int pos = p0 + tid;
                if (pos < cp1) {
                    const int e = ttab0[pos];
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const float *sp = (e >= 0 && half * 4 < g.C) ? xb + e + int64_t(half) * x_plane * 4 : g_zero_words;
                        __builtin_amdgcn_global_load_lds((gptr_t)sp, (lptr_t)(xl + (half * t.P1s + p0 + wave * 64) * 4), 16, 0, 0);
                    }
                }
            }
        } else
        for (int p0 = 0; p0 < cp1; p0 += NT / 4) {
            const int pos = p0 + (tid >> 2);
            if (pos < cp1) {
                const int e = ttab0[pos];
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int c = half * 4 + j;
                    const float *sp = (e >= 0 && c < g.C) ? xb + e + int64_t(c) * x_plane : g_zero_words;
                    __builtin_amdgcn_global_load_lds((gptr_t)sp, (lptr_t)(xl + (half * t.P1s + p0 + wave * 16) * 4), 4, 0, 0);
                }
            }
        }
    }
    int step = 0;  // flattened (tile, chunk) counter; its parity selects the staging buffer
    int tile_par = 0;
    while (cur < t.n_tiles) {
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
        int nxt = t.n_tiles;
        for (int chunk = 0; chunk < t.n_chunks; ++chunk, ++step) {
            __builtin_amdgcn_s_waitcnt(0);  // this thread's copies for this step have landed
            __syncthreads();                // ... everyone's have; all waves are done with the other buffer
            if (chunk == 0) {
                nxt = __builtin_amdgcn_readfirstlane(sched[tile_par]);  // written at least one barrier ago
                if (tid == 0) {
                    int drawn = atomicAdd(tile_counters + parity, 1);
                    // The tiles of a last round that fills at most one workgroup per CU belong to the first workgroups by
                    // number, one each (they sit on different CUs): drawn freely, two of them land on one CU -- its two
                    // workgroups finish together -- and run at half speed while other CUs idle, a whole round again.
                    if (drawn >= pk.tail_start) {
                        drawn = (sched[2] == 0 && int(blockIdx.x) < pk.tail_n) ? pk.tail_start + int(blockIdx.x) : t.n_tiles;
                        sched[2] = 1;
                    }
                    sched[tile_par ^ 1] = drawn;
                }
                if (nxt < t.n_tiles) {
                    decode(nxt, nn0, noh0, nkb, noff, np1);
                    // no copy is in flight here (the wait above), and the slot's last readers were the copies of the
                    // previous tile; its first readers come a barrier later unless the tile has a single chunk
                    fill_ttab(tile_par ? ttab0 : ttab1, nn0, noh0, np1);
                    if (t.n_chunks == 1) __syncthreads();
                }
            }
            const bool same_tile = chunk + 1 < t.n_chunks;
            const bool do_issue = same_tile || nxt < t.n_tiles;
            const int ichunk = same_tile ? chunk + 1 : 0;
            float *dma = (step & 1) ? buf0 : buf1;
            const float *cmp = (step & 1) ? buf1 : buf0;
            const int *ttab = (same_tile ? tile_par == 0 : tile_par != 0) ? ttab0 : ttab1;  // tile k's table is slot k & 1
            conv_step<MT, WM, WN, KV, TT>(dma, cmp, ttab, x, wp, g, t, do_issue, same_tile ? cn0 : nn0, same_tile ? ckb : nkb,
                                          ichunk, same_tile ? cp1 : np1, lds_off, acc);
        }

        // ---- epilogue: bias (+ReLU), coalesced NCHW stores; the next tile's first chunk is in flight ----
        {
            const int n0 = cn0, oh0 = coh0, kb = ckb;
            const int rows_here = min(t.TH, g.OH - oh0);
            const int imgs_here = min(t.NB, g.N - n0);
            const int64_t plane = int64_t(g.OH) * g.OW;
            const int kbase = kb * K_BLK + wn * 32 + lh * 4;
            const bool full_k = (kb + 1) * K_BLK <= g.K;
            // (hand-issued LDS reads: the next tile's first copies are in flight, and a read the compiler sees would
            // wait for them)
            float bv[16];
            {
                const unsigned ba = lds_addr_of(bias_l) + unsigned(kbase) * 4u;
                int raw[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) raw[v] = lds_read32_async(ba + unsigned((v >> 2) * 8 + (v & 3)) * 4u);
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) lds_wait_all(raw[q4 * 4], raw[q4 * 4 + 1], raw[q4 * 4 + 2], raw[q4 * 4 + 3]);
#pragma unroll
                for (int v = 0; v < 16; ++v) bv[v] = __int_as_float(raw[v]);
            }
            if constexpr (POOL) {
                // max over the window, then bias and ReLU: both are monotone, so this equals pool(relu(conv + bias)).
                // The lane's pooled position inside the tile (image, row, column) never changes: it was divided out once,
                // before the tile loop (pool_pos).
                const int prows_here = min(t.TH / 2, g.OH / 2 - oh0 / 2);
                const int64_t pplane = int64_t(g.OH / 2) * t.POW;
#pragma unroll
                for (int j = 0; j < MT / 4; ++j) {
                    const int img = pool_pos[j] >> 20, pr = (pool_pos[j] >> 10) & 1023, pc = pool_pos[j] & 1023;
                    if (img < imgs_here && pr < prows_here) {
                        float *yp = y + (int64_t(n0 + img) * g.K + kbase) * pplane + int64_t(oh0 / 2 + pr) * t.POW + pc;
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int dk = (v >> 2) * 8 + (v & 3);
                            if (full_k || kbase + dk < g.K) {
                                const float o = vmax(vmax3(acc[4 * j][v], acc[4 * j + 1][v], acc[4 * j + 2][v]), acc[4 * j + 3][v]) + bv[v];
                                yp[dk * pplane] = relu ? vmax(o, 0.0f) : o;
                            }
                        }
                    }
                }
            } else
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                // (image, row, column) of the lane's position slot i inside the tile: divided out once (out_pos)
                const int img = int(unsigned(out_pos[i]) >> 24), r = (out_pos[i] >> 12) & 0xfff, c = out_pos[i] & 0xfff;
                if (img < imgs_here && r < rows_here) {
                    float *yp = y + (int64_t(n0 + img) * g.K + kbase) * plane + int64_t(oh0 + r) * g.OW + c;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int dk = (v >> 2) * 8 + (v & 3);
                        const float o = acc[i][v] + bv[v];
                        if (full_k || kbase + dk < g.K) yp[dk * plane] = relu ? vmax(o, 0.0f) : o;  // (a NaN passes where there is no ReLU)
                    }
                }
            }
        }
        cur = nxt;
        cn0 = nn0; coh0 = noh0; ckb = nkb; cp1 = np1;
        set_slots(noff);  // (the table reads wait for the copies in flight; so does the top of the next step)
        tile_par ^= 1;
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

// Few-input-channel convolution (C*KH*KW = CKK small: first layers with 1 or 3 channels).  The
// implicit-GEMM K is then far below one MFMA tile and the layer is bound by writing its output, so
// each thread keeps the CKK input taps of one output position in registers and streams all K output
// channels (weights are wave-uniform: scalar loads); a wave writes 256 contiguous bytes per channel.
template <int CKK>
__global__ void __launch_bounds__(256) conv_f32_smallc_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                             const float *__restrict__ bias, float *__restrict__ y,
                                                             ConvGeom g, int relu) {
    const int64_t plane = int64_t(g.OH) * g.OW;
    const int64_t total = int64_t(g.N) * plane;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    const int taps = g.KH * g.KW;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int n = int(i / plane);
        const int pos = int(i - int64_t(n) * plane);
        const int oh = pos / g.OW, ow = pos - oh * g.OW;
        float xin[CKK];
#pragma unroll
        for (int e = 0; e < CKK; ++e) {
            const int c = e / taps, t = e - c * taps;
            const int kh = t / g.KW, kw = t - kh * g.KW;
            const int ih = oh * g.sh - g.pt + kh * g.dh, iw = ow * g.sw - g.pl + kw * g.dw;
            const bool ok = ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
            xin[e] = ok ? x[((int64_t(n) * g.C + c) * g.H + ih) * g.W + iw] : 0.0f;
        }
        float *yp = y + int64_t(n) * g.K * plane + pos;
        for (int k = 0; k < g.K; ++k) {
            const float *wk = w + int64_t(k) * CKK;
            float acc = 0.0f;
#pragma unroll
            for (int e = 0; e < CKK; ++e) acc = __builtin_fmaf(xin[e], wk[e], acc);
            float r = acc + (bias ? bias[k] : 0.0f);
            if (relu) r = r > 0.0f ? r : 0.0f;
            yp[int64_t(k) * plane] = r;
        }
    }
}

// Few-input-channel convolution fused with ReLU and a 2x2 / stride-2 max pool (stride-1, undilated
// convolution).  One thread owns one POOLED position: it keeps the (KH+1) x (KW+1) input patch of each
// channel in registers, forms the four convolution outputs of the pooling window for every output
// channel, and writes only their (ReLU'd) maximum: the full-resolution activation never reaches HBM.
template <int C, int KH, int KW>
__global__ void __launch_bounds__(256)
conv_f32_smallc_pool_kernel(const float *__restrict__ x, const float *__restrict__ w, const float *__restrict__ bias,
                            float *__restrict__ y, ConvGeom g, int POH, int POW, int relu) {
    constexpr int PH = KH + 1, PW = KW + 1, CKK = C * KH * KW;
    const int64_t pplane = int64_t(POH) * POW;
    const int64_t total = int64_t(g.N) * pplane;
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += step) {
        const int n = int(i / pplane);
        const int pos = int(i - int64_t(n) * pplane);
        const int ph = pos / POW, pw = pos - ph * POW;
        const int ih0 = 2 * ph - g.pt, iw0 = 2 * pw - g.pl;
        float patch[C][PH][PW];
#pragma unroll
        for (int c = 0; c < C; ++c)
#pragma unroll
            for (int r = 0; r < PH; ++r)
#pragma unroll
                for (int q = 0; q < PW; ++q) {
                    const int ih = ih0 + r, iw = iw0 + q;
                    const bool ok = ih >= 0 && ih < g.H && iw >= 0 && iw < g.W;
                    patch[c][r][q] = ok ? x[((int64_t(n) * C + c) * g.H + ih) * g.W + iw] : 0.0f;
                }
        float *yp = y + int64_t(n) * g.K * pplane + pos;
        // The weights of a channel are wave-uniform (scalar loads).  Those of channel k + 1 are requested before the
        // arithmetic of channel k, so the scalar-load latency hides behind 4 * CKK FMAs instead of stalling every channel.
        float wcur[CKK], wnext[CKK];
        const float *bp = bias ? bias : w;  // always loadable: the value is dropped below when there is no bias
        float bcur = bias ? bp[0] : 0.0f, bnext = 0.0f;
#pragma unroll
        for (int e = 0; e < CKK; ++e) wcur[e] = w[e];
        for (int k = 0; k < g.K; ++k) {
            const int kn = k + 1 < g.K ? k + 1 : k;
            const float *wk = w + int64_t(kn) * CKK;
#pragma unroll
            for (int e = 0; e < CKK; ++e) wnext[e] = wk[e];
            const float bl = bp[kn];
            __builtin_amdgcn_sched_barrier(0);  // keep the requests ahead of the arithmetic
            bnext = bias ? bl : 0.0f;
            float a00 = 0.f, a01 = 0.f, a10 = 0.f, a11 = 0.f;
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int kh = 0; kh < KH; ++kh)
#pragma unroll
                    for (int kw = 0; kw < KW; ++kw) {
                        const float wv = wcur[(c * KH + kh) * KW + kw];
                        a00 = __builtin_fmaf(patch[c][kh][kw], wv, a00);
                        a01 = __builtin_fmaf(patch[c][kh][kw + 1], wv, a01);
                        a10 = __builtin_fmaf(patch[c][kh + 1][kw], wv, a10);
                        a11 = __builtin_fmaf(patch[c][kh + 1][kw + 1], wv, a11);
                    }
            // adding the same bias is monotone and so is its rounding: max(a_i + b) == max(a_i) + b exactly
            float r = fmaxf(fmaxf(a00, a01), fmaxf(a10, a11)) + bcur;
            if (relu) r = r > 0.0f ? r : 0.0f;  // max and ReLU commute (both monotone)
            yp[int64_t(k) * pplane] = r;
#pragma unroll
            for (int e = 0; e < CKK; ++e) wcur[e] = wnext[e];
            bcur = bnext;
        }
    }
}

// Single-channel 3x3 first layer + ReLU + MaxPool 2x2/2 on the matrix cores (stride 1, no padding).
//   D[k, p] = sum_t W[k, t] * X[window(p) + tap t]: output channels are the MFMA rows (32 per workgroup), pooled
// positions the columns, and the nine taps the reduction axis, two per v_mfma_f32_32x32x2_f32: (0,0)|(0,1), (1,0)|(1,1),
// (2,0)|(2,1), (0,2)|(1,2), (2,2)|none.  The pairing makes the address of a lane's tap a per-lane base plus an offset
// that is the same for both halves of the wave; the tenth, absent tap reads a word holding 1.0 against the channel's bias
// as its weight, so the matrix cores add the bias too.
// A workgroup copies `imgs` whole images to LDS and walks their pooled positions 32 at a time per wave; the four members
// of a pooling window are four accumulator tiles of the same lane, so the pool is a register-wise max (then ReLU, which
// commutes with it).  20 MFMAs produce 32 positions x 32 channels.  Vector instructions of a SIMD's other waves do not
// hide behind its matrix instructions here (a tile's wall time measured as the sum of both), so everything around the
// MFMAs is kept to a minimum: two instructions per output value and a store without address arithmetic.
template <bool RELU, bool FULLK>
__global__ void __launch_bounds__(256, 4) conv_f32_c1k3_pool_mfma_kernel(const float *__restrict__ x, const float *__restrict__ w,
                                                                     const float *__restrict__ bias, float *__restrict__ y,
                                                                     int N, int H, int W, int K, int POH, int POW, int imgs,
                                                                     FastDiv dpp, FastDiv dpw, int y_c4) {
    extern __shared__ __attribute__((aligned(16))) float img_lds[];  // [imgs][H][W], four words (1, 0, 0, 0), weights, bias
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction; says so to the compiler (LDS
                                                                // copy destinations then stay in scalar registers)
    const int l32 = lane & 31, lh = lane >> 5;
    const int HW = H * W, PP = POH * POW;
    const int n0 = blockIdx.x * imgs, imgs_here = min(imgs, N - n0);
    const int kb = blockIdx.y * 32;
    const int cnt = imgs_here * HW;
    const float *src = x + int64_t(n0) * HW;
    if ((HW & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        for (int i = tid; i < (cnt >> 2); i += 256)
            reinterpret_cast<f32x4 *>(img_lds)[i] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + i);
    } else {
        for (int i = tid; i < cnt; i += 256) img_lds[i] = src[i];
    }
    // [0]: the word the absent tenth tap of the upper half-wave reads -- 1.0, against the channel's bias as its weight, so
    // the last MFMA adds the bias; [1..3]: zero
    const int one_idx = imgs * HW;
    if (tid < 4) img_lds[one_idx + tid] = tid == 0 ? 1.0f : 0.0f;
    // Weights and bias of the workgroup's 32 channels go through LDS: one coalesced read per workgroup, where per-lane
    // reads would be 21 scattered loads per wave, queued in front of the other workgroups' image loads on the CU.
    float *wl = img_lds + one_idx + 4;  // [32][9] weights, then [32] bias
    for (int i = tid; i < 32 * 9 + 32; i += 256) {
        float v = 0.0f;
        if (i < 32 * 9) {
            if (kb + i / 9 < K) v = w[int64_t(kb) * 9 + i];
        } else if (bias != nullptr && kb + i - 32 * 9 < K) {
            v = bias[kb + i - 32 * 9];
        }
        wl[i] = v;
    }
    __syncthreads();

    // this lane's A operands: channel kb + l32, tap pair member lh; the tenth "tap" is the bias
    float wa[5];
    {
        const float *wr = wl + l32 * 9;
        wa[0] = wr[0 + lh];
        wa[1] = wr[3 + lh];
        wa[2] = wr[6 + lh];
        wa[3] = wr[lh ? 5 : 2];
        wa[4] = lh ? wl[32 * 9 + l32] : wr[8];
    }

    const int total = imgs_here * PP;
    // store bases of this lane group's 16 output channels: workgroup-uniform, pinned to scalar registers
    unsigned long long ybase[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const unsigned long long a = reinterpret_cast<unsigned long long>(y + (int64_t(n0) * K + kb + (v >> 2) * 8 + (v & 3)) * PP);
        // (the builtin returns int: without the casts the low word would be sign-extended over the high one)
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(unsigned(a))));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(unsigned(a >> 32))));
        ybase[v] = (static_cast<unsigned long long>(hi) << 32) | static_cast<unsigned long long>(lo);
    }
    // quad-blocked output ([N][K/4][PP][4]): this lane's four groups of four consecutive channels are four 16-byte units,
    // 2 * PP units apart; their bases (group offset included) likewise sit in scalar registers
    unsigned long long ybase4[4];
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
        const unsigned long long a = reinterpret_cast<unsigned long long>(y + (int64_t(n0) * K + kb + gq * 8) * PP);
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(unsigned(a))));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<int>(unsigned(a >> 32))));
        ybase4[gq] = (static_cast<unsigned long long>(hi) << 32) | static_cast<unsigned long long>(lo);
    }
    for (int p0 = wave * 32; p0 < total; p0 += 4 * 32) {
        // Waves with more steps left go first.  Left alone the SIMD serves its oldest waves first: the youngest workgroup on
        // a CU then runs most of its steps after the others are gone, one wave per SIMD, which keeps the matrix pipe half
        // busy; with the laggards in front the four waves of a SIMD finish together.
        {
            const int left = (total - p0 + 127) >> 7;
            if (left >= 5) __builtin_amdgcn_s_setprio(3);
            else if (left >= 3) __builtin_amdgcn_s_setprio(2);
            else if (left == 2) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
        }
        const int p = p0 + l32;
        const bool valid = p < total;
        const unsigned pc_ = valid ? unsigned(p) : 0u;
        const unsigned img = fastdiv(pc_, dpp), pp = pc_ - img * unsigned(PP);
        const unsigned pr = fastdiv(pp, dpw), pcol = pp - pr * unsigned(POW);
        const int wb = int(img) * HW + int(2 * pr) * W + int(2 * pcol);  // window origin in LDS
        const int a012 = wb + lh, a3 = wb + 2 + lh * W;
        f32x16 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[j][v] = 0.0f;
        float b[5][4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int to = (j >> 1) * W + (j & 1);  // window member (dy, dx)
            b[0][j] = img_lds[a012 + to];
            b[1][j] = img_lds[a012 + to + W];
            b[2][j] = img_lds[a012 + to + 2 * W];
            b[3][j] = img_lds[a3 + to];
            b[4][j] = img_lds[lh ? one_idx : wb + to + 2 * W + 2];
        }
        // tap pairs outermost: consecutive MFMAs go to different accumulators
#pragma unroll
        for (int t = 0; t < 5; ++t)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(wa[t], b[t][j], acc[j], 0, 0, 0);
        if (valid) {
            // One 32-bit byte offset per lane and a uniform base per output channel, kept in scalar registers (the host
            // checks that N * K * PP * 4 fits in 32 bits): the stores need no address arithmetic in the vector unit, which
            // this kernel's matrix instructions leave little room for.  The bias came in through the tenth tap; adding the
            // same bias to the four window members is monotone, so the maximum below is pool(conv + bias) exactly.
            const unsigned byte_off = ((unsigned(img) * unsigned(K) + unsigned(lh * 4)) * unsigned(PP) + pp) * 4u;
            // The first three window members first, for all 16 values: the fourth accumulator tile is the one the last
            // MFMA is still writing, and these 16 instructions are the distance its readers must keep from it.
            float m3[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) m3[v] = vmax3(acc[0][v], acc[1][v], acc[2][v]);
            __builtin_amdgcn_sched_barrier(0);
            if (y_c4) {
                // quad (kb + gq*8 + lh*4) / 4 of image n0 + img: unit ((img * K/4 + lh) * PP + pp) past the group's base
                const unsigned off16 = ((unsigned(img) * unsigned(K >> 2) + unsigned(lh)) * unsigned(PP) + pp) * 16u;
#pragma unroll
                for (int gq = 0; gq < 4; ++gq) {
                    if (FULLK || kb + gq * 8 + lh * 4 < K) {  // K is a multiple of 4 here: a quad is whole or absent
                        f32x4 o4;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            o4[e] = RELU ? vmax3(m3[gq * 4 + e], acc[3][gq * 4 + e], 0.0f) : vmax(m3[gq * 4 + e], acc[3][gq * 4 + e]);
                        // (a store of more than 8 bytes reads its data over the next cycles: the two wait states keep the
                        // next vector write to these registers -- which the compiler cannot tell apart through the
                        // statement -- behind it)
                        asm volatile("global_store_dwordx4 %0, %1, %2\n\ts_nop 1" : : "v"(off16), "v"(o4), "s"(ybase4[gq]) : "memory");
                    }
                }
            } else {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int dk = (v >> 2) * 8 + (v & 3);
                if (FULLK || kb + lh * 4 + dk < K) {
                    const float o = RELU ? vmax3(m3[v], acc[3][v], 0.0f) : vmax(m3[v], acc[3][v]);
                    asm volatile("global_store_dword %0, %1, %2" : : "v"(byte_off), "v"(o), "s"(ybase[v]) : "memory");
                }
            }
            }
        }
    }
}

struct MfmaPlan : TilePlan {
    int pack_S = 0;  // > 0: window-packed pooled tiles of this many window slots
};

// Tile shape with the best useful-lane fraction whose LDS footprint allows two workgroups per CU.
// LDS the kernel keeps beyond the planner's count: the bias of every output channel (padded to whole channel blocks)
// (and two more scheduler words)
inline size_t bias_lds_bytes(const ConvGeom &g) { return size_t((g.K + 63) / 64) * 64 * sizeof(float) + 8; }

// Window-packed plan for the pooled kernel (MT = 4: one group of 32 window slots per wave): tiles of S = WM*32 pooling
// windows cut from the batch's flat window sequence.  The patch stages every image a run of S windows can touch.
bool plan_packed(const ConvGeom &g, int WM, int WN, size_t cap, MfmaPlan *out) {
    const int rows = g.OH / 2, cols = g.OW / 2, S = WM * 32, K_BLK = WN * 32, T = g.KH * g.KW;
    if (rows < 1 || cols < 1) return false;
    const int per = rows * cols;
    if (per >= S) return false;  // whole pooled images only
    TileGeom t;
    t.x_c4 = 0;
    t.POW = cols;
    t.NB = (per - 1 + S - 1) / per + 1;
    t.TH = 2 * rows;
    t.n_row_tiles = 1;
    t.PH = (t.TH - 1) * g.sh + (g.KH - 1) * g.dh + 1;
    t.PW = (2 * cols - 1) * g.sw + (g.KW - 1) * g.dw + 1;  // (the column an odd OW ends with is never pooled)
    t.P1 = t.NB * t.PH * t.PW;
    t.P1s = (t.P1 + 3) & ~3;
    if (t.PH >= 4096 || t.PW >= 4096 || t.NB >= 256 || rows >= 1024 || cols >= 1024) return false;  // the packed table fields
    if (int64_t(t.NB) * g.C * g.H * g.W * 4 >= (int64_t(1) << 31)) return false;
    const int64_t windows = int64_t(g.N) * per;
    if (windows + S >= (int64_t(1) << 31)) return false;
    t.n_chunks = (g.C + CC - 1) / CC;
    t.n_kblocks = (g.K + K_BLK - 1) / K_BLK;
    t.n_sblocks = int((windows + S - 1) / S);
    const int64_t n_tiles = int64_t(t.n_sblocks) * t.n_kblocks;
    if (n_tiles >= (int64_t(1) << 30)) return false;
    t.n_tiles = int(n_tiles);
    // two staging buffers, two tile tables, scheduler slots, window table
    const size_t lds = 2 * (size_t(T) * 32 * K_BLK + size_t(32) * t.P1s) + size_t(t.P1s) * 8 + 8 + size_t(t.NB) * per * 8;
    if (lds > cap) return false;
    out->MT = 4; out->WM = WM; out->WN = WN; out->t = t; out->lds_bytes = lds;
    out->eff = double(windows) / (double(t.n_sblocks) * S);
    out->score = out->eff;
    out->pack_S = S;
    return true;
}

bool plan_mfma(const ConvGeom &g, MfmaPlan *best, bool pool = false) {
    const size_t cap = 80 * 1024 - bias_lds_bytes(g);
    if (g.K <= 32) return zant_plan_conv_tiles(g, 4, 1, 8, CC, sizeof(float), cap, best, pool, 0, 32, 0, 2, 4, 256, 4096);
    // 64 output channels per workgroup (2 x 2 waves) stage the input patch once per 64 channels; 32 per workgroup
    // (4 x 1 waves) stage it twice but have twice the position slots, which can fit small feature maps much better
    // (e.g. 5 whole 5x5 pooled images in 128 slots instead of 2 in 64).  Take the narrow shape only for a clear win: at
    // 0.98 against 0.78 useful columns the two measured the same time, and the wide one reads the input once.
    MfmaPlan wide, narrow;
    const bool ok_w = zant_plan_conv_tiles(g, 2, 2, 8, CC, sizeof(float), cap, &wide, pool, 0, 32, 0, 2, 4, 256, 4096);
    const bool ok_n = zant_plan_conv_tiles(g, 4, 1, 8, CC, sizeof(float), cap, &narrow, pool, 0, 32, 0, 2, 4, 256, 4096);
    bool ok = false;
    if (ok_n && (!ok_w || narrow.eff > wide.eff + 0.25)) { *best = narrow; ok = true; }
    else if (ok_w) { *best = wide; ok = true; }
    if (pool) {
        // small pooled images leave window slots empty (25 windows in 32): cut the tiles from the flat window sequence
        MfmaPlan packed;
        if (plan_packed(g, 2, 2, cap, &packed) && (!ok || packed.eff > best->eff + 0.1)) { *best = packed; ok = true; }
    }
    return ok;
}

template <int MT, int WM, int WN, int TT, bool POOL, bool PACK = false>
void launch_mfma_tt(zant_ctx *ctx, const float *x, const float *wp, const float *bias, float *y, const ConvGeom &g,
                    const MfmaPlan &p, int relu, int *counter, int grid, int parity) {
    constexpr int KV = MT >= 8 ? 2 : 4;  // 64-bit operand reads keep 8 accumulator tiles inside 256 VGPRs
    // more than 64 KB of dynamic LDS has to be opted into once per kernel
    if (!zant_raise_lds_limit(ctx, reinterpret_cast<const void *>(&conv_f32_mfma_kernel<MT, WM, WN, KV, TT, POOL, PACK>), 160 * 1024)) return;
    PackGeom pk = {PACK ? p.pack_S : 0, p.t.n_tiles, 0};
    // a last round that fills at most one workgroup per CU is dealt out by workgroup number (both of the first two tiles
    // of a workgroup are static, so the tail starts behind them)
    const int rem = p.t.n_tiles % grid;
    if (rem > 0 && rem <= ctx->num_cus && p.t.n_tiles - rem >= 2 * grid) { pk.tail_start = p.t.n_tiles - rem; pk.tail_n = rem; }
    ZANT_KERNEL_NAME(ctx, "conv_f32_mfma_kernel<%d,%d,%d,%d,%d,%s,%s>", MT, WM, WN, KV, TT, POOL ? "true" : "false", PACK ? "true" : "false");
    hipLaunchKernelGGL((conv_f32_mfma_kernel<MT, WM, WN, KV, TT, POOL, PACK>), dim3(grid), dim3(WM * WN * 64), p.lds_bytes + bias_lds_bytes(g),
                       ctx->stream, x, wp, bias, y, g, p.t, relu, counter, parity, pk);
}

template <int MT, int WM, int WN, bool POOL>
void launch_mfma(zant_ctx *ctx, const float *x, const float *wp, const float *bias, float *y, const ConvGeom &g,
                 const MfmaPlan &p, int relu, int *counter, int grid, int parity) {
    const int T = g.KH * g.KW;
    if (T == 9) launch_mfma_tt<MT, WM, WN, 9, POOL>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity);
    else if (T == 1 && !POOL) launch_mfma_tt<MT, WM, WN, 1, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity);
    else launch_mfma_tt<MT, WM, WN, 0, POOL>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity);
}

template <int WM, int WN>
bool dispatch_mt(zant_ctx *ctx, const float *x, const float *wp, const float *bias, float *y, const ConvGeom &g,
                 const MfmaPlan &p, int relu, int *counter, int grid, bool pool, int parity) {
    if (pool && p.pack_S > 0) {
        if constexpr (WM == 2 && WN == 2) {
            if (p.MT != 4) return false;
            if (g.KH * g.KW == 9) launch_mfma_tt<4, WM, WN, 9, true, true>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity);
            else launch_mfma_tt<4, WM, WN, 0, true, true>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity);
            return true;
        } else {
            return false;
        }
    }
    if (pool) {
        switch (p.MT) {
        case 4: launch_mfma<4, WM, WN, true>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
        case 8: launch_mfma<8, WM, WN, true>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
        default: return false;
        }
    }
    switch (p.MT) {
    case 1: launch_mfma<1, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 2: launch_mfma<2, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 3: launch_mfma<3, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 4: launch_mfma<4, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 5: launch_mfma<5, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 6: launch_mfma<6, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 7: launch_mfma<7, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    case 8: launch_mfma<8, WM, WN, false>(ctx, x, wp, bias, y, g, p, relu, counter, grid, parity); return true;
    default: return false;
    }
}

// Whether the implicit-GEMM kernel takes this convolution (optionally with the fused 2x2/2 max pool), and its plan.
bool mfma_eligible(const ConvGeom &g, bool pool, MfmaPlan *plan) {
    const int64_t macs_per_out = int64_t(g.C) * g.KH * g.KW;
    const bool want = g.C >= 4 && macs_per_out >= 32 && int64_t(g.N) * g.OH * g.OW >= 64 &&
                      int64_t(g.N) * g.C * g.H * g.W < (int64_t(1) << 40);
    return want && plan_mfma(g, plan, pool) && plan->eff >= 0.5;
}

// Packs the weights, resets the tile counter and launches the persistent implicit-GEMM kernel.
int run_conv_mfma(zant_ctx *ctx, const float *x, const float *w, const float *bias, float *y, const ConvGeom &g,
                  const MfmaPlan &plan_in, int relu, bool pool, zant_pack_slot *slot, int x_c4 = 0) {
    if (x_c4 && (g.C & 3)) return ZANT_InvalidInput;
    MfmaPlan plan = plan_in;
    plan.t.x_c4 = x_c4 ? 1 : 0;
    const int T = g.KH * g.KW, K_BLK = plan.WN * 32;
    const size_t wp_floats = size_t(plan.t.n_chunks) * plan.t.n_kblocks * T * CC * K_BLK;
    void *ws = nullptr, *dyn = nullptr;
    bool need_pack = true;
    int parity = 0;
    int rc = zant_pack_region(ctx, slot, 256 + wp_floats * sizeof(float), 0, &ws, &dyn, &need_pack, &parity);  // [tile counters | packed weights]
    if (rc) return rc;
    int *counter = static_cast<int *>(ws);
    float *wp = reinterpret_cast<float *>(static_cast<char *>(ws) + 256);
    // persistent workgroups: two per CU; the first two tiles of each are static, the rest dynamic
    const int grid = int(std::min<int64_t>(plan.t.n_tiles, int64_t(ctx->num_cus) * 2));
    const unsigned pb = unsigned(std::min<int64_t>(ceil_div64(int64_t(wp_floats), 256), 1024));
    if (need_pack) {
        hipLaunchKernelGGL(pack_weights_f32_kernel, dim3(pb), dim3(256), 0, ctx->stream, w, wp, g.K, g.C, T,
                           plan.t.n_chunks, plan.t.n_kblocks, K_BLK, counter, 2 * grid);
        ZANT_LAUNCH_CHECK(ctx);
    }
    KernelTimer kt(ctx);
    const bool ok = plan.WN == 2 ? dispatch_mt<2, 2>(ctx, x, wp, bias, y, g, plan, relu, counter, grid, pool, parity)
                                 : dispatch_mt<4, 1>(ctx, x, wp, bias, y, g, plan, relu, counter, grid, pool, parity);
    if (!ok) return 1;
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
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
    return zant_conv2d_f32_slot(ctx, x, xdim, w, wdim, bias, y, ydim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad,
                                fuse_act, nullptr);
}

// ---- zant_hip_conv2d_f32_static: the same convolution for callers that cannot allocate ---------------------------
//
// The tiled kernel's scratch (two tile counters and the packed weights) lives in a static device array instead of
// the context workspace.  `scratch` below is only the host-side handle of that array: every device holds its own
// copy at its own address, which hipGetSymbolAddress returns and which is what kernels, copies and fills must be
// given.  The array is shared by every call on a device and keeps the previous call's contents; each call re-packs
// the weights and re-arms the counters before its convolution kernel, in stream order, so calls on ONE stream are
// safe back to back, while calls that overlap on one device (two contexts, two streams) race.
static __device__ __align__(256) unsigned char scratch[ZANT_HIP_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];        // device address of `scratch` per device, nullptr until resolved
hipError_t g_scratch_err[kMaxDevices];   // what hipGetSymbolAddress returned on that device
bool g_scratch_tried[kMaxDevices];
}  // namespace

void zant_conv_static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_tried[device]) return;
    g_scratch_tried[device] = true;
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));  // `device` is current (see the caller)
    g_scratch_err[device] = e;
    g_scratch_ptr[device] = e == hipSuccess ? ptr : nullptr;
}

extern "C" int zant_hip_conv2d_f32_static(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w,
                                          const int64_t wdim[4], const float *bias, float *y, const int64_t ydim[4],
                                          const int64_t *stride, int n_stride, const int64_t *pads, int n_pads,
                                          const int64_t *dil, int n_dil, int64_t group, const char *auto_pad,
                                          int fuse_act) {
    if (!ctx) return ZANT_NullPointer;
    if (ctx->device < 0 || ctx->device >= kMaxDevices) return ZANT_InvalidInput;
    void *ptr;
    hipError_t e;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        ptr = g_scratch_ptr[ctx->device];
        e = g_scratch_err[ctx->device];
    }
    if (!ptr) return zant_fail_hip(ctx, e == hipSuccess ? hipErrorNotInitialized : e, "hipGetSymbolAddress(scratch)");
    zant_pack_slot slot;
    slot.dev = ptr;
    slot.bytes = ZANT_HIP_STATIC_SCRATCH_BYTES;
    slot.fixed = true;
    return zant_conv2d_f32_slot(ctx, x, xdim, w, wdim, bias, y, ydim, stride, n_stride, pads, n_pads, dil, n_dil, group,
                                auto_pad, fuse_act, &slot);
}

int zant_conv2d_f32_slot(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                         const float *bias, float *y, const int64_t ydim[4], const int64_t *stride, int n_stride,
                         const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group, const char *auto_pad,
                         int fuse_act, zant_pack_slot *slot, int x_c4) {
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
    if (mfma_eligible(g, false, &plan)) {
        rc = run_conv_mfma(ctx, x, w, bias, y, g, plan, relu, false, slot, x_c4);
        if (rc <= 0) {
            if (rc == ZANT_OK) zant_log("OnnxConvLean4");
            return rc;
        }
    }
    if (x_c4) return ZANT_InvalidInput;  // only the matrix-core kernel reads the quad-blocked layout (see zant_conv2d_f32_c4_caps)
    const int ckk = g.C * g.KH * g.KW;
    if (ckk == 9 || ckk == 25 || ckk == 27) {
        const int64_t positions = int64_t(g.N) * g.OH * g.OW;
        const unsigned pb = unsigned(std::min<int64_t>(ceil_div64(positions, 256), int64_t(ctx->num_cus) * 16));
        KernelTimer kt(ctx);
        ZANT_KERNEL_NAME(ctx, "conv_f32_smallc_kernel<%d>", ckk);
        if (ckk == 9) hipLaunchKernelGGL(conv_f32_smallc_kernel<9>, dim3(pb), dim3(256), 0, ctx->stream, x, w, bias, y, g, relu);
        else if (ckk == 25) hipLaunchKernelGGL(conv_f32_smallc_kernel<25>, dim3(pb), dim3(256), 0, ctx->stream, x, w, bias, y, g, relu);
        else hipLaunchKernelGGL(conv_f32_smallc_kernel<27>, dim3(pb), dim3(256), 0, ctx->stream, x, w, bias, y, g, relu);
        ZANT_LAUNCH_CHECK(ctx);
        zant_log("OnnxConvLean4");
        return ZANT_OK;
    }
    const int64_t total = int64_t(g.N) * g.K * g.OH * g.OW;
    int64_t blocks = ceil_div64(total, 256);
    if (blocks > int64_t(ctx->num_cus) * 32) blocks = int64_t(ctx->num_cus) * 32;
    KernelTimer kt(ctx);
    ZANT_KERNEL_NAME(ctx, "conv_f32_direct_kernel");
    hipLaunchKernelGGL(conv_f32_direct_kernel, dim3(unsigned(blocks)), dim3(256), 0, ctx->stream, x, w, bias, y, g, relu);
    ZANT_LAUNCH_CHECK(ctx);
    zant_log("OnnxConvLean4");
    return ZANT_OK;
}

// Conv (+ReLU) + MaxPool 2x2/2 in one kernel (few-channel first layers: direct kernel; many-channel layers: the
// implicit-GEMM kernel with a register-wise pool in its epilogue); returns 1 when the shape is
// not one this kernel takes (the caller then runs the two operators separately).
int zant_conv2d_f32_fused_pool(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                               const float *bias, float *y, const int64_t ydim[4], const int64_t *stride, int n_stride,
                               const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                               const char *auto_pad, int relu, bool query_only, zant_pack_slot *slot, int x_c4, int y_c4) {
    int64_t s[2], d[2], p[4];
    if (zant_conv_resolve(xdim, wdim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad, s, d, p)) return 1;
    if (s[0] != 1 || s[1] != 1 || d[0] != 1 || d[1] != 1 || xdim[1] != wdim[1]) return 1;
    const int C = int(wdim[1]), KH = int(wdim[2]), KW = int(wdim[3]);
    const bool k133 = C == 1 && KH == 3 && KW == 3, k155 = C == 1 && KH == 5 && KW == 5, k333 = C == 3 && KH == 3 && KW == 3;
    const int64_t OH = xdim[2] + p[0] + p[2] - KH + 1, OW = xdim[3] + p[1] + p[3] - KW + 1;
    if (OH < 2 || OW < 2) return 1;
    if (ydim[0] != xdim[0] || ydim[1] != wdim[0] || ydim[2] != OH / 2 || ydim[3] != OW / 2) return 1;
    for (int i = 0; i < 4; ++i)
        if (xdim[i] <= 0 || wdim[i] <= 0 || xdim[i] > INT32_MAX || wdim[i] > INT32_MAX) return 1;
    ConvGeom g;
    g.N = int(xdim[0]); g.C = C; g.H = int(xdim[2]); g.W = int(xdim[3]);
    g.K = int(wdim[0]); g.CG = C; g.KH = KH; g.KW = KW; g.OH = int(OH); g.OW = int(OW);
    g.sh = g.sw = g.dh = g.dw = 1; g.pt = int(p[0]); g.pl = int(p[1]); g.groups = 1;
    if (!k133 && !k155 && !k333) {
        // many-channel layers: the implicit-GEMM kernel with the pool folded into its epilogue
        MfmaPlan plan;
        if (!mfma_eligible(g, true, &plan) || (plan.MT != 4 && plan.MT != 8)) return 1;
        if (query_only) return ZANT_OK;
        if (y_c4) return ZANT_InvalidInput;  // (zant_conv2d_f32_c4_caps says which kernel writes that layout)
        return run_conv_mfma(ctx, x, w, bias, y, g, plan, relu, true, slot, x_c4);
    }
    if (query_only) return ZANT_OK;
    if (x_c4) return ZANT_InvalidInput;
    const int POH = int(OH / 2), POW = int(OW / 2);
    if (k133 && g.pt == 0 && g.pl == 0 && OH == xdim[2] - 2 && OW == xdim[3] - 2 && int64_t(g.H) * g.W * 4 <= 40 * 1024 &&
        int64_t(POH) * POW < (1 << 20) && int64_t(g.N) * g.K * POH * POW < (int64_t(1) << 30)) {
        // the matrix-core first layer: four whole images per workgroup (fewer if they do not fit in 40 KB of LDS); with
        // its 104 registers four workgroups share a CU, which measured better than eight images and two workgroups
        const int imgs = int(std::min<int64_t>(4, (40 * 1024) / (int64_t(g.H) * g.W * 4)));
        const dim3 grid(unsigned(ceil_div64(g.N, imgs)), unsigned(ceil_div64(g.K, 32)));
        KernelTimer kt(ctx);
        const size_t lds = size_t(imgs) * g.H * g.W * 4 + 16 + (32 * 9 + 32) * 4;
        const FastDiv dpp = make_fastdiv(unsigned(POH * POW)), dpw = make_fastdiv(unsigned(POW));
        const bool fullk = g.K % 32 == 0;
        ZANT_KERNEL_NAME(ctx, "conv_f32_c1k3_pool_mfma_kernel<%s,%s>", relu ? "true" : "false", fullk ? "true" : "false");
#define ZANT_C1K3(R, F)                                                                                                      \
    hipLaunchKernelGGL((conv_f32_c1k3_pool_mfma_kernel<R, F>), grid, dim3(256), lds, ctx->stream, x, w, bias, y, g.N, g.H, g.W, g.K, \
                       POH, POW, imgs, dpp, dpw, (y_c4 && g.K % 4 == 0) ? 1 : 0)
        if (y_c4 && g.K % 4 != 0) return ZANT_InvalidInput;
        if (relu) { if (fullk) ZANT_C1K3(true, true); else ZANT_C1K3(true, false); }
        else { if (fullk) ZANT_C1K3(false, true); else ZANT_C1K3(false, false); }
#undef ZANT_C1K3
        ZANT_LAUNCH_CHECK(ctx);
        return ZANT_OK;
    }
    if (y_c4) return ZANT_InvalidInput;
    const int64_t positions = int64_t(g.N) * POH * POW;
    const unsigned pb = unsigned(std::min<int64_t>(ceil_div64(positions, 256), int64_t(ctx->num_cus) * 16));
    KernelTimer kt(ctx);
    ZANT_KERNEL_NAME(ctx, "conv_f32_smallc_pool_kernel<%s>", k133 ? "1,3,3" : k155 ? "1,5,5" : "3,3,3");
    if (k133) hipLaunchKernelGGL((conv_f32_smallc_pool_kernel<1, 3, 3>), dim3(pb), dim3(256), 0, ctx->stream, x, w, bias, y, g, POH, POW, relu);
    else if (k155) hipLaunchKernelGGL((conv_f32_smallc_pool_kernel<1, 5, 5>), dim3(pb), dim3(256), 0, ctx->stream, x, w, bias, y, g, POH, POW, relu);
    else hipLaunchKernelGGL((conv_f32_smallc_pool_kernel<3, 3, 3>), dim3(pb), dim3(256), 0, ctx->stream, x, w, bias, y, g, POH, POW, relu);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

// Which kernel will run a convolution node decides which of its tensors may be quad-blocked: the implicit-GEMM kernel
// reads that layout (with the fused pool or without), the single-channel 3x3 first-layer kernel with the fused pool
// writes it.  The conditions repeat those of zant_conv2d_f32_slot / zant_conv2d_f32_fused_pool above.
void zant_conv2d_f32_c4_caps(const int64_t xdim[4], const int64_t wdim[4], const int64_t ydim[4], const int64_t *stride,
                             int n_stride, const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                             const char *auto_pad, bool fuse_pool, int *in_ok, int *out_ok) {
    *in_ok = *out_ok = 0;
    int64_t s[2], d[2], p[4];
    if (zant_conv_resolve(xdim, wdim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad, s, d, p)) return;
    for (int i = 0; i < 4; ++i)
        if (xdim[i] <= 0 || wdim[i] <= 0 || xdim[i] > INT32_MAX || wdim[i] > INT32_MAX) return;
    if (xdim[1] != wdim[1]) return;
    const int64_t PH = xdim[2] + p[0] + p[2], PW = xdim[3] + p[1] + p[3];
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1;
    if (PH < dkh || PW < dkw) return;
    const int64_t OH = (PH - dkh) / s[0] + 1, OW = (PW - dkw) / s[1] + 1;
    if (OH > INT32_MAX || OW > INT32_MAX) return;
    ConvGeom g;
    g.N = int(xdim[0]); g.C = int(xdim[1]); g.H = int(xdim[2]); g.W = int(xdim[3]);
    g.K = int(wdim[0]); g.CG = int(wdim[1]); g.KH = int(wdim[2]); g.KW = int(wdim[3]);
    g.OH = int(OH); g.OW = int(OW);
    g.sh = int(s[0]); g.sw = int(s[1]); g.dh = int(d[0]); g.dw = int(d[1]);
    g.pt = int(p[0]); g.pl = int(p[1]); g.groups = 1;
    MfmaPlan plan;
    if (!fuse_pool) {
        *in_ok = (g.C % 4 == 0) && mfma_eligible(g, false, &plan);
        return;
    }
    if (s[0] != 1 || s[1] != 1 || d[0] != 1 || d[1] != 1) return;
    const bool k133 = g.C == 1 && g.KH == 3 && g.KW == 3, k155 = g.C == 1 && g.KH == 5 && g.KW == 5,
               k333 = g.C == 3 && g.KH == 3 && g.KW == 3;
    if (!k133 && !k155 && !k333) {
        *in_ok = (g.C % 4 == 0) && mfma_eligible(g, true, &plan) && (plan.MT == 4 || plan.MT == 8);
        return;
    }
    const int POH = int(OH / 2), POW = int(OW / 2);
    *out_ok = k133 && g.K % 4 == 0 && g.pt == 0 && g.pl == 0 && OH == xdim[2] - 2 && OW == xdim[3] - 2 &&
              int64_t(g.H) * g.W * 4 <= 40 * 1024 && int64_t(POH) * POW < (1 << 20) &&
              int64_t(g.N) * g.K * POH * POW < (int64_t(1) << 30) && ydim[2] == POH && ydim[3] == POW;
}

namespace {
__global__ void __launch_bounds__(256) from_c4_f32_kernel(const f32x4 *__restrict__ x, float *__restrict__ y, int64_t units,
                                                          int64_t HW) {
    const int64_t step = int64_t(gridDim.x) * blockDim.x;
    for (int64_t u = int64_t(blockIdx.x) * blockDim.x + threadIdx.x; u < units; u += step) {
        const int64_t q = u / HW, pos = u - q * HW;  // q = n * C/4 + quad: NCHW plane 4q + e
        const f32x4 v = x[u];
#pragma unroll
        for (int e = 0; e < 4; ++e) y[(q * 4 + e) * HW + pos] = v[e];
    }
}
}  // namespace

int zant_from_c4_f32(zant_ctx *ctx, const float *x, int64_t N, int64_t C, int64_t HW, float *y) {
    if (!ctx || !x || !y) return ZANT_NullPointer;
    if (C % 4 != 0) return ZANT_InvalidInput;
    const int64_t units = N * (C / 4) * HW;
    if (units == 0) return ZANT_OK;
    const unsigned blocks = unsigned(std::min<int64_t>(ceil_div64(units, 256), int64_t(ctx->num_cus) * 16));
    hipLaunchKernelGGL(from_c4_f32_kernel, dim3(blocks), dim3(256), 0, ctx->stream, reinterpret_cast<const f32x4 *>(x), y, units, HW);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
