// f32 MatMul / Gemm (mat_mul_lean, gemm_lean; reference op_mat_mul.zig:92-172, op_gemm.zig:91-185).
//
// One kernel: Y = act(alpha * op(A) * op(B) + beta * bcast(C)) on the f32 matrix cores
// (v_mfma_f32_32x32x2_f32).  The reference materialises transposed copies and makes two extra passes
// over Y for alpha and beta*C; here transposes are folded into the global->LDS staging and alpha,
// beta*C and the optional ReLU are the epilogue.  A workgroup owns a BM x BN tile and walks K in
// chunks of 32 through double-buffered LDS with the next chunk's global loads in flight during the
// MFMAs.  Rows of Y are the MFMA rows, columns the MFMA columns, so each accumulator register holds
// 32 consecutive floats of a Y row (128-byte coalesced stores).
#include "common.h"
#include <type_traits>

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
constexpr int BK = 32;

struct GemmArgs {
    int M, N, K;
    int lda, ldb;            // leading dimensions of the stored matrices
    float alpha, beta;
    int c_mode;              // 0 none, else C[ci*c_ld_r + cj*c_ld_c]
    int c_ld_r, c_ld_c;      // 0 strides for broadcast axes
    int relu;
    int a_vec, b_vec;        // 16-byte vector loads are legal for A / B
};

// Loads 4 consecutive floats p[0..3]; elements at or beyond `valid` read as 0.
__device__ __forceinline__ float4 load4(const float *p, int valid, int vec_ok) {
    if (valid >= 4 && vec_ok) return *reinterpret_cast<const float4 *>(p);
    float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
    if (valid > 0) r.x = p[0];
    if (valid > 1) r.y = p[1];
    if (valid > 2) r.z = p[2];
    if (valid > 3) r.w = p[3];
    return r;
}

// A_KC: A is stored with k contiguous ([M][K], no transA).  B_KC: B stored with k contiguous ([N][K], transB).
template <int TM, int WM, int WN, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(WM *WN * 64)
gemm_f32_mfma_kernel(const float *__restrict__ A, const float *__restrict__ B, const float *__restrict__ C,
                     float *__restrict__ Y, GemmArgs g) {
    constexpr int NT = WM * WN * 64;
    constexpr int BM = WM * TM * 32, BN = WN * 32;
    constexpr int A_LD = A_KC ? BK + 1 : BM + 4;      // As[m][k] (odd stride) or As[k][m]
    constexpr int B_LD = B_KC ? BK + 1 : BN + 4;      // Bs[n][k] or Bs[k][n]
    constexpr int A_SZ = A_KC ? BM * A_LD : BK * A_LD;
    constexpr int B_SZ = B_KC ? BN * B_LD : BK * B_LD;
    constexpr int A_V = BM * BK / 4 / NT;             // float4 per thread per chunk
    constexpr int B_V = (BN * BK / 4 + NT - 1) / NT;
    static_assert(BM * BK / 4 % NT == 0, "A tile must divide over the workgroup");
    __shared__ float As[2][A_SZ];
    __shared__ float Bs[2][B_SZ];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;
    // N tiles vary fastest so that workgroups sharing a row panel of A are dispatched together.
    const int n_tiles = (g.N + BN - 1) / BN;
    // Workgroups are dealt round-robin to the 8 XCDs (each with its own L2): give every XCD a contiguous range of
    // tiles so that the tiles sharing a row panel of A meet in one L2.
    const int per_xcd = (gridDim.x + 7) >> 3;
    int sb = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if ((gridDim.x & 7) != 0) sb = blockIdx.x;
    const int bm = sb / n_tiles, bn = sb - bm * n_tiles;
    const int m0 = bm * BM, n0 = bn * BN;

    float4 ra[A_V], rb[B_V];

    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_V; ++i) {
            const int e = tid + i * NT;
            if (A_KC) {
                const int row = e / (BK / 4), kq = e % (BK / 4);
                const int m = m0 + row, k = k0 + kq * 4;
                ra[i] = (m < g.M) ? load4(A + int64_t(m) * g.lda + k, g.K - k, g.a_vec) : make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                const int kr = e / (BM / 4), mq = e % (BM / 4);
                const int k = k0 + kr, m = m0 + mq * 4;
                ra[i] = (k < g.K) ? load4(A + int64_t(k) * g.lda + m, g.M - m, g.a_vec) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        }
#pragma unroll
        for (int i = 0; i < B_V; ++i) {
            const int e = tid + i * NT;
            rb[i] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (e < BN * BK / 4) {
                if (B_KC) {
                    const int col = e / (BK / 4), kq = e % (BK / 4);
                    const int n = n0 + col, k = k0 + kq * 4;
                    if (n < g.N) rb[i] = load4(B + int64_t(n) * g.ldb + k, g.K - k, g.b_vec);
                } else {
                    const int kr = e / (BN / 4), nq = e % (BN / 4);
                    const int k = k0 + kr, n = n0 + nq * 4;
                    if (k < g.K) rb[i] = load4(B + int64_t(k) * g.ldb + n, g.N - n, g.b_vec);
                }
            }
        }
    };

    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_V; ++i) {
            const int e = tid + i * NT;
            if (A_KC) {
                const int row = e / (BK / 4), kq = e % (BK / 4);
                float *d = &As[buf][row * A_LD + kq * 4];
                d[0] = ra[i].x; d[1] = ra[i].y; d[2] = ra[i].z; d[3] = ra[i].w;
            } else {
                const int kr = e / (BM / 4), mq = e % (BM / 4);
                *reinterpret_cast<float4 *>(&As[buf][kr * A_LD + mq * 4]) = ra[i];
            }
        }
#pragma unroll
        for (int i = 0; i < B_V; ++i) {
            const int e = tid + i * NT;
            if (e < BN * BK / 4) {
                if (B_KC) {
                    const int col = e / (BK / 4), kq = e % (BK / 4);
                    float *d = &Bs[buf][col * B_LD + kq * 4];
                    d[0] = rb[i].x; d[1] = rb[i].y; d[2] = rb[i].z; d[3] = rb[i].w;
                } else {
                    const int kr = e / (BN / 4), nq = e % (BN / 4);
                    *reinterpret_cast<float4 *>(&Bs[buf][kr * B_LD + nq * 4]) = rb[i];
                }
            }
        }
    };

    f32x16 acc[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

    const int n_chunks = (g.K + BK - 1) / BK;
    fetch(0);
    for (int ch = 0; ch < n_chunks; ++ch) {
        const int buf = ch & 1;
        stage(buf);
        __syncthreads();  // chunk ch visible; everyone left chunk ch-1 (the buffer staged next time)
        if (ch + 1 < n_chunks) fetch((ch + 1) * BK);
        const float *as = As[buf];
        const float *bs = Bs[buf];
#pragma unroll
        for (int ks = 0; ks < BK / 2; ++ks) {
            const int k = ks * 2 + lh;
            const float b = B_KC ? bs[(wn * 32 + l32) * B_LD + k] : bs[k * B_LD + wn * 32 + l32];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = (wm * TM + i) * 32 + l32;
                const float a = A_KC ? as[m * A_LD + k] : as[k * A_LD + m];
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
            }
        }
    }

    // ---- epilogue: alpha, beta*C (broadcast), ReLU ----
    const int n = n0 + wn * 32 + l32;
    if (n < g.N) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + (wm * TM + i) * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                if (m < g.M) {
                    float r = acc[i][v] * g.alpha;
                    if (g.c_mode) r = r + C[int64_t(m) * g.c_ld_r + int64_t(n) * g.c_ld_c] * g.beta;
                    if (g.relu) r = r > 0.0f ? r : 0.0f;
                    Y[int64_t(m) * g.N + n] = r;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------------------
// Fast path: asynchronous global->LDS staging (no VGPR round trip), a ring of S stages, 128-bit operand reads.
// ------------------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;
__device__ __attribute__((aligned(16))) const float g_gemm_zero[4] = {0.f, 0.f, 0.f, 0.f};

// How an operand panel [ROWS x 32 k] is staged.  KC*: the matrix is stored with k contiguous ([rows][K]);
// RC4: stored with the row index contiguous ([K][rows]).  In LDS a "unit" is 4 consecutive k of one row (16 bytes):
//   KC layout  unit(row, u) at row*8 + (u ^ swz(row))     (XOR swizzle: a 128-byte global row segment lands in one
//              128-byte LDS row, and lanes that read 32 different rows at the same u still hit 8 different columns)
//   RC layout  unit(row, u) at u*ROWS + row
// RC16 (the B operand only, 64 rows): stored like RC4, copied as it lies -- 16 bytes are four consecutive rows at one
// k, a quarter of RC4's copy instructions and 256 contiguous bytes per k row -- into a [k][row] panel; a lane then
// gathers its four consecutive k with two ds_read2_b32 (row stride 64 dwords) instead of one 128-bit read.
enum { KC16 = 0, KC4 = 1, RC4 = 2, RC16 = 3 };

// The LDS serves 128-bit reads 16 lanes at a time from 64 four-byte banks: 16 consecutive rows (two 128-byte rows
// per 256-byte bank line) must land on 16 different 16-byte columns, so the XOR term steps every second row.
__device__ __forceinline__ constexpr int swz(int row) { return (row >> 1) & 7; }

template <int MODE, int ROWS>
constexpr int stage_instrs() { return (MODE == KC16 || MODE == RC16) ? ROWS / 8 : ROWS / 2; }

// The copies of one operand panel for chunk k0.  Every wave issues the same number of instructions whatever the
// masks are (masked lanes fetch zeros), so the number of copies in flight per wave is known at compile time.
template <int MODE, int ROWS, int NW>
__device__ __forceinline__ void stage_panel(float *dst, const float *__restrict__ src, int ld, int r0, int R, int k0,
                                            int K, int wave, int lane) {
    constexpr int INSTRS = stage_instrs<MODE, ROWS>();
    static_assert(INSTRS % NW == 0, "staging instructions must divide over the waves");
#pragma unroll
    for (int ii = 0; ii < INSTRS / NW; ++ii) {
        const int i = ii * NW + wave;
        const float *sp;
        if (MODE == KC16) {
            const int U = i * 64 + lane, row = U >> 3, slot = U & 7;
            const int k = k0 + ((slot ^ swz(row)) << 2);
            sp = (r0 + row < R && k < K) ? src + int64_t(r0 + row) * ld + k : g_gemm_zero;
            __builtin_amdgcn_global_load_lds((gptr_t)sp, (lptr_t)(dst + i * 256), 16, 0, 0);
        } else if (MODE == KC4) {
            const int F = i * 64 + lane, row = F >> 5, slot = (F >> 2) & 7, j = F & 3;
            const int k = k0 + ((slot ^ swz(row)) << 2) + j;
            sp = (r0 + row < R && k < K) ? src + int64_t(r0 + row) * ld + k : g_gemm_zero;
            __builtin_amdgcn_global_load_lds((gptr_t)sp, (lptr_t)(dst + i * 64), 4, 0, 0);
        } else if (MODE == RC16) {
            const int U = i * 64 + lane, kk = U / (ROWS / 4), row = (U % (ROWS / 4)) << 2;
            const int k = k0 + kk;
            sp = (r0 + row < R && k < K) ? src + int64_t(k) * ld + r0 + row : g_gemm_zero;  // (R is a multiple of 4)
            __builtin_amdgcn_global_load_lds((gptr_t)sp, (lptr_t)(dst + i * 256), 16, 0, 0);
        } else {
            const int F = i * 64 + lane, j = F & 3, row = (F >> 2) % ROWS, u = F / (4 * ROWS);
            const int k = k0 + (u << 2) + j;
            sp = (r0 + row < R && k < K) ? src + int64_t(k) * ld + r0 + row : g_gemm_zero;
            __builtin_amdgcn_global_load_lds((gptr_t)sp, (lptr_t)(dst + i * 64), 4, 0, 0);
        }
    }
}

// Per-lane source pointers of a panel at chunk 0 for the unmasked fast path.  Rows beyond the matrix are clamped to
// its last row: what they produce lands in accumulator rows / columns that are never stored.
template <int MODE, int ROWS, int NW>
__device__ __forceinline__ void stage_ptrs(const float *(&p)[stage_instrs<MODE, ROWS>() / NW], const float *src, int ld,
                                           int r0, int R, int wave, int lane) {
#pragma unroll
    for (int ii = 0; ii < stage_instrs<MODE, ROWS>() / NW; ++ii) {
        const int i = ii * NW + wave;
        if (MODE == KC16) {
            const int U = i * 64 + lane, row = U >> 3, slot = U & 7;
            p[ii] = src + int64_t(min(r0 + row, R - 1)) * ld + ((slot ^ swz(row)) << 2);
        } else if (MODE == KC4) {
            const int F = i * 64 + lane, row = F >> 5, slot = (F >> 2) & 7, j = F & 3;
            p[ii] = src + int64_t(min(r0 + row, R - 1)) * ld + ((slot ^ swz(row)) << 2) + j;
        } else if (MODE == RC16) {
            const int U = i * 64 + lane, kk = U / (ROWS / 4), row = (U % (ROWS / 4)) << 2;
            p[ii] = src + int64_t(kk) * ld + min(r0 + row, R - 4);
        } else {
            const int F = i * 64 + lane, j = F & 3, row = (F >> 2) % ROWS, u = F / (4 * ROWS);
            p[ii] = src + int64_t((u << 2) + j) * ld + min(r0 + row, R - 1);
        }
    }
}

// Fast-path copies of one panel: chunk offset `koff` (floats) is uniform, nothing is masked.
template <int MODE, int ROWS, int NW>
__device__ __forceinline__ void stage_fast(float *dst, const float *const (&p)[stage_instrs<MODE, ROWS>() / NW],
                                           int64_t koff, int wave) {
#pragma unroll
    for (int ii = 0; ii < stage_instrs<MODE, ROWS>() / NW; ++ii) {
        const int i = ii * NW + wave;
        if (MODE == KC16 || MODE == RC16) __builtin_amdgcn_global_load_lds((gptr_t)(p[ii] + koff), (lptr_t)(dst + i * 256), 16, 0, 0);
        else __builtin_amdgcn_global_load_lds((gptr_t)(p[ii] + koff), (lptr_t)(dst + i * 64), 4, 0, 0);
    }
}

// Copy instruction ii of this wave's share of a panel (fast path).
template <int MODE, int NW>
__device__ __forceinline__ void stage_fast_one(float *dst, const float *p, int64_t koff, int wave, int ii) {
    const int i = ii * NW + wave;
    if (MODE == KC16 || MODE == RC16) __builtin_amdgcn_global_load_lds((gptr_t)(p + koff), (lptr_t)(dst + i * 256), 16, 0, 0);
    else __builtin_amdgcn_global_load_lds((gptr_t)(p + koff), (lptr_t)(dst + i * 64), 4, 0, 0);
}

// LDS float offset of unit (row, u) of a panel.
template <int MODE, int ROWS>
__device__ __forceinline__ int unit_off(int row, int u) {
    return MODE == RC16 ? u * 4 * ROWS + row : MODE == RC4 ? (u * ROWS + row) * 4 : (row * 8 + (u ^ swz(row))) * 4;
}

// Operand reads and their waits are written by hand.  The compiler cannot count LDS reads that are still in flight
// when newer ones have been issued (it waits for ALL of them, lgkmcnt(0)), which exposes the full LDS latency once per
// group.  LDS returns data in order, so after "lgkmcnt(n)" with n = number of reads issued later, a read has landed.
__device__ __forceinline__ unsigned lds_addr(const float *p) {
    return unsigned(reinterpret_cast<uintptr_t>((lptr_t)const_cast<float *>(p)));
}
template <int OFF>
__device__ __forceinline__ void lds_read128(f32x4 &v, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
}
template <int OFF0, int OFF1>
__device__ __forceinline__ void lds_read2x32(f32x2 &v, unsigned addr) {
    asm volatile("ds_read2_b32 %0, %1 offset0:%2 offset1:%3" : "=v"(v) : "v"(addr), "n"(OFF0), "n"(OFF1));
}
// A lane's B operand of one group (four consecutive k): one 128-bit register tuple, or for RC16 the two pairs its
// two reads fill (kept apart so that no register copy is needed to put them side by side while they are in flight).
template <int BMODE>
struct BOperand {
    f32x4 v;
    __device__ __forceinline__ float at(int j) const { return v[j]; }
};
template <>
struct BOperand<RC16> {
    f32x2 lo, hi;
    __device__ __forceinline__ float at(int j) const { return j < 2 ? lo[j] : hi[j - 2]; }
};
template <int BMODE>
constexpr int b_reads() { return BMODE == RC16 ? 2 : 1; }  // LDS reads per group for the B operand

// Waits until at most N LDS reads are outstanding.  The operand registers are in/out operands so that nothing
// that consumes them can be scheduled above the wait.
template <int N, int MT, int BMODE>
__device__ __forceinline__ void lds_wait(f32x4 (&a)[MT], BOperand<BMODE> &b) {
    static_assert(MT == 1 || MT == 2 || MT == 4, "unsupported tile count");
    if constexpr (BMODE == RC16) {
        if constexpr (MT == 1) asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a[0]), "+v"(b.lo), "+v"(b.hi) : "n"(N));
        else if constexpr (MT == 2) asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(a[0]), "+v"(a[1]), "+v"(b.lo), "+v"(b.hi) : "n"(N));
        else asm volatile("s_waitcnt lgkmcnt(%6)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b.lo), "+v"(b.hi) : "n"(N));
    } else {
        if constexpr (MT == 1) asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a[0]), "+v"(b.v) : "n"(N));
        else if constexpr (MT == 2) asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(a[0]), "+v"(a[1]), "+v"(b.v) : "n"(N));
        else asm volatile("s_waitcnt lgkmcnt(%5)" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b.v) : "n"(N));
    }
}

// The reads of group gi of the chunk at LDS byte address `stage`: MT units of A and one of B per lane.
//   offa / offb: this lane's byte offsets of its group-0..3 units inside a stage (tile i of A adds i * 32 rows).
template <int MT, int AM, int BMODE, int BM, int BN>
__device__ __forceinline__ void read_group(unsigned stage, int gi, const unsigned (&offa)[BK / 8],
                                           const unsigned (&offb)[BK / 8], f32x4 (&av)[MT], BOperand<BMODE> &bv) {
    constexpr int A_TILE = (AM == RC4 ? 32 * 16 : 32 * 128);  // bytes between rows r and r + 32 of a panel
    const unsigned pa = stage + offa[gi], pb = stage + BM * BK * 4 + offb[gi];
    lds_read128<0>(av[0], pa);
    if constexpr (MT >= 2) lds_read128<A_TILE>(av[1], pa);
    if constexpr (MT >= 4) {
        lds_read128<2 * A_TILE>(av[2], pa);
        lds_read128<3 * A_TILE>(av[3], pa);
    }
    if constexpr (BMODE == RC16) {
        static_assert(BN * 3 < 256, "ds_read2_b32 offsets are 8-bit dword counts");
        lds_read2x32<0, BN>(bv.lo, pb);
        lds_read2x32<2 * BN, 3 * BN>(bv.hi, pb);
    } else {
        lds_read128<0>(bv.v, pb);
    }
}

// One pipeline step: start the copies of chunk `ichunk` into `dma`, multiply the chunk at LDS address `cmp_addr`,
// request the first operands of the chunk at `nxt_addr`.
template <int MT, int WM, int WN, int AM, int BMODE, bool FAST>
__device__ __forceinline__ void gemm_step(float *__restrict__ dma, unsigned cmp_addr, unsigned nxt_addr,
                                          const unsigned (&offa)[BK / 8], const unsigned (&offb)[BK / 8],
                                          f32x4 (&a)[2][MT], BOperand<BMODE> (&b)[2],
                                          const float *__restrict__ A, const float *__restrict__ B, const GemmArgs &g,
                                          const float *const (&pa)[stage_instrs<AM, WM * MT * 32>() / (WM * WN)],
                                          const float *const (&pb)[stage_instrs<BMODE, WN * 32>() / (WM * WN)],
                                          int m0, int n0, int ichunk, f32x16 (&acc)[MT]) {
    constexpr int NW = WM * WN, BM = WM * MT * 32, BN = WN * 32;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int PA = stage_instrs<AM, BM>() / NW, PB = stage_instrs<BMODE, BN>() / NW;
    static_assert(PA + PB <= 4 * MT * (BK / 8), "one copy instruction per MFMA at most");
    // FAST: the whole chunk lies inside K: no masks, addresses are a uniform offset from chunk 0, and the copy
    // instructions are spread between the MFMAs (each is issued while the previous MFMA of the dependent chain
    // executes).  Otherwise (the K tail and the zero chunks behind it) the masked copies are issued up front.  The
    // caller runs the fast steps and the others in two loops of their own: with both in one loop body the operand
    // registers of the two paths were reconciled by eight 64-bit register copies per step, paid in matrix-pipe time.
    const int64_t koffa = AM == RC4 ? int64_t(ichunk) * BK * g.lda : int64_t(ichunk) * BK;
    const int64_t koffb = (BMODE == RC4 || BMODE == RC16) ? int64_t(ichunk) * BK * g.ldb : int64_t(ichunk) * BK;
    if (!FAST) {
        stage_panel<AM, BM, NW>(dma, A, g.lda, m0, g.M, ichunk * BK, g.K, wave, lane);
        stage_panel<BMODE, BN, NW>(dma + BM * BK, B, g.ldb, n0, g.N, ichunk * BK, g.K, wave, lane);
    }
    __builtin_amdgcn_sched_barrier(0);

    static_assert((BK / 8) % 2 == 0, "group 0 of every chunk uses operand registers 0");
    int q = 0;  // MFMAs issued so far in this step (a constant after unrolling)
#pragma unroll
    for (int gi = 0; gi < BK / 8; ++gi) {
        const int cur = gi & 1;
        // The next group's operands are requested before this group's MFMAs start: a whole burst to land.  After the
        // last group that is group 0 of the next chunk, which the barrier of THIS step already proved complete, so the
        // next step starts with its operands in registers (or on their way).
        if (gi + 1 < BK / 8) read_group<MT, AM, BMODE, BM, BN>(cmp_addr, gi + 1, offa, offb, a[cur ^ 1], b[cur ^ 1]);
        else read_group<MT, AM, BMODE, BM, BN>(nxt_addr, 0, offa, offb, a[0], b[0]);
        lds_wait<MT + b_reads<BMODE>(), MT>(a[cur], b[cur]);  // everything but the reads just issued has landed
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i][j], b[cur].at(j), acc[i], 0, 0, 0);
                if (FAST) {
                    if (q < PA) stage_fast_one<AM, NW>(dma, pa[q < PA ? q : 0], koffa, wave, q);
                    else if (q < PA + PB) stage_fast_one<BMODE, NW>(dma + BM * BK, pb[q >= PA && q < PA + PB ? q - PA : 0], koffb, wave, q - PA);
                }
                __builtin_amdgcn_sched_barrier(0);
                ++q;
            }
    }
    // The look-ahead reads were issued a whole burst ago; make sure they have landed before the step ends: a value
    // still in flight across the loop edge would be at the mercy of any register copy the compiler puts there.
    lds_wait<0, MT>(a[0], b[0]);
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14).
constexpr int vmcnt_imm(int n) { return (n & 15) | ((n >> 4) << 14) | 0x0F70; }

template <int MT, int WM, int WN, int AM, int BMODE, int S>
__global__ void __launch_bounds__(WM *WN * 64)
gemm_f32_dma_kernel(const float *__restrict__ A, const float *__restrict__ B, const float *__restrict__ C,
                    float *__restrict__ Y, GemmArgs g) {
    constexpr int NW = WM * WN, BM = WM * MT * 32, BN = WN * 32;
    constexpr int STAGE = (BM + BN) * BK;  // floats
    constexpr int P = (stage_instrs<AM, BM>() + stage_instrs<BMODE, BN>()) / NW;  // copies per wave and chunk
    static_assert(S >= 3 && P * (S - 2) < 64, "vmcnt is a 6-bit counter");
    extern __shared__ __attribute__((aligned(16))) float lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int l32 = lane & 31, lh = lane >> 5;
    const int n_tiles = (g.N + BN - 1) / BN;
    const int per_xcd = (gridDim.x + 7) >> 3;
    int sb = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);  // contiguous tile range per XCD (one L2 each)
    if ((gridDim.x & 7) != 0) sb = blockIdx.x;
    const int bm = sb / n_tiles, bn = sb - bm * n_tiles;
    const int m0 = bm * BM, n0 = bn * BN;
    // A C that is broadcast along the rows (a bias vector) is one value per lane: fetched now, it is there when the
    // epilogue wants it instead of costing a memory round trip after the last MFMA.
    float c_row = 0.0f;
    {
        const int nc = n0 + wn * 32 + l32;
        if (g.c_mode && g.c_ld_r == 0 && nc < g.N) c_row = C[int64_t(nc) * g.c_ld_c];
    }

    f32x16 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

    const float *pa[stage_instrs<AM, BM>() / NW], *pb[stage_instrs<BMODE, BN>() / NW];
    stage_ptrs<AM, BM, NW>(pa, A, g.lda, m0, g.M, wave, lane);
    stage_ptrs<BMODE, BN, NW>(pb, B, g.ldb, n0, g.N, wave, lane);

    const int n_chunks = (g.K + BK - 1) / BK;
    // prologue: chunks 0 .. S-2 in flight (chunks beyond the end copy zeros: the count per wave stays fixed)
#pragma unroll
    for (int c = 0; c < S - 1; ++c) {
        stage_panel<AM, BM, NW>(lds + c * STAGE, A, g.lda, m0, g.M, c * BK, g.K, wave, lane);
        stage_panel<BMODE, BN, NW>(lds + c * STAGE + BM * BK, B, g.ldb, n0, g.N, c * BK, g.K, wave, lane);
    }
    // Chunk 0 must be complete for everyone before its first operands are fetched.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(P * (S - 2)));
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // this lane's operand units: group gi reads k-unit 2*gi + lh of rows (wm*MT + i)*32 + l32 (A) and wn*32 + l32 (B)
    unsigned offa[BK / 8], offb[BK / 8];
#pragma unroll
    for (int gi = 0; gi < BK / 8; ++gi) {
        offa[gi] = unsigned(unit_off<AM, BM>(wm * MT * 32 + l32, gi * 2 + lh)) * 4u;
        offb[gi] = unsigned(unit_off<BMODE, BN>(wn * 32 + l32, gi * 2 + lh)) * 4u;
    }
    const unsigned lds0 = lds_addr(lds);
    f32x4 ra[2][MT];
    BOperand<BMODE> rb[2];
    read_group<MT, AM, BMODE, BM, BN>(lds0, 0, offa, offb, ra[0], rb[0]);
    int cbuf = 0, dbuf = S - 1;
    // After the barrier of a step: chunk c+1 is complete for everyone (each wave waited for its own copies of it), and
    // everyone is done with chunk c-1, whose stage is refilled now.  A bare s_barrier: __syncthreads() carries a
    // fence that drains ALL outstanding copies, which would serialise the ring.  The step multiplies chunk c,
    // whose first operands were fetched at the end of the previous step, and ends by fetching those of chunk c+1.
    const int n_fast = max(0, min(n_chunks, g.K / BK - (S - 1)));  // steps whose refill chunk c + S - 1 lies inside K
    int c = 0;
    for (; c < n_fast; ++c) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(P * (S - 3)));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int nbuf = cbuf + 1 == S ? 0 : cbuf + 1;
        gemm_step<MT, WM, WN, AM, BMODE, true>(lds + dbuf * STAGE, lds0 + cbuf * (STAGE * 4), lds0 + nbuf * (STAGE * 4), offa,
                                               offb, ra, rb, A, B, g, pa, pb, m0, n0, c + S - 1, acc);
        cbuf = nbuf;
        dbuf = dbuf + 1 == S ? 0 : dbuf + 1;
    }
    for (; c < n_chunks; ++c) {
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(P * (S - 3)));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const int nbuf = cbuf + 1 == S ? 0 : cbuf + 1;
        gemm_step<MT, WM, WN, AM, BMODE, false>(lds + dbuf * STAGE, lds0 + cbuf * (STAGE * 4), lds0 + nbuf * (STAGE * 4), offa,
                                                offb, ra, rb, A, B, g, pa, pb, m0, n0, c + S - 1, acc);
        cbuf = nbuf;
        dbuf = dbuf + 1 == S ? 0 : dbuf + 1;
    }
    lds_wait<0, MT>(ra[0], rb[0]);             // the last step's look-ahead reads
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // trailing zero copies must not outlive the workgroup's LDS

    const int n = n0 + wn * 32 + l32;
    if (n < g.N) {
        // all C values first (independent loads in flight together), one per lane when C is broadcast along rows
        float cv[MT][16];
        if (g.c_mode) {
            if (g.c_ld_r == 0) {
                const float c0 = c_row;
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) cv[i][v] = c0;
            } else {
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int m = m0 + (wm * MT + i) * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                        cv[i][v] = C[int64_t(min(m, g.M - 1)) * g.c_ld_r + int64_t(n) * g.c_ld_c];
                    }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + (wm * MT + i) * 32 + (v >> 2) * 8 + lh * 4 + (v & 3);
                if (m < g.M) {
                    float r = acc[i][v] * g.alpha;
                    if (g.c_mode) r = r + cv[i][v] * g.beta;
                    if (g.relu) r = r > 0.0f ? r : 0.0f;
                    Y[int64_t(m) * g.N + n] = r;
                }
            }
        }
    }
}

template <int MT, int WM, int WN, int AM, int BMODE, int S = 5>
void launch_gemm_dma(zant_ctx *ctx, const float *A, const float *B, const float *C, float *Y, const GemmArgs &g) {
    constexpr int BM = WM * MT * 32, BN = WN * 32;
    constexpr size_t lds_bytes = size_t(S) * (BM + BN) * BK * sizeof(float);
    auto kern = &gemm_f32_dma_kernel<MT, WM, WN, AM, BMODE, S>;
    if (!zant_raise_lds_limit(ctx, reinterpret_cast<const void *>(kern), int(lds_bytes))) return;
    const unsigned blocks = unsigned(((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN));
    ZANT_KERNEL_NAME(ctx, "gemm_f32_dma_kernel<%d,%d,%d,%d,%d,%d>", MT, WM, WN, AM, BMODE, S);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(WM * WN * 64), lds_bytes, ctx->stream, A, B, C, Y, g);
}

template <int MT, int WM, int WN>
void dispatch_gemm_dma(zant_ctx *ctx, const float *A, const float *B, const float *C, float *Y, const GemmArgs &g,
                       int am, int bmode) {
#define ZANT_GEMM_CASE(a, b) if (am == a && bmode == b) return launch_gemm_dma<MT, WM, WN, a, b>(ctx, A, B, C, Y, g);
    ZANT_GEMM_CASE(KC16, KC16) ZANT_GEMM_CASE(KC16, KC4) ZANT_GEMM_CASE(KC16, RC4)
    ZANT_GEMM_CASE(KC4, KC16) ZANT_GEMM_CASE(KC4, KC4) ZANT_GEMM_CASE(KC4, RC4)
    ZANT_GEMM_CASE(RC4, KC16) ZANT_GEMM_CASE(RC4, KC4) ZANT_GEMM_CASE(RC4, RC4)
    ZANT_GEMM_CASE(KC16, RC16) ZANT_GEMM_CASE(KC4, RC16) ZANT_GEMM_CASE(RC4, RC16)
#undef ZANT_GEMM_CASE
}

// ------------------------------------------------------------------------------------------------------------
// Skinny Gemm (N <= 16, A row-major): the classifier head.  HBM-bound on A: every wave owns 4 rows, its lanes split
// K, B sits in LDS, and the 4 x 16 partial sums per lane are reduced across the wave by recursive halving (63
// exchanges instead of 64 x 6, 48 of them register swaps), which leaves result (row r, column n) in lane r*16 + n --
// where bias, ReLU or the row softmax (16-lane groups) are applied before one coalesced store.
// ------------------------------------------------------------------------------------------------------------
constexpr int SK_KC = 512;  // k per LDS stage of B

template <int NU>  // column units of 4 that hold data: ceil(N / 4); the others stay zero and cost no arithmetic
__global__ void __launch_bounds__(256)
gemm_f32_skinny_kernel(const float *__restrict__ A, const float *__restrict__ B, const float *__restrict__ C,
                       float *__restrict__ Y, GemmArgs g, int ldb_k, int ldb_n, int softmax) {
    __shared__ f32x4 bs[SK_KC * 4];  // [k][4 units of 4 columns]; unit u of row k at u ^ ((k >> 2) & 3): conflict-free reads
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row0 = (blockIdx.x * 4 + wave) * 4;
    float v[64];
#pragma unroll
    for (int i = 0; i < 64; ++i) v[i] = 0.0f;

    for (int kc = 0; kc < g.K; kc += SK_KC) {
        const int kend = min(SK_KC, g.K - kc);
        // this lane's A values of the whole stage first: 32 independent loads in flight while B is staged
        float a[SK_KC / 64][4];
#pragma unroll
        for (int it = 0; it < SK_KC / 64; ++it)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int k = it * 64 + lane;
                a[it][r] = (k < kend && row0 + r < g.M) ? A[int64_t(row0 + r) * g.lda + kc + k] : 0.0f;
            }
        // B stage: all of a thread's loads are issued before the first LDS store (fixed trip count, unrolled)
        float bv[SK_KC * 16 / 256];
#pragma unroll
        for (int i = 0; i < SK_KC * 16 / 256; ++i) {
            const int idx = i * 256 + tid, k = idx >> 4, n = idx & 15;
            bv[i] = (k < kend && n < g.N) ? B[int64_t(kc + k) * ldb_k + int64_t(n) * ldb_n] : 0.0f;
        }
        if (kc) __syncthreads();
#pragma unroll
        for (int i = 0; i < SK_KC * 16 / 256; ++i) {
            const int idx = i * 256 + tid, k = idx >> 4, n = idx & 15;
            reinterpret_cast<float *>(bs)[(k * 4 + ((n >> 2) ^ ((k >> 2) & 3))) * 4 + (n & 3)] = bv[i];
        }
        __syncthreads();
#pragma unroll
        for (int it = 0; it < SK_KC / 64; ++it) {
            const int kq = it * 64 + lane;
            if (it * 64 < kend) {
#pragma unroll
                for (int u = 0; u < NU; ++u) {
                    const f32x4 b = bs[kq * 4 + (u ^ ((kq >> 2) & 3))];
#pragma unroll
                    for (int r = 0; r < 4; ++r)
#pragma unroll
                        for (int c = 0; c < 4; ++c) v[r * 16 + u * 4 + c] = __builtin_fmaf(a[it][r], b[c], v[r * 16 + u * 4 + c]);
                }
            }
        }
    }
    // recursive halving: after the step with distance s a lane keeps the half of its values selected by (lane & s).
    // Distances 32 and 16 are one half-wave / row swap of the two registers and an add: after the swap the lower lanes
    // (even rows) hold both lanes' parts of value i, the upper lanes (odd rows) those of value i + s.
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v[i]), __float_as_uint(v[i + 32]), false, false);
        v[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(v[i]), __float_as_uint(v[i + 16]), false, false);
        v[i] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
#pragma unroll
    for (int s = 8; s >= 1; s >>= 1) {
        const bool up = (lane & s) != 0;
#pragma unroll
        for (int i = 0; i < s; ++i) {
            const float keep = up ? v[i + s] : v[i];
            const float give = up ? v[i] : v[i + s];
            v[i] = keep + __shfl_xor(give, s, 64);
        }
    }
    const int r = lane >> 4, n = lane & 15, m = row0 + r;
    const bool valid = m < g.M && n < g.N;
    float res = v[0] * g.alpha;
    if (g.c_mode && valid) res = res + C[int64_t(m) * g.c_ld_r + int64_t(n) * g.c_ld_c] * g.beta;
    if (g.relu) res = res > 0.0f ? res : 0.0f;
    if (softmax) {  // lean_softmax on the row: exp(x - max) / sum
        float mx = n < g.N ? res : -INFINITY;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float e = n < g.N ? expf(res - mx) : 0.0f;
        float sum = e;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        res = e / sum;
    }
    if (valid) Y[int64_t(m) * g.N + n] = res;
}

template <int TM, int WM, int WN>
void launch_gemm(zant_ctx *ctx, const float *A, const float *B, const float *C, float *Y, const GemmArgs &g,
                 bool a_kc, bool b_kc) {
    constexpr int BM = WM * TM * 32, BN = WN * 32;
    const unsigned blocks = unsigned(((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN));
    const dim3 grid(blocks), block(WM * WN * 64);
    ZANT_KERNEL_NAME(ctx, "gemm_f32_mfma_kernel<%d,%d,%d,%s,%s>", TM, WM, WN, a_kc ? "true" : "false", b_kc ? "true" : "false");
    if (a_kc && b_kc) hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, true, true>), grid, block, 0, ctx->stream, A, B, C, Y, g);
    else if (a_kc && !b_kc) hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, true, false>), grid, block, 0, ctx->stream, A, B, C, Y, g);
    else if (!a_kc && b_kc) hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, false, true>), grid, block, 0, ctx->stream, A, B, C, Y, g);
    else hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, false, false>), grid, block, 0, ctx->stream, A, B, C, Y, g);
}

// M, N, K of op(A)[M,K] * op(B)[K,N]; lda/ldb are the stored row lengths.
int run_gemm(zant_ctx *ctx, const float *A, const float *B, const float *C, float *Y, int64_t M, int64_t N, int64_t K,
             bool trans_a, bool trans_b, float alpha, float beta, int c_mode, int64_t c_ld_r, int64_t c_ld_c, int relu,
             int softmax = 0) {
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return ZANT_InvalidDimensions;
    GemmArgs g;
    g.M = int(M); g.N = int(N); g.K = int(K);
    g.lda = int(trans_a ? M : K);
    g.ldb = int(trans_b ? K : N);
    g.alpha = alpha; g.beta = beta;
    g.c_mode = c_mode; g.c_ld_r = int(c_ld_r); g.c_ld_c = int(c_ld_c);
    g.relu = relu;
    g.a_vec = (reinterpret_cast<uintptr_t>(A) & 15) == 0 && (g.lda & 3) == 0;
    g.b_vec = (reinterpret_cast<uintptr_t>(B) & 15) == 0 && (g.ldb & 3) == 0;
    const bool a_kc = !trans_a, b_kc = trans_b;
    if (softmax && (trans_a || N > 16)) return ZANT_InvalidInput;
    KernelTimer kt(ctx);
    if (!trans_a && N <= 16) {
        const int nu = int((N + 3) / 4);
        ZANT_KERNEL_NAME(ctx, "gemm_f32_skinny_kernel<%d>", nu);
#define ZANT_SKINNY(NU)                                                                                                     \
    hipLaunchKernelGGL(gemm_f32_skinny_kernel<NU>, dim3(unsigned((M + 15) / 16)), dim3(256), 0, ctx->stream, A, B, C, Y, g, \
                       trans_b ? 1 : g.ldb, trans_b ? g.ldb : 1, softmax)
        if (nu == 1) ZANT_SKINNY(1); else if (nu == 2) ZANT_SKINNY(2); else if (nu == 3) ZANT_SKINNY(3); else ZANT_SKINNY(4);
#undef ZANT_SKINNY
        ZANT_LAUNCH_CHECK(ctx);
        return ZANT_OK;
    }
    const int am = a_kc ? (g.a_vec ? KC16 : KC4) : RC4;
    const int bmode = b_kc ? (g.b_vec ? KC16 : KC4) : (g.b_vec ? RC16 : RC4);  // (b_vec with B stored [K][N]: N is a multiple of 4)
    // 128 x 64 tiles (8 waves, 5 stages) while they give at least every other CU one; below that 64 x 64 tiles (4 waves,
    // two workgroups per CU): twice the tiles at half the work each (2048 x 256 x 4096: 144 -> 86 us), 4 % slower per
    // flop where both fill the GPU.
    const int64_t tiles_128 = ((M + 127) / 128) * ((N + 63) / 64);
    if (N > 32 && 2 * tiles_128 <= ctx->num_cus) dispatch_gemm_dma<1, 2, 2>(ctx, A, B, C, Y, g, am, bmode);
    else if (N > 32) dispatch_gemm_dma<1, 4, 2>(ctx, A, B, C, Y, g, am, bmode);
    else launch_gemm<1, 4, 1>(ctx, A, B, C, Y, g, a_kc, b_kc);              // 128 x 32 tile
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

}  // namespace

extern "C" int zant_hip_matmul_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank) {
    if (!adim || !bdim) return ZANT_NullPointer;
    if (a_rank != b_rank) return ZANT_InputTensorDifferentShape;                  // op_mat_mul.zig:26-29
    if (a_rank < 2) return ZANT_InputTensorsWrongShape;                           // :40-43
    if (adim[a_rank - 1] != bdim[b_rank - 2]) return ZANT_InputTensorsWrongShape;  // :34-37
    const int64_t M = adim[a_rank - 2], N = bdim[b_rank - 1], K = adim[a_rank - 1];
    if (M * N == 0 || K == 0) return ZANT_InputTensorsWrongShape;                 // :52-55
    return ZANT_OK;
}

extern "C" int zant_hip_matmul_f32(zant_ctx *ctx, const float *a, const int64_t *adim, int a_rank, const float *b,
                                   const int64_t *bdim, int b_rank, float *y) {
    if (!ctx || !adim || !bdim) return ZANT_NullPointer;
    if (a_rank < 2 || b_rank < 2) return ZANT_InputTensorsWrongShape;
    // lean_mat_mul reads only the last two dims and the first matrix of each operand (:93-97)
    const int64_t M = adim[a_rank - 2], K = adim[a_rank - 1], N = bdim[b_rank - 1];
    if (M < 0 || N < 0 || K < 0) return ZANT_InvalidDimensions;
    if (M == 0 || N == 0) return ZANT_OK;
    if (!a || !b || !y) return ZANT_NullPointer;
    return run_gemm(ctx, a, b, nullptr, y, M, N, K, false, false, 1.0f, 0.0f, 0, 0, 0, 0);
}

extern "C" int zant_hip_gemm_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank,
                                   const int64_t *cdim, int c_rank, int has_c, int trans_a, int trans_b,
                                   int64_t ydim[4]) {
    if (!adim || !bdim || !ydim || (has_c && !cdim)) return ZANT_NullPointer;
    if (a_rank != 4 || b_rank != 4) return ZANT_InputTensorsWrongShape;                        // op_gemm.zig:22-24
    if (adim[0] != bdim[0] || adim[1] != bdim[1]) return ZANT_InputTensorDifferentShape;       // :25-27
    const int64_t cond_a = trans_a ? adim[2] : adim[3], rows = trans_a ? adim[3] : adim[2];    // :30-36
    const int64_t cond_b = trans_b ? bdim[3] : bdim[2], cols = trans_b ? bdim[2] : bdim[3];    // :38-44
    if (cond_a != cond_b) return ZANT_InputTensorDimensionMismatch;                            // :46-48
    if (has_c) {
        if (c_rank != 4) return ZANT_InputTensorsWrongShape;                                   // :52-54
        if (cdim[0] != adim[0] || cdim[1] != adim[1]) return ZANT_InputTensorDifferentShape;   // :55-57
        if ((cdim[2] != rows && cdim[2] != 1) || (cdim[3] != cols && cdim[3] != 1))
            return ZANT_IncompatibleBroadcastShapes;                                           // :58-60
    }
    ydim[0] = adim[0]; ydim[1] = adim[1]; ydim[2] = rows; ydim[3] = cols;
    return ZANT_OK;
}

extern "C" int zant_hip_gemm_f32(zant_ctx *ctx, const float *a, const int64_t adim[4], const float *b,
                                 const int64_t bdim[4], const float *c, const int64_t *cdim, int c_rank, float alpha,
                                 float beta, int trans_a, int trans_b, float *y, const int64_t ydim[4], int fuse_act) {
    if (!ctx || !adim || !bdim || !ydim) return ZANT_NullPointer;
    if (fuse_act != ZANT_ACT_NONE && fuse_act != ZANT_ACT_RELU && fuse_act != ZANT_ACT_SOFTMAX) return ZANT_InvalidInput;
    const int64_t M = trans_a ? adim[3] : adim[2], K = trans_a ? adim[2] : adim[3];
    const int64_t Kb = trans_b ? bdim[3] : bdim[2], N = trans_b ? bdim[2] : bdim[3];
    if (K != Kb) return ZANT_InputTensorDimensionMismatch;
    if (ydim[2] != M || ydim[3] != N) return ZANT_InvalidDimensions;
    if (M == 0 || N == 0) return ZANT_OK;
    if (!a || !b || !y) return ZANT_NullPointer;
    int c_mode = 0;
    int64_t ld_r = 0, ld_c = 0;
    if (c && beta != 0.0f) {  // op_gemm.zig:135-139
        if (!cdim || c_rank < 1) return ZANT_NullPointer;
        const int64_t c_rows = c_rank >= 2 ? cdim[c_rank - 2] : 1, c_cols = cdim[c_rank - 1];
        if ((c_rows != M && c_rows != 1) || (c_cols != N && c_cols != 1)) return ZANT_IncompatibleBroadcastShapes;
        c_mode = 1;
        ld_r = c_rows == 1 ? 0 : c_cols;  // :165-170
        ld_c = c_cols == 1 ? 0 : 1;
    }
    return run_gemm(ctx, a, b, c, y, M, N, K, trans_a != 0, trans_b != 0, alpha, beta, c_mode, ld_r, ld_c,
                    fuse_act == ZANT_ACT_RELU, fuse_act == ZANT_ACT_SOFTMAX);
}
