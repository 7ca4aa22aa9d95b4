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

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
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
    const int bm = blockIdx.x / n_tiles, bn = blockIdx.x - bm * n_tiles;
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

template <int TM, int WM, int WN>
void launch_gemm(zant_ctx *ctx, const float *A, const float *B, const float *C, float *Y, const GemmArgs &g,
                 bool a_kc, bool b_kc) {
    constexpr int BM = WM * TM * 32, BN = WN * 32;
    const unsigned blocks = unsigned(((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN));
    const dim3 grid(blocks), block(WM * WN * 64);
    if (a_kc && b_kc) hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, true, true>), grid, block, 0, ctx->stream, A, B, C, Y, g);
    else if (a_kc && !b_kc) hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, true, false>), grid, block, 0, ctx->stream, A, B, C, Y, g);
    else if (!a_kc && b_kc) hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, false, true>), grid, block, 0, ctx->stream, A, B, C, Y, g);
    else hipLaunchKernelGGL((gemm_f32_mfma_kernel<TM, WM, WN, false, false>), grid, block, 0, ctx->stream, A, B, C, Y, g);
}

// M, N, K of op(A)[M,K] * op(B)[K,N]; lda/ldb are the stored row lengths.
int run_gemm(zant_ctx *ctx, const float *A, const float *B, const float *C, float *Y, int64_t M, int64_t N, int64_t K,
             bool trans_a, bool trans_b, float alpha, float beta, int c_mode, int64_t c_ld_r, int64_t c_ld_c, int relu) {
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
    KernelTimer kt(ctx);
    if (N > 32) launch_gemm<2, 2, 2>(ctx, A, B, C, Y, g, a_kc, b_kc);   // 128 x 64 tile
    else launch_gemm<1, 4, 1>(ctx, A, B, C, Y, g, a_kc, b_kc);          // 128 x 32 tile
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
    if (fuse_act != ZANT_ACT_NONE && fuse_act != ZANT_ACT_RELU) return ZANT_InvalidInput;
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
                    fuse_act == ZANT_ACT_RELU);
}
