/*
 * zant_oracle.c -- CPU restatement of Z-Ant's tensor-math hot path.
 *
 * TEST INFRASTRUCTURE ONLY (see zant_oracle.h): the checker, never the product.
 *
 * Pinning status
 *   f32 Conv / MatMul / Gemm / MaxPool / ReLU / LeakyReLU / Softmax / add_bias / Reshape:
 *     pinned by the reference's own known-answer tests (transcribed under
 *     tests/golden/), by a brute-force 7-loop convolution, by numpy/scipy
 *     library routines and by closed forms (tests/test_oracle_*.py).
 *   Sigmoid / ReduceMean / Concat / Resize(nearest): pinned by the reference's
 *     known-answer tests (tests/golden/), numpy (mean, concatenate), scipy's
 *     expit and closed forms (integer upscales repeat elements).
 *   AveragePool (pool_forward, .Avg) / BatchNormalization (inference form of
 *     BatchNormLayer.forward): the reference's tests hold no expected values for
 *     either (test_op_pooling.zig pools with .Max only; test_layers.zig:539-611
 *     checks shapes only): parity unpinned by the reference; pinned by brute
 *     force, torch.nn.functional.avg_pool2d / batch_norm on the CPU and the
 *     closed forms (constant input, identity statistics).
 *   broadcast Add: the reference has no test for the broadcast branch and its
 *     stride computation reads out of bounds for mid-axis broadcasts; restated
 *     to NumPy semantics and pinned by numpy.
 *   QuantizeLinear / DequantizeLinear / QLinearConv / depthwise / qlinear act,
 *     add, maxpool, global-avg-pool: parity unpinned by the reference (it holds
 *     no such code or tests); pinned by exact int64 numpy accumulation, tie /
 *     saturation known answers, scipy.signal.correlate2d and reductions to the
 *     f32 path (tests/test_oracle_int8.py).
 */
#include "zant_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* helpers                                                                   */
/* ------------------------------------------------------------------------- */

static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static int64_t imax(int64_t a, int64_t b) { return a > b ? a : b; }
static size_t nz(int64_t n) { return n > 0 ? (size_t)n : 1; } /* never malloc(0) */

const char *zo_error_name(int code) {
    switch (code) {
    case ZO_OK: return "OK";
    case ZO_InvalidDimensions: return "InvalidDimensions";
    case ZO_InvalidPadding: return "InvalidPadding";
    case ZO_InputTensorsWrongShape: return "InputTensorsWrongShape";
    case ZO_InputTensorDifferentShape: return "InputTensorDifferentShape";
    case ZO_InputTensorDimensionMismatch: return "InputTensorDimensionMismatch";
    case ZO_IncompatibleBroadcastShapes: return "IncompatibleBroadcastShapes";
    case ZO_InputTensorDifferentSize: return "InputTensorDifferentSize";
    case ZO_EmptyTensor: return "EmptyTensor";
    case ZO_ZeroSizeTensor: return "ZeroSizeTensor";
    case ZO_InvalidInput: return "InvalidInput";
    case ZO_InputArrayWrongSize: return "InputArrayWrongSize";
    case ZO_WrongStride: return "WrongStride";
    case ZO_MemError: return "MemError";
    case ZO_InvalidAxes: return "InvalidAxes";
    case ZO_AxisOutOfBounds: return "AxisOutOfBounds";
    case ZO_MismatchedShape: return "MismatchedShape";
    case ZO_MismatchedRank: return "MismatchedRank";
    case ZO_EmptyTensorList: return "EmptyTensorList";
    case ZO_UnsupportedMode: return "UnsupportedMode";
    default: return "Unknown";
    }
}

/* Resolves stride / dilation defaults and the four pad amounts exactly as
 * OnnxConvLean does (op_convolution.zig:67-129). */
static int conv_resolve(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride, int n_stride,
                        const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                        const char *auto_pad, int64_t s[2], int64_t d[2], int64_t p[4]) {
    if (group >= 0 && group != 1) return ZO_InvalidDimensions; /* :60-65 */
    if (n_stride < 1) return ZO_WrongStride; /* stride[0] would index an empty slice */
    s[0] = stride[0];                                  /* :68 */
    s[1] = n_stride > 1 ? stride[1] : stride[0];       /* :69 */
    d[0] = (dil && n_dil > 0) ? dil[0] : 1;            /* :70 */
    d[1] = dil ? (n_dil > 1 ? dil[1] : (n_dil > 0 ? dil[0] : 1)) : 1; /* :71 */
    if (s[0] <= 0 || s[1] <= 0 || d[0] <= 0 || d[1] <= 0) return ZO_WrongStride;
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1; /* :74-75 */
    p[0] = p[1] = p[2] = p[3] = 0; /* h_begin, w_begin, h_end, w_end */
    if (auto_pad) {
        if (!strcmp(auto_pad, "VALID")) {
        } else if (!strcmp(auto_pad, "SAME_UPPER") || !strcmp(auto_pad, "SAME_LOWER")) {
            const int64_t oh = ceil_div(xdim[2], s[0]), ow = ceil_div(xdim[3], s[1]);      /* :92-93 */
            const int64_t th = imax((oh - 1) * s[0] + dkh - xdim[2], 0);                   /* :96 */
            const int64_t tw = imax((ow - 1) * s[1] + dkw - xdim[3], 0);                   /* :97 */
            if (!strcmp(auto_pad, "SAME_UPPER")) {
                p[0] = th / 2; p[2] = th - p[0]; p[1] = tw / 2; p[3] = tw - p[1];           /* :101-104 */
            } else {
                p[2] = th / 2; p[0] = th - p[2]; p[3] = tw / 2; p[1] = tw - p[3];           /* :106-109 */
            }
        } else if (!strcmp(auto_pad, "NOTSET")) {
            if (!pads) return ZO_InvalidPadding;                                            /* :120-125 */
            if (n_pads >= 4) { p[0] = pads[0]; p[1] = pads[1]; p[2] = pads[2]; p[3] = pads[3]; } /* :114-119 */
        }
        /* any other string falls through untouched (:126-128 is unreachable) */
    }
    /* auto_pad == null: pads are ignored altogether */
    return ZO_OK;
}

/* ------------------------------------------------------------------------- */
/* f32 Conv: zero-pad copy -> im2col -> W^T -> mat_mul -> scatter + bias     */
/* ------------------------------------------------------------------------- */

/* lean_im2col, op_convolution.zig:424-514.  Row = (b,oh,ow), col = (c,kh,kw);
 * taps beyond the (padded) input are skipped and stay zero.  The 4-wide
 * vector branch there copies the same elements, so one scalar loop restates both. */
static void im2col_f32(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t kh_, int64_t kw_,
                       int64_t sh, int64_t sw, int64_t dh, int64_t dw, int64_t OH, int64_t OW, float *col) {
    const int64_t ksz = kh_ * kw_, cols = C * ksz;
    for (int64_t row = 0; row < N * OH * OW; ++row) {
        const int64_t b = row / (OH * OW), oh = (row % (OH * OW)) / OW, ow = row % OW;
        for (int64_t c = 0; c < C; ++c) {
            const float *src = x + (b * C + c) * H * W;
            float *dst = col + row * cols + c * ksz;
            for (int64_t kh = 0; kh < kh_; ++kh) {
                const int64_t ih = oh * sh + kh * dh;
                if (ih >= H) continue;
                for (int64_t kw = 0; kw < kw_; ++kw) {
                    const int64_t iw = ow * sw + kw * dw;
                    if (iw >= W) continue;
                    dst[kh * kw_ + kw] = src[ih * W + iw];
                }
            }
        }
    }
}

/* lean_mat_mul, op_mat_mul.zig:92-172.  Each output element is accumulated
 * on its own in k-ascending order with a rounded product then a rounded sum
 * (the @Vector lanes never interact), so the lane width does not change the
 * result; 8 lanes are kept to mirror the loop structure for timing. */
typedef float v8f __attribute__((vector_size(32)));
static void mat_mul_f32(const float *A, const float *B, float *Y, int64_t M, int64_t N, int64_t K) {
    for (int64_t i = 0; i < M; ++i) {
        const float *a = A + i * K;
        float *y = Y + i * N;
        int64_t j = 0;
        for (; j + 8 <= N; j += 8) {
            v8f sum = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int64_t k = 0; k < K; ++k) {
                v8f bv;
                memcpy(&bv, B + k * N + j, sizeof bv);
                const float av = a[k];
                const v8f as = {av, av, av, av, av, av, av, av};
                sum += as * bv;
            }
            memcpy(y + j, &sum, sizeof sum);
        }
        for (; j < N; ++j) {
            float sum = 0;
            for (int64_t k = 0; k < K; ++k) sum += a[k] * B[k * N + j];
            y[j] = sum;
        }
    }
}

int zo_convolve_with_bias_f32(const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                              const float *bias, const int64_t stride[2], const int64_t dil[2], float *y,
                              int64_t ydim_out[4]) {
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3];
    const int64_t F = wdim[0], KH = wdim[2], KW = wdim[3];
    const int64_t dkh = (KH - 1) * dil[0] + 1, dkw = (KW - 1) * dil[1] + 1; /* :240-241 */
    if (H < dkh || W < dkw || H < KH || W < KW) return ZO_InvalidDimensions; /* :250, :394 (usize underflow) */
    const int64_t OH = (H - dkh) / stride[0] + 1, OW = (W - dkw) / stride[1] + 1; /* :247-248 */
    if (OH <= 0 || OW <= 0) return ZO_InvalidDimensions;
    const int64_t rows = N * OH * OW, kel = wdim[1] * KH * KW, cols = C * KH * KW;
    if (cols != kel) return ZO_InputTensorsWrongShape; /* mat_mul's A[-1] != B[-2], op_mat_mul.zig:34 */
    float *col = (float *)calloc(nz(rows * cols), sizeof(float));
    float *km = (float *)malloc(nz(kel * F) * sizeof(float));
    float *res = (float *)malloc(nz(rows * F) * sizeof(float));
    if (!col || !km || !res) { free(col); free(km); free(res); return ZO_MemError; }
    im2col_f32(x, N, C, H, W, KH, KW, stride[0], stride[1], dil[0], dil[1], OH, OW, col); /* :268 */
    for (int64_t f = 0; f < F; ++f)                                                        /* :290-295 */
        for (int64_t i = 0; i < kel; ++i) km[i * F + f] = w[f * kel + i];
    mat_mul_f32(col, km, res, rows, F, cols);                                              /* :299 */
    int64_t idx = 0;                                                                        /* :316-328 */
    for (int64_t b = 0; b < N; ++b)
        for (int64_t h = 0; h < OH; ++h)
            for (int64_t ww = 0; ww < OW; ++ww) {
                for (int64_t f = 0; f < F; ++f) {
                    const float bv = bias ? bias[f] : 0.0f;
                    y[((b * F + f) * OH + h) * OW + ww] = res[idx * F + f] + bv;
                }
                ++idx;
            }
    ydim_out[0] = N; ydim_out[1] = F; ydim_out[2] = OH; ydim_out[3] = OW;
    free(col); free(km); free(res);
    return ZO_OK;
}

int zo_conv_lean_f32(const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                     const float *bias, float *y, const int64_t ydim[4], const int64_t *stride, int n_stride,
                     const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                     const char *auto_pad) {
    int64_t s[2], d[2], p[4];
    int rc = conv_resolve(xdim, wdim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad, s, d, p);
    if (rc) return rc;
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3];
    const int64_t PH = H + p[0] + p[2], PW = W + p[1] + p[3];               /* :134-139 */
    float *padded = (float *)calloc(nz(N * C * PH * PW), sizeof(float));
    if (!padded) return ZO_MemError;
    for (int64_t bc = 0; bc < N * C; ++bc)                                   /* :155-164 */
        for (int64_t h = 0; h < H; ++h)
            memcpy(padded + (bc * PH + h + p[0]) * PW + p[1], x + (bc * H + h) * W, (size_t)W * sizeof(float));
    const int64_t pdim[4] = {N, C, PH, PW};
    const int64_t F = wdim[0];
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1;
    if (PH < dkh || PW < dkw) { free(padded); return ZO_InvalidDimensions; }
    const int64_t OH = (PH - dkh) / s[0] + 1, OW = (PW - dkw) / s[1] + 1;
    float *res = (float *)malloc(nz(N * F * OH * OW) * sizeof(float));
    if (!res) { free(padded); return ZO_MemError; }
    int64_t rdim[4];
    rc = zo_convolve_with_bias_f32(padded, pdim, w, wdim, bias, s, d, res, rdim); /* :187-199 */
    free(padded);
    if (rc) { free(res); return rc; }
    if (rdim[0] != ydim[0] || rdim[1] != ydim[1] || rdim[2] != ydim[2] || rdim[3] != ydim[3]) { /* :212-217 */
        free(res);
        return ZO_InvalidDimensions;
    }
    memcpy(y, res, (size_t)(N * F * OH * OW) * sizeof(float));               /* :218 */
    free(res);
    return ZO_OK;
}

int zo_conv_out_shape(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride, int n_stride,
                      const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                      const char *auto_pad, int64_t ydim[4]) {
    /* OnnxConv, op_convolution.zig:647-732 */
    if (group >= 0 && group != 1) return ZO_InvalidDimensions;
    if (n_stride < 1) return ZO_WrongStride;
    const int64_t sh = stride[0], sw = n_stride > 1 ? stride[1] : stride[0];
    const int64_t dh = (dil && n_dil > 0) ? dil[0] : 1;
    const int64_t dw = dil ? (n_dil > 1 ? dil[1] : (n_dil > 0 ? dil[0] : 1)) : 1;
    const int64_t dkh = (wdim[2] - 1) * dh + 1, dkw = (wdim[3] - 1) * dw + 1;
    const int64_t H = xdim[2], W = xdim[3];
    int64_t oh, ow;
    if (auto_pad) {
        if (!strcmp(auto_pad, "VALID")) {
            oh = (H - dkh) / sh + 1; ow = (W - dkw) / sw + 1;
        } else if (!strcmp(auto_pad, "SAME_UPPER") || !strcmp(auto_pad, "SAME_LOWER")) {
            oh = ceil_div(H, sh); ow = ceil_div(W, sw);
        } else if (!strcmp(auto_pad, "NOTSET")) {
            if (pads) {
                if (n_pads < 4) return ZO_InvalidPadding;                    /* :713-715 */
                oh = (H + pads[0] + pads[2] - dkh) / sh + 1;
                ow = (W + pads[1] + pads[3] - dkw) / sw + 1;
            } else {
                oh = (H - dkh) / sh + 1; ow = (W - dkw) / sw + 1;           /* :717-718 */
            }
        } else {
            return ZO_InvalidPadding;                                        /* :720-722 */
        }
    } else {
        const int64_t th = (pads && n_pads >= 4) ? pads[0] + pads[2] : 0;   /* :725-728 */
        const int64_t tw = (pads && n_pads >= 4) ? pads[1] + pads[3] : 0;
        oh = (H + th - dkh) / sh + 1; ow = (W + tw - dkw) / sw + 1;
    }
    ydim[0] = xdim[0]; ydim[1] = wdim[0]; ydim[2] = oh; ydim[3] = ow;
    return ZO_OK;
}

int zo_conv_direct_f64acc(const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                          const float *bias, float *y, const int64_t ydim[4], const int64_t stride[2],
                          const int64_t pads[4], const int64_t dil[2], int64_t group) {
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3];
    const int64_t K = wdim[0], CG = wdim[1], KH = wdim[2], KW = wdim[3];
    if (group < 1 || C % group || K % group || C / group != CG) return ZO_InvalidDimensions;
    const int64_t OH = ydim[2], OW = ydim[3], KG = K / group;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            const int64_t g = k / KG;
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow) {
                    double acc = 0.0;
                    for (int64_t c = 0; c < CG; ++c)
                        for (int64_t kh = 0; kh < KH; ++kh)
                            for (int64_t kw = 0; kw < KW; ++kw) {
                                const int64_t ih = oh * stride[0] - pads[0] + kh * dil[0];
                                const int64_t iw = ow * stride[1] - pads[1] + kw * dil[1];
                                if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                                acc += (double)x[((n * C + g * CG + c) * H + ih) * W + iw] *
                                       (double)w[((k * CG + c) * KH + kh) * KW + kw];
                            }
                    y[((n * K + k) * OH + oh) * OW + ow] = (float)(acc + (bias ? (double)bias[k] : 0.0));
                }
        }
    return ZO_OK;
}

/* ------------------------------------------------------------------------- */
/* MatMul / Gemm                                                             */
/* ------------------------------------------------------------------------- */

int zo_mat_mul_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank) {
    if (a_rank != b_rank) return ZO_InputTensorDifferentShape;                 /* op_mat_mul.zig:26-29 */
    if (a_rank < 2) return ZO_InputTensorsWrongShape;                          /* :40-43 (checked first here: :34 would index dim -1) */
    if (adim[a_rank - 1] != bdim[b_rank - 2]) return ZO_InputTensorsWrongShape; /* :34-37 */
    const int64_t M = adim[a_rank - 2], N = bdim[b_rank - 1], K = adim[a_rank - 1];
    if (M * N == 0 || K == 0) return ZO_InputTensorsWrongShape;               /* :52-55 */
    return ZO_OK;
}

int zo_mat_mul_lean_f32(const float *a, const int64_t *adim, int a_rank, const float *b, const int64_t *bdim,
                        int b_rank, float *y) {
    /* only the last two dims are used; leading dims are ignored (:93-97) */
    const int64_t M = adim[a_rank - 2], K = adim[a_rank - 1], N = bdim[b_rank - 1];
    mat_mul_f32(a, b, y, M, N, K);
    return ZO_OK;
}

int zo_gemm_check(const int64_t *adim, int a_rank, const int64_t *bdim, int b_rank, const int64_t *cdim,
                  int c_rank, int has_c, int trans_a, int trans_b, int64_t ydim[4]) {
    if (a_rank != 4 || b_rank != 4) return ZO_InputTensorsWrongShape;                     /* op_gemm.zig:22-24 */
    if (adim[0] != bdim[0] || adim[1] != bdim[1]) return ZO_InputTensorDifferentShape;    /* :25-27 */
    const int64_t cond_a = trans_a ? adim[2] : adim[3], rows = trans_a ? adim[3] : adim[2]; /* :30-36 */
    const int64_t cond_b = trans_b ? bdim[3] : bdim[2], cols = trans_b ? bdim[2] : bdim[3]; /* :38-44 */
    if (cond_a != cond_b) return ZO_InputTensorDimensionMismatch;                         /* :46-48 */
    if (has_c) {
        if (c_rank != 4) return ZO_InputTensorsWrongShape;                                /* :52-54 */
        if (cdim[0] != adim[0] || cdim[1] != adim[1]) return ZO_InputTensorDifferentShape; /* :55-57 */
        if ((cdim[2] != rows && cdim[2] != 1) || (cdim[3] != cols && cdim[3] != 1))
            return ZO_IncompatibleBroadcastShapes;                                        /* :58-60 */
    }
    ydim[0] = adim[0]; ydim[1] = adim[1]; ydim[2] = rows; ydim[3] = cols;
    return ZO_OK;
}

/* transposeLastTwo, op_gemm.zig:187-268 (4-D branch). */
static float *transpose_last_two(const float *t, const int64_t d[4]) {
    const int64_t n = d[0] * d[1] * d[2] * d[3];
    float *o = (float *)malloc(nz(n) * sizeof(float));
    if (!o) return NULL;
    for (int64_t bc = 0; bc < d[0] * d[1]; ++bc)
        for (int64_t i = 0; i < d[2]; ++i)
            for (int64_t j = 0; j < d[3]; ++j) o[(bc * d[3] + j) * d[2] + i] = t[(bc * d[2] + i) * d[3] + j];
    return o;
}

int zo_gemm_lean_f32(const float *a, const int64_t adim[4], const float *b, const int64_t bdim[4],
                     const float *c, const int64_t *cdim, int c_rank, float alpha, float beta, int trans_a,
                     int trans_b, float *y, const int64_t ydim[4]) {
    int64_t ad[4] = {adim[0], adim[1], adim[2], adim[3]}, bd[4] = {bdim[0], bdim[1], bdim[2], bdim[3]};
    float *ta = NULL, *tb = NULL;
    if (trans_a) { ta = transpose_last_two(a, adim); if (!ta) return ZO_MemError; ad[2] = adim[3]; ad[3] = adim[2]; a = ta; } /* :111-117 */
    if (trans_b) { tb = transpose_last_two(b, bdim); if (!tb) { free(ta); return ZO_MemError; } bd[2] = bdim[3]; bd[3] = bdim[2]; b = tb; } /* :118-124 */
    mat_mul_f32(a, b, y, ad[2], bd[3], ad[3]);                                              /* :128 */
    const int64_t ysize = ydim[0] * ydim[1] * ydim[2] * ydim[3];
    for (int64_t i = 0; i < ysize; ++i) y[i] *= alpha;                                      /* :130-132 */
    if (c && beta != 0) {                                                                   /* :135-139 */
        int64_t csize = 1;
        for (int i = 0; i < c_rank; ++i) csize *= cdim[i];
        if (csize == ysize) {
            for (int64_t i = 0; i < ysize; ++i) y[i] += c[i] * beta;                        /* :142-146 */
        } else {
            const int64_t rr = ydim[2], rc = ydim[3];                                       /* :151-175 */
            const int64_t c_rows = c_rank >= 2 ? cdim[c_rank - 2] : 1, c_cols = c_rank >= 1 ? cdim[c_rank - 1] : 1;
            const int64_t cd1 = c_rank == 4 ? cdim[1] : 1, cd2 = c_rank >= 2 ? cdim[c_rank - 2] : 1,
                          cd3 = c_rank >= 1 ? cdim[c_rank - 1] : 1;
            for (int64_t bb = 0; bb < ad[0]; ++bb)
                for (int64_t cc = 0; cc < ad[1]; ++cc)
                    for (int64_t i = 0; i < rr; ++i)
                        for (int64_t j = 0; j < rc; ++j) {
                            const int64_t ci = c_rows == 1 ? 0 : i, cj = c_cols == 1 ? 0 : j;
                            const int64_t ri = ((bb * ydim[1] + cc) * ydim[2] + i) * ydim[3] + j;
                            const int64_t cx = ((bb * cd1 + cc) * cd2 + ci) * cd3 + cj;
                            y[ri] += c[cx] * beta;
                        }
        }
    }
    free(ta); free(tb);
    return ZO_OK;
}

/* ------------------------------------------------------------------------- */
/* MaxPool                                                                   */
/* ------------------------------------------------------------------------- */

int zo_maxpool_out_shape(const int64_t xdim[4], const int64_t kernel[2], const int64_t strides[2],
                         const int64_t dil[2], const int64_t pads[4], int auto_pad, int ceil_mode,
                         int64_t ydim[4]) {
    const int64_t H = xdim[2], W = xdim[3];
    const int64_t ekh = (kernel[0] - 1) * dil[0] + 1, ekw = (kernel[1] - 1) * dil[1] + 1; /* op_pooling.zig:509-510 */
    int64_t ph = 0, pw = 0;
    switch (auto_pad) {
    case ZO_PAD_NOTSET: ph = pads[0] + pads[2]; pw = pads[1] + pads[3]; break;           /* :513-520 */
    case ZO_PAD_VALID: break;
    case ZO_PAD_SAME_UPPER:
    case ZO_PAD_SAME_LOWER: {
        const int64_t oh = (H + strides[0] - 1) / strides[0], ow = (W + strides[1] - 1) / strides[1]; /* :531-532 */
        ph = (oh - 1) * strides[0] + ekh - H;                                            /* :534-535 */
        pw = (ow - 1) * strides[1] + ekw - W;
        break;
    }
    default: return ZO_InvalidPadding;
    }
    if (H + ph < ekh || W + pw < ekw) return ZO_InvalidDimensions; /* usize underflow in the reference */
    if (ceil_mode) {                                                                     /* :555-561 */
        ydim[2] = (H + ph - ekh + strides[0] - 1) / strides[0] + 1;
        ydim[3] = (W + pw - ekw + strides[1] - 1) / strides[1] + 1;
    } else {
        ydim[2] = (H + ph - ekh) / strides[0] + 1;
        ydim[3] = (W + pw - ekw) / strides[1] + 1;
    }
    ydim[0] = xdim[0]; ydim[1] = xdim[1];
    return ZO_OK;
}

/* Pads for lean_onnx_maxpool, op_pooling.zig:593-618: SAME_* use the plain
 * (undilated) kernel extent there. */
static void maxpool_pads(const int64_t xdim[4], const int64_t ydim[4], const int64_t kernel[2],
                         const int64_t strides[2], const int64_t *pads, int n_pads, int auto_pad, int64_t *top,
                         int64_t *left) {
    *top = 0; *left = 0;
    if (auto_pad == ZO_PAD_NOTSET) {
        if (pads && n_pads >= 4) { *top = pads[0]; *left = pads[1]; }
    } else if (auto_pad == ZO_PAD_SAME_UPPER || auto_pad == ZO_PAD_SAME_LOWER) {
        const int64_t th = (ydim[2] - 1) * strides[0] + kernel[0] - xdim[2];
        const int64_t tw = (ydim[3] - 1) * strides[1] + kernel[1] - xdim[3];
        if (auto_pad == ZO_PAD_SAME_UPPER) { *top = th / 2; *left = tw / 2; }
        else { *top = th - th / 2; *left = tw - tw / 2; }
    }
}

int zo_maxpool_lean_f32(const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4],
                        const int64_t kernel[2], const int64_t strides[2], const int64_t dil[2],
                        const int64_t *pads, int n_pads, int auto_pad) {
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3], OH = ydim[2], OW = ydim[3];
    int64_t top, left;
    maxpool_pads(xdim, ydim, kernel, strides, pads, n_pads, auto_pad, &top, &left);
    for (int64_t bc = 0; bc < N * C; ++bc) {                                               /* :621-658 */
        const float *src = x + bc * H * W;
        float *dst = y + bc * OH * OW;
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                float m = -INFINITY;
                for (int64_t kh = 0; kh < kernel[0]; ++kh)
                    for (int64_t kw = 0; kw < kernel[1]; ++kw) {
                        const int64_t ih = oh * strides[0] - top + kh * dil[0];
                        const int64_t iw = ow * strides[1] - left + kw * dil[1];
                        if (ih >= 0 && ih < H && iw >= 0 && iw < W) {
                            const float v = src[ih * W + iw];
                            m = fmaxf(m, v); /* Zig @max on floats == fmax (NaN loses) */
                        }
                    }
                dst[oh * OW + ow] = m;
            }
    }
    return ZO_OK;
}

int zo_maxpool_lean_u8(const uint8_t *x, const int64_t xdim[4], uint8_t *y, const int64_t ydim[4],
                       const int64_t kernel[2], const int64_t strides[2], const int64_t dil[2],
                       const int64_t *pads, int n_pads, int auto_pad) {
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3], OH = ydim[2], OW = ydim[3];
    int64_t top, left;
    maxpool_pads(xdim, ydim, kernel, strides, pads, n_pads, auto_pad, &top, &left);
    for (int64_t bc = 0; bc < N * C; ++bc) {
        const uint8_t *src = x + bc * H * W;
        uint8_t *dst = y + bc * OH * OW;
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                uint8_t m = 0;
                for (int64_t kh = 0; kh < kernel[0]; ++kh)
                    for (int64_t kw = 0; kw < kernel[1]; ++kw) {
                        const int64_t ih = oh * strides[0] - top + kh * dil[0];
                        const int64_t iw = ow * strides[1] - left + kw * dil[1];
                        if (ih >= 0 && ih < H && iw >= 0 && iw < W) {
                            const uint8_t v = src[ih * W + iw];
                            if (v > m) m = v;
                        }
                    }
                dst[oh * OW + ow] = m;
            }
    }
    return ZO_OK;
}

/* Average pooling: pool_forward's .Avg branch (op_pooling.zig:223-260, 373-408): for each window the sum of the taps
 * that lie inside the input, in kr, kc order, divided by their count.  The reference takes no padding (output
 * (H - k) / s + 1, so every tap is inside); `pads` [top, left, bottom, right] extends it to ONNX AveragePool:
 * with count_include_pad the divisor is the number of taps inside the PADDED input (ONNX: pad cells count as
 * zeros, cells past the padded input -- ceil_mode -- do not), otherwise the in-bounds count as in the reference. */
int zo_avgpool_f32(const float *x, const int64_t xdim[4], float *y, const int64_t ydim[4], const int64_t kernel[2],
                   const int64_t strides[2], const int64_t pads[4], int count_include_pad) {
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3], OH = ydim[2], OW = ydim[3];
    if (kernel[0] <= 0 || kernel[1] <= 0 || strides[0] <= 0 || strides[1] <= 0) return ZO_InvalidDimensions; /* :233-236 */
    if (ydim[0] != N || ydim[1] != C || OH <= 0 || OW <= 0) return ZO_InvalidDimensions;
    const int64_t top = pads ? pads[0] : 0, left = pads ? pads[1] : 0;
    const int64_t bottom = pads ? pads[2] : 0, right = pads ? pads[3] : 0;
    for (int64_t bc = 0; bc < N * C; ++bc) {
        const float *src = x + bc * H * W;
        float *dst = y + bc * OH * OW;
        for (int64_t oh = 0; oh < OH; ++oh)
            for (int64_t ow = 0; ow < OW; ++ow) {
                float sum = 0.0f;
                int64_t count = 0, padded = 0;
                for (int64_t kr = 0; kr < kernel[0]; ++kr)
                    for (int64_t kc = 0; kc < kernel[1]; ++kc) {
                        const int64_t ih = oh * strides[0] - top + kr, iw = ow * strides[1] - left + kc;
                        if (ih >= 0 && ih < H && iw >= 0 && iw < W) { sum += src[ih * W + iw]; ++count; } /* :381-387 */
                        if (ih >= -top && ih < H + bottom && iw >= -left && iw < W + right) ++padded;
                    }
                const int64_t div = count_include_pad ? padded : count;
                dst[oh * OW + ow] = div > 0 ? sum / (float)div : 0.0f; /* :401 */
            }
    }
    return ZO_OK;
}

/* BatchNormalization, inference form (BatchNormLayer.forward with is_training false, batchNormLayer.zig:130-148):
 * x_normalized = (x - running_mean[f]) / sqrt(running_var[f] + epsilon); y = x_normalized * gamma[f] + beta[f].
 * The reference's layer takes [batch, features]; here the feature axis is axis 1 of a tensor of any rank (ONNX
 * BatchNormalization on NCHW), `inner` = elements per (batch, feature) pair. */
int zo_batchnorm_f32(const float *x, int64_t outer, int64_t features, int64_t inner, const float *gamma,
                     const float *beta, const float *mean, const float *var, float epsilon, float *y) {
    for (int64_t b = 0; b < outer; ++b)
        for (int64_t f = 0; f < features; ++f) {
            const float sd = sqrtf(var[f] + epsilon);
            for (int64_t i = 0; i < inner; ++i) {
                const int64_t idx = (b * features + f) * inner + i;
                const float xn = (x[idx] - mean[f]) / sd;
                y[idx] = xn * gamma[f] + beta[f];
            }
        }
    return ZO_OK;
}

/* ------------------------------------------------------------------------- */
/* Activations, Add, Reshape                                                 */
/* ------------------------------------------------------------------------- */

int zo_relu_lean_f32(const float *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; ++i)
        if (x[i] > 0) y[i] = x[i]; /* no else branch: lib_activation_function_math.zig:25-27 */
    return ZO_OK;
}

int zo_leaky_relu_lean_f32(const float *x, float slope, float *y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = x[i] <= 0 ? slope * x[i] : x[i]; /* :70-76 */
    return ZO_OK;
}

int zo_sigmoid_lean_f32(const float *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = 1.0f / (1.0f + expf(-x[i])); /* :116-120 */
    return ZO_OK;
}

int zo_reduce_mean_f32(const float *x, const int64_t *xdim, int rank, const int64_t *axes, int n_axes, int keepdims,
                       int noop_with_empty_axes, float *y, int64_t *ydim_out, int *y_rank_out) {
    if (rank < 0 || rank > 8) return ZO_InvalidDimensions;
    int64_t size = 1;
    for (int i = 0; i < rank; ++i) size *= xdim[i];
    if (!axes || n_axes == 0) { /* lib_reduction_math.zig:35-46, 111-128 */
        if (noop_with_empty_axes) {
            for (int i = 0; i < rank; ++i) ydim_out[i] = xdim[i];
            *y_rank_out = rank;
            if (y) memcpy(y, x, (size_t)size * sizeof(float));
            return ZO_OK;
        }
        if (keepdims) { for (int i = 0; i < rank; ++i) ydim_out[i] = 1; *y_rank_out = rank; }
        else { ydim_out[0] = 1; *y_rank_out = 1; }
        if (y) {
            float sum = 0.0f;
            for (int64_t i = 0; i < size; ++i) sum += x[i];
            y[0] = sum / (float)size;
        }
        return ZO_OK;
    }
    int reduced[8] = {0};
    int64_t ax[8];
    if (n_axes > 8) return ZO_InvalidAxes;
    for (int i = 0; i < n_axes; ++i) { /* :131-141 */
        const int64_t a = axes[i] < 0 ? axes[i] + rank : axes[i];
        if (a < 0 || a >= rank || reduced[a]) return ZO_InvalidAxes;
        reduced[a] = 1;
        ax[i] = a;
    }
    int out_rank = 0, n_rem = 0, rem[8];
    for (int i = 0; i < rank; ++i) { /* :62-76 */
        if (!reduced[i] || keepdims) ydim_out[out_rank++] = reduced[i] ? 1 : xdim[i];
        if (!reduced[i]) rem[n_rem++] = i;
    }
    *y_rank_out = out_rank;
    if (!y) return ZO_OK;
    int64_t istr[8], count = 1, out_size = 1;
    { int64_t st = 1; for (int i = rank - 1; i >= 0; --i) { istr[i] = st; st *= xdim[i]; } }
    for (int i = 0; i < n_axes; ++i) count *= xdim[ax[i]];
    for (int i = 0; i < n_rem; ++i) out_size *= xdim[rem[i]];
    /* reduced extents innermost first: the last listed axis varies fastest (:236-243) */
    int64_t rsize[8], rstr[8];
    for (int i = 0; i < n_axes; ++i) { rsize[n_axes - 1 - i] = xdim[ax[i]]; rstr[n_axes - 1 - i] = istr[ax[i]]; }
    for (int64_t o = 0; o < out_size; ++o) {
        int64_t r = o, base = 0;
        for (int i = n_rem - 1; i >= 0; --i) { base += (r % xdim[rem[i]]) * istr[rem[i]]; r /= xdim[rem[i]]; }
        float sum = 0.0f;
        for (int64_t k = 0; k < count; ++k) { /* :246-258 */
            int64_t t = k, off = base;
            for (int i = 0; i < n_axes; ++i) { off += (t % rsize[i]) * rstr[i]; t /= rsize[i]; }
            sum += x[off];
        }
        y[o] = sum / (float)count; /* :266 */
    }
    return ZO_OK;
}

int zo_concatenate(const void *const *xs, const int64_t *const *dims, const int *ranks, int n, int64_t axis,
                   size_t elem_size, void *y, int64_t *ydim_out, int *y_rank_out) {
    if (n <= 0) return ZO_EmptyTensorList; /* lib_shape_math.zig:308 */
    int rank = 0;
    for (int t = 0; t < n; ++t) if (ranks[t] > rank) rank = ranks[t]; /* :314-320 */
    if (rank > 8) return ZO_InvalidDimensions;
    if (axis < 0) axis += rank; /* :363-370 */
    if (axis < 0 || axis >= rank) return ZO_AxisOutOfBounds;
    int64_t shp[16][8];
    if (n > 16) return ZO_InvalidDimensions;
    for (int t = 0; t < n; ++t) { /* leading ones, :335-358 */
        const int off = rank - ranks[t];
        for (int d = 0; d < rank; ++d) shp[t][d] = d < off ? 1 : dims[t][d - off];
    }
    int64_t total = 0;
    for (int t = 0; t < n; ++t) { /* :374-380 */
        for (int d = 0; d < rank; ++d)
            if (d != axis && shp[t][d] != shp[0][d]) return ZO_MismatchedShape;
        total += shp[t][axis];
    }
    for (int d = 0; d < rank; ++d) ydim_out[d] = d == axis ? total : shp[0][d];
    *y_rank_out = rank;
    if (!y) return ZO_OK;
    int64_t slices = 1, inner = 1;
    for (int d = 0; d < axis; ++d) slices *= shp[0][d];
    for (int d = (int)axis + 1; d < rank; ++d) inner *= shp[0][d];
    char *dst = (char *)y;
    for (int64_t sl = 0; sl < slices; ++sl) /* :398-424 */
        for (int t = 0; t < n; ++t) {
            const size_t bytes = (size_t)(shp[t][axis] * inner) * elem_size;
            memcpy(dst, (const char *)xs[t] + (size_t)sl * bytes, bytes);
            dst += bytes;
        }
    return ZO_OK;
}

int zo_resize_nearest(const void *x, const int64_t *xdim, int rank, size_t elem_size, const float *scales,
                      const int64_t *sizes, int n_param, int coord_mode, void *y, int64_t *ydim_out) {
    if ((!scales && !sizes) || (scales && sizes)) return ZO_InvalidInput; /* lib_shape_math.zig:23-28 */
    if (n_param != rank || rank < 1 || rank > 8) return ZO_InvalidInput;  /* :35-37, 43-45 */
    for (int i = 0; i < rank; ++i)
        ydim_out[i] = scales ? (int64_t)floorf((float)xdim[i] * scales[i]) : sizes[i]; /* :38-40 */
    if (!y) return ZO_OK;
    int64_t istr[8], total = 1;
    { int64_t st = 1; for (int i = rank - 1; i >= 0; --i) { istr[i] = st; st *= xdim[i]; } }
    for (int i = 0; i < rank; ++i) total *= ydim_out[i];
    for (int64_t o = 0; o < total; ++o) {
        int64_t r = o, in_idx = 0;
        for (int i = rank - 1; i >= 0; --i) {
            const int64_t oi = r % ydim_out[i];
            r /= ydim_out[i];
            const float scale = (float)ydim_out[i] / (float)xdim[i]; /* :130 */
            float pos;
            if (coord_mode == 0) pos = ((float)oi + 0.5f) / scale - 0.5f; /* :133-134 */
            else if (coord_mode == 1) pos = (float)oi * (float)(xdim[i] - 1) / (float)(ydim_out[i] - 1); /* :136 */
            else pos = (float)oi / scale; /* :138 */
            if (!(pos == pos)) pos = 0.0f; /* 0 / 0 of a one-element axis under align_corners */
            int64_t ii = (int64_t)roundf(pos); /* @round: half away from zero (:141) */
            if (ii < 0) ii = 0;
            if (ii > xdim[i] - 1) ii = xdim[i] - 1;
            in_idx += ii * istr[i];
        }
        memcpy((char *)y + (size_t)o * elem_size, (const char *)x + (size_t)in_idx * elem_size, elem_size);
    }
    return ZO_OK;
}

int zo_softmax_lean_f32(const float *x, float *y, int64_t rows, int64_t cols) {
    for (int64_t i = 0; i < rows; ++i) {                                       /* :163-186 */
        float mx = x[i * cols];
        for (int64_t j = 0; j < cols; ++j)
            if (x[i * cols + j] > mx) mx = x[i * cols + j];
        float sum = 0.0f;
        for (int64_t j = 0; j < cols; ++j) {
            const float v = expf(x[i * cols + j] - mx);
            y[i * cols + j] = v;
            sum += v;
        }
        for (int64_t j = 0; j < cols; ++j) y[i * cols + j] /= sum;
    }
    return ZO_OK;
}

int zo_sum_tensors_lean_f32(const float *a, const int64_t *adim, int a_rank, const float *b,
                            const int64_t *bdim, int b_rank, float *y, int64_t *ydim_out, int *y_rank_out) {
    int64_t asz = 1, bsz = 1;
    for (int i = 0; i < a_rank; ++i) asz *= adim[i];
    for (int i = 0; i < b_rank; ++i) bsz *= bdim[i];
    if (asz == bsz) {                                                           /* lib_elementWise_math.zig:72-110 */
        for (int64_t i = 0; i < asz; ++i) y[i] = a[i] + b[i];
        if (y_rank_out) { *y_rank_out = a_rank; for (int i = 0; i < a_rank; ++i) ydim_out[i] = adim[i]; }
        return ZO_OK;
    }
    const int r = a_rank > b_rank ? a_rank : b_rank;                            /* :113-115 */
    if (r > 8) return ZO_InvalidDimensions;
    int64_t s1[8], s2[8], so[8], st1[8], st2[8];
    for (int i = 0; i < r; ++i) s1[i] = s2[i] = 1;
    for (int i = 0; i < a_rank; ++i) s1[r - a_rank + i] = adim[i];              /* :143-150 */
    for (int i = 0; i < b_rank; ++i) s2[r - b_rank + i] = bdim[i];
    int64_t osz = 1;
    for (int i = 0; i < r; ++i) {                                               /* :153-158 */
        if (s1[i] != s2[i] && s1[i] != 1 && s2[i] != 1) return ZO_IncompatibleBroadcastShapes;
        so[i] = s1[i] > s2[i] ? s1[i] : s2[i];
        osz *= so[i];
    }
    int64_t t1 = 1, t2 = 1;
    for (int i = r - 1; i >= 0; --i) { /* each operand's OWN contiguous strides */
        st1[i] = s1[i] > 1 ? t1 : 0; t1 *= s1[i];
        st2[i] = s2[i] > 1 ? t2 : 0; t2 *= s2[i];
    }
    for (int64_t i = 0; i < osz; ++i) {
        int64_t rem = i, i1 = 0, i2 = 0;
        for (int dd = r - 1; dd >= 0; --dd) {
            const int64_t pos = rem % so[dd];
            rem /= so[dd];
            i1 += pos * st1[dd];
            i2 += pos * st2[dd];
        }
        y[i] = a[i1] + b[i2];                                                    /* :208 */
    }
    if (y_rank_out) { *y_rank_out = r; for (int i = 0; i < r; ++i) ydim_out[i] = so[i]; }
    return ZO_OK;
}

int zo_add_bias_f32(float *t, const int64_t *tdim, int t_rank, const float *bias, const int64_t *bdim, int b_rank) {
    int64_t tsz = 1, bsz = 1;
    for (int i = 0; i < t_rank; ++i) tsz *= tdim[i];
    for (int i = 0; i < b_rank; ++i) bsz *= bdim[i];
    if (tsz == 0 || bsz == 0) return ZO_EmptyTensor;                            /* :24-29 */
    if (b_rank != 1) return ZO_InputTensorsWrongShape;                          /* :30-32 */
    const int64_t len = bdim[0];
    if (len != tdim[t_rank - 1]) return ZO_InputTensorDimensionMismatch;        /* :33-36 */
    for (int64_t i = 0; i < tsz; i += len)                                      /* :39-44 */
        for (int64_t j = 0; j < len; ++j) t[i + j] += bias[j];
    return ZO_OK;
}

int zo_reshape_lean(const void *x, const int64_t *xdim, int x_rank, size_t elem_size, const int64_t *new_shape,
                    int new_rank, void *y, int64_t *ydim_out) {
    int64_t in_size = 1;
    for (int i = 0; i < x_rank; ++i) in_size *= xdim[i];
    int neg = -1;
    int64_t known = 1;
    for (int i = 0; i < new_rank; ++i) {                                        /* lib_shape_math.zig:1153-1170 */
        if (new_shape[i] == 0) {
            if (i >= x_rank) return ZO_InvalidInput;
            ydim_out[i] = xdim[i];
            known *= xdim[i];
        } else if (new_shape[i] < 0) {
            if (neg >= 0) return ZO_InvalidInput;
            neg = i;
            ydim_out[i] = 1;
        } else {
            ydim_out[i] = new_shape[i];
            known *= new_shape[i];
        }
    }
    if (neg >= 0) {                                                             /* :1178-1188 */
        if (known == 0) return ZO_InvalidInput;
        if (in_size % known != 0) return ZO_InputArrayWrongSize;
        ydim_out[neg] = in_size / known;
    }
    int64_t total = 1;
    for (int i = 0; i < new_rank; ++i) total *= ydim_out[i];
    if (total != in_size) return ZO_InputArrayWrongSize;                        /* :1197-1199 */
    if (y != x) memcpy(y, x, (size_t)in_size * elem_size);                      /* :1208 */
    return ZO_OK;
}

/* ------------------------------------------------------------------------- */
/* int8 family (ONNX operator definitions)                                   */
/* ------------------------------------------------------------------------- */

/* The one requantisation sequence every int8 op ends with:
 * round-half-to-even (rintf under the default rounding mode), add the zero
 * point as a float (exact: both are small integers), saturate, convert. */
static inline uint8_t sat_u8_rne(float v, uint8_t zp) {
    float r = rintf(v) + (float)zp;
    r = fmaxf(r, 0.0f);  /* NaN -> 0 (maxNum) */
    r = fminf(r, 255.0f);
    return (uint8_t)r;
}

static inline float act_f32(float v, int act, float alpha) {
    switch (act) {
    case ZO_ACT_RELU: return v > 0 ? v : 0.0f;
    case ZO_ACT_LEAKY: return v <= 0 ? alpha * v : v; /* lean_leakyReLU's comparison */
    case ZO_ACT_RELU6: return fminf(fmaxf(v, 0.0f), 6.0f);
    default: return v;
    }
}

static void axis_geometry(const int64_t *dim, int rank, int axis, int64_t n_scale, int64_t *inner, int64_t *alen) {
    *inner = 1; *alen = 1;
    if (n_scale > 1) {
        if (axis < 0) axis += rank;
        *alen = dim[axis];
        for (int i = axis + 1; i < rank; ++i) *inner *= dim[i];
    }
}

int zo_quantize_linear_f32_u8(const float *x, const int64_t *xdim, int rank, const float *y_scale,
                              const uint8_t *y_zp, int64_t n_scale, int axis, uint8_t *y) {
    int64_t n = 1, inner, alen;
    for (int i = 0; i < rank; ++i) n *= xdim[i];
    if (n_scale > 1 && (axis < -rank || axis >= rank)) return ZO_InvalidDimensions;
    axis_geometry(xdim, rank, axis, n_scale, &inner, &alen);
    if (n_scale > 1 && n_scale != alen) return ZO_InputTensorDimensionMismatch;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t c = n_scale > 1 ? (i / inner) % alen : 0;
        y[i] = sat_u8_rne(x[i] / y_scale[c], y_zp ? y_zp[c] : 0);
    }
    return ZO_OK;
}

int zo_dequantize_linear_u8_f32(const uint8_t *x, const int64_t *xdim, int rank, const float *x_scale,
                                const uint8_t *x_zp, int64_t n_scale, int axis, float *y) {
    int64_t n = 1, inner, alen;
    for (int i = 0; i < rank; ++i) n *= xdim[i];
    if (n_scale > 1 && (axis < -rank || axis >= rank)) return ZO_InvalidDimensions;
    axis_geometry(xdim, rank, axis, n_scale, &inner, &alen);
    if (n_scale > 1 && n_scale != alen) return ZO_InputTensorDimensionMismatch;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t c = n_scale > 1 ? (i / inner) % alen : 0;
        y[i] = (float)((int)x[i] - (int)(x_zp ? x_zp[c] : 0)) * x_scale[c];
    }
    return ZO_OK;
}

/* QuantizeLinear to int8: the same sequence saturating to [-128, 127] (ONNX QuantizeLinear, int8 output). */
int zo_quantize_linear_f32_i8(const float *x, const int64_t *xdim, int rank, const float *y_scale,
                              const int8_t *y_zp, int64_t n_scale, int axis, int8_t *y) {
    int64_t n = 1, inner, alen;
    for (int i = 0; i < rank; ++i) n *= xdim[i];
    if (n_scale > 1 && (axis < -rank || axis >= rank)) return ZO_InvalidDimensions;
    axis_geometry(xdim, rank, axis, n_scale, &inner, &alen);
    if (n_scale > 1 && n_scale != alen) return ZO_InputTensorDimensionMismatch;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t c = n_scale > 1 ? (i / inner) % alen : 0;
        float r = rintf(x[i] / y_scale[c]) + (float)(y_zp ? y_zp[c] : 0);
        r = fmaxf(r, -128.0f); /* NaN -> -128 */
        r = fminf(r, 127.0f);
        y[i] = (int8_t)r;
    }
    return ZO_OK;
}

/* DequantizeLinear from int8 and from int32 (the accumulator / bias type): y = (x - zp) * scale. */
int zo_dequantize_linear_i8_f32(const int8_t *x, const int64_t *xdim, int rank, const float *x_scale,
                                const int8_t *x_zp, int64_t n_scale, int axis, float *y) {
    int64_t n = 1, inner, alen;
    for (int i = 0; i < rank; ++i) n *= xdim[i];
    if (n_scale > 1 && (axis < -rank || axis >= rank)) return ZO_InvalidDimensions;
    axis_geometry(xdim, rank, axis, n_scale, &inner, &alen);
    if (n_scale > 1 && n_scale != alen) return ZO_InputTensorDimensionMismatch;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t c = n_scale > 1 ? (i / inner) % alen : 0;
        y[i] = (float)((int)x[i] - (int)(x_zp ? x_zp[c] : 0)) * x_scale[c];
    }
    return ZO_OK;
}

int zo_dequantize_linear_i32_f32(const int32_t *x, const int64_t *xdim, int rank, const float *x_scale,
                                 const int32_t *x_zp, int64_t n_scale, int axis, float *y) {
    int64_t n = 1, inner, alen;
    for (int i = 0; i < rank; ++i) n *= xdim[i];
    if (n_scale > 1 && (axis < -rank || axis >= rank)) return ZO_InvalidDimensions;
    axis_geometry(xdim, rank, axis, n_scale, &inner, &alen);
    if (n_scale > 1 && n_scale != alen) return ZO_InputTensorDimensionMismatch;
    for (int64_t i = 0; i < n; ++i) {
        const int64_t c = n_scale > 1 ? (i / inner) % alen : 0;
        /* the difference in 64 bits (it cannot wrap), converted to f32 once */
        y[i] = (float)((int64_t)x[i] - (int64_t)(x_zp ? x_zp[c] : 0)) * x_scale[c];
    }
    return ZO_OK;
}

int zo_qconv_acc_i32(const uint8_t *x, const int64_t xdim[4], uint8_t x_zp, const int8_t *w,
                     const int64_t wdim[4], const int8_t *w_zp, const int32_t *bias, int32_t *acc,
                     const int64_t ydim[4], const int64_t stride[2], const int64_t pads[4],
                     const int64_t dil[2], int64_t group) {
    const int64_t N = xdim[0], C = xdim[1], H = xdim[2], W = xdim[3];
    const int64_t K = wdim[0], CG = wdim[1], KH = wdim[2], KW = wdim[3];
    if (group < 1 || C % group || K % group || C / group != CG) return ZO_InvalidDimensions;
    const int64_t dkh = (KH - 1) * dil[0] + 1, dkw = (KW - 1) * dil[1] + 1;
    if (H + pads[0] + pads[2] < dkh || W + pads[1] + pads[3] < dkw) return ZO_InvalidDimensions;
    const int64_t OH = (H + pads[0] + pads[2] - dkh) / stride[0] + 1, OW = (W + pads[1] + pads[3] - dkw) / stride[1] + 1;
    if (ydim[0] != N || ydim[1] != K || ydim[2] != OH || ydim[3] != OW) return ZO_InvalidDimensions;
    const int64_t KG = K / group;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            const int64_t g = k / KG;
            const int32_t wz = w_zp ? w_zp[k] : 0;
            for (int64_t oh = 0; oh < OH; ++oh)
                for (int64_t ow = 0; ow < OW; ++ow) {
                    int32_t a = bias ? bias[k] : 0;
                    for (int64_t c = 0; c < CG; ++c)
                        for (int64_t kh = 0; kh < KH; ++kh) {
                            const int64_t ih = oh * stride[0] - pads[0] + kh * dil[0];
                            if (ih < 0 || ih >= H) continue;
                            for (int64_t kw = 0; kw < KW; ++kw) {
                                const int64_t iw = ow * stride[1] - pads[1] + kw * dil[1];
                                if (iw < 0 || iw >= W) continue; /* pad pixel == x_zp -> contributes 0 */
                                a += ((int32_t)x[((n * C + g * CG + c) * H + ih) * W + iw] - (int32_t)x_zp) *
                                     ((int32_t)w[((k * CG + c) * KH + kh) * KW + kw] - wz);
                            }
                        }
                    acc[((n * K + k) * OH + oh) * OW + ow] = a;
                }
        }
    return ZO_OK;
}

int zo_qlinearconv_u8i8(const uint8_t *x, const int64_t xdim[4], float x_scale, uint8_t x_zp,
                        const int8_t *w, const int64_t wdim[4], const float *w_scale, int64_t n_wscale,
                        const int8_t *w_zp, float y_scale, uint8_t y_zp, const int32_t *bias, uint8_t *y,
                        const int64_t ydim[4], const int64_t stride[2], const int64_t pads[4],
                        const int64_t dil[2], int64_t group, int act, float act_alpha, float act_scale,
                        uint8_t act_zp) {
    const int64_t total = ydim[0] * ydim[1] * ydim[2] * ydim[3], K = wdim[0], plane = ydim[2] * ydim[3];
    if (n_wscale != 1 && n_wscale != K) return ZO_InputTensorDimensionMismatch;
    int32_t *acc = (int32_t *)malloc(nz(total) * sizeof(int32_t));
    if (!acc) return ZO_MemError;
    int rc = zo_qconv_acc_i32(x, xdim, x_zp, w, wdim, w_zp, bias, acc, ydim, stride, pads, dil, group);
    if (rc) { free(acc); return rc; }
    for (int64_t i = 0; i < total; ++i) {
        const int64_t k = (i / plane) % K;
        const float m = (x_scale * w_scale[n_wscale == 1 ? 0 : k]) / y_scale;
        uint8_t q = sat_u8_rne((float)acc[i] * m, y_zp);
        if (act != ZO_ACT_NONE) {
            const float v = act_f32((float)((int)q - (int)y_zp) * y_scale, act, act_alpha);
            q = sat_u8_rne(v / act_scale, act_zp);
        }
        y[i] = q;
    }
    free(acc);
    return ZO_OK;
}

int zo_qlinear_act_u8(const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act, float alpha,
                      float y_scale, uint8_t y_zp, uint8_t *y) {
    for (int64_t i = 0; i < n; ++i) {
        const float v = act_f32((float)((int)x[i] - (int)x_zp) * x_scale, act, alpha);
        y[i] = sat_u8_rne(v / y_scale, y_zp);
    }
    return ZO_OK;
}

int zo_qlinear_add_u8(const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b, float b_scale,
                      uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        const float fa = (float)((int)a[i] - (int)a_zp) * a_scale;
        const float fb = (float)((int)b[i] - (int)b_zp) * b_scale;
        y[i] = sat_u8_rne((fa + fb) / y_scale, y_zp);
    }
    return ZO_OK;
}

int zo_qlinear_global_avgpool_u8(const uint8_t *x, const int64_t xdim[4], float x_scale, uint8_t x_zp,
                                 float y_scale, uint8_t y_zp, uint8_t *y) {
    const int64_t NC = xdim[0] * xdim[1], HW = xdim[2] * xdim[3];
    for (int64_t i = 0; i < NC; ++i) {
        int32_t s = 0;
        for (int64_t j = 0; j < HW; ++j) s += (int32_t)x[i * HW + j] - (int32_t)x_zp;
        const float mean = ((float)s * x_scale) / (float)HW;
        y[i] = sat_u8_rne(mean / y_scale, y_zp);
    }
    return ZO_OK;
}
