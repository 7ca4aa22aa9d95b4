// QLinearConv: u8 activations x i8 weights -> i32 accumulators -> u8 (ONNX definition; the reference has
// no quantised or grouped convolution).  Accumulation is exact integer arithmetic; the epilogue is the
// single f32 requantisation sequence shared with the CPU checker, optionally followed by the fused
// Dequantize -> activation -> Quantize step.
#include "quant_common.h"

namespace {

struct QConvArgs {
    float x_scale, y_scale;
    int x_zp;
    uint8_t y_zp;
    int n_wscale;       // 1 or K
    int has_act;
    QAct act;
};

// Requantises one accumulator of output channel k.
__device__ __forceinline__ uint8_t requant(int acc, float m, const QConvArgs &q) {
    uint8_t r = sat_u8_rne(float(acc) * m, q.y_zp);
    if (q.has_act) r = qact_apply(r, q.act);
    return r;
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

}  // namespace

extern "C" int zant_hip_qlinearconv_u8i8(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale,
                                         uint8_t x_zp, const int8_t *w, const int64_t wdim[4], const float *w_scale,
                                         int64_t n_wscale, const int8_t *w_zp, float y_scale, uint8_t y_zp,
                                         const int32_t *bias, uint8_t *y, const int64_t ydim[4], const int64_t stride[2],
                                         const int64_t pads[4], const int64_t dil[2], int64_t group, int act,
                                         float act_alpha, float act_scale, uint8_t act_zp) {
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
    if (ydim[0] != xdim[0] || ydim[1] != K || ydim[2] != OH || ydim[3] != OW) return ZANT_InvalidDimensions;
    // the i32 accumulator must not overflow: |x - zp| <= 255, |w - wzp| <= 255
    if (wdim[1] * wdim[2] * wdim[3] > (int64_t(1) << 31) / (255 * 255) - 1) return ZANT_InvalidDimensions;
    if (!x || !w || !w_scale || !y) return ZANT_NullPointer;

    ConvGeom g;
    g.N = int(xdim[0]); g.C = int(C); g.H = int(xdim[2]); g.W = int(xdim[3]);
    g.K = int(K); g.CG = int(wdim[1]); g.KH = int(wdim[2]); g.KW = int(wdim[3]);
    g.OH = int(OH); g.OW = int(OW);
    g.sh = int(stride[0]); g.sw = int(stride[1]); g.dh = int(dil[0]); g.dw = int(dil[1]);
    g.pt = int(pads[0]); g.pl = int(pads[1]); g.groups = int(group);
    QConvArgs q;
    q.x_scale = x_scale; q.y_scale = y_scale; q.x_zp = x_zp; q.y_zp = y_zp; q.n_wscale = int(n_wscale);
    q.has_act = act != ZANT_ACT_NONE;
    q.act.act = act; q.act.alpha = act_alpha; q.act.in_scale = y_scale; q.act.in_zp = y_zp;
    q.act.out_scale = act_scale; q.act.out_zp = act_zp;

    const int64_t total = int64_t(g.N) * g.K * g.OH * g.OW;
    int64_t blocks = ceil_div64(total, 256);
    if (blocks > int64_t(ctx->num_cus) * 32) blocks = int64_t(ctx->num_cus) * 32;
    KernelTimer kt(ctx);
    hipLaunchKernelGGL(qconv_direct_kernel, dim3(unsigned(blocks)), dim3(256), 0, ctx->stream, x, w, w_scale, w_zp, bias, y,
                       g, q);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}
