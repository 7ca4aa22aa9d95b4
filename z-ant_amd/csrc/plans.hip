// Prepared-weights handles for callers that issue one lean operator per node with the SAME weights call after call.
//
// The reference's lean operators receive the weights on every call (op_convolution.zig:42), so the plain entry points
// must assume they changed and re-derive everything weight-dependent (packed weights, requantisation tables) each
// time.  A plan fixes shapes, attributes and weights once; the first run packs into memory the plan owns, every later
// run launches the main kernel only.  The int8 plan also lets the caller keep activations in the channel-blocked
// layout between calls, which removes the layout conversion in front of the matrix-core kernels.
#include <new>

#include "common.h"
#include "quant_layout.h"

struct zant_qconv_plan {
    int64_t xdim[4], wdim[4], ydim[4], stride[2], pads[4], dil[2], group, n_wscale;
    float x_scale, y_scale, act_alpha, act_scale;
    uint8_t x_zp, y_zp, act_zp;
    int act, x_layout, y_layout;
    const int8_t *w, *w_zp;
    const float *w_scale;
    const int32_t *bias;
    zant_pack_slot slot;
};

struct zant_conv_plan {
    int64_t xdim[4], wdim[4], ydim[4], stride[2], pads[4], dil[2], group;
    int n_stride, n_pads, n_dil, has_group, fuse_act, fuse_pool;
    char auto_pad[16];
    bool has_auto_pad;
    const float *w, *bias;
    zant_pack_slot slot;
};

extern "C" size_t zant_hip_blocked16_bytes(const int64_t dim[4]) { return dim ? zant_blocked_bytes(dim) : 0; }

extern "C" int zant_hip_to_blocked16_u8(zant_ctx *ctx, const uint8_t *x, const int64_t dim[4], uint8_t *xb) {
    if (!ctx || !x || !dim || !xb) return ZANT_NullPointer;
    for (int i = 0; i < 4; ++i)
        if (dim[i] <= 0 || dim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    return zant_to_blocked(ctx, x, dim[0], dim[1], dim[2] * dim[3], xb);
}

extern "C" int zant_hip_from_blocked16_u8(zant_ctx *ctx, const uint8_t *xb, const int64_t dim[4], uint8_t *y) {
    if (!ctx || !xb || !dim || !y) return ZANT_NullPointer;
    for (int i = 0; i < 4; ++i)
        if (dim[i] <= 0 || dim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    return zant_from_blocked(ctx, xb, dim[0], dim[1], dim[2] * dim[3], y);
}

extern "C" int zant_hip_qlinearconv_prepack(zant_ctx *ctx, const int64_t xdim[4], float x_scale, uint8_t x_zp, const int8_t *w,
                                            const int64_t wdim[4], const float *w_scale, int64_t n_wscale, const int8_t *w_zp,
                                            float y_scale, uint8_t y_zp, const int32_t *bias, const int64_t ydim[4],
                                            const int64_t stride[2], const int64_t pads[4], const int64_t dil[2], int64_t group,
                                            int act, float act_alpha, float act_scale, uint8_t act_zp, int x_layout,
                                            int y_layout, zant_qconv_plan **out) {
    if (!out) return ZANT_NullPointer;
    *out = nullptr;
    if (!ctx || !w || !w_scale) return ZANT_NullPointer;
    if ((x_layout != ZANT_LAYOUT_NCHW && x_layout != ZANT_LAYOUT_BLOCKED16) ||
        (y_layout != ZANT_LAYOUT_NCHW && y_layout != ZANT_LAYOUT_BLOCKED16))
        return ZANT_InvalidInput;
    // the checks of the plain entry point, without touching a tensor
    const int rc = zant_qlinearconv_layout_pool(ctx, nullptr, xdim, x_scale, x_zp, w, wdim, w_scale, n_wscale, w_zp, y_scale, y_zp,
                                                bias, nullptr, ydim, stride, pads, dil, group, act, act_alpha, act_scale, act_zp,
                                                x_layout, y_layout, 0, true, nullptr);
    if (rc) return rc;
    zant_qconv_plan *p = new (std::nothrow) zant_qconv_plan();
    if (!p) return ZANT_MemError;
    for (int i = 0; i < 4; ++i) { p->xdim[i] = xdim[i]; p->wdim[i] = wdim[i]; p->ydim[i] = ydim[i]; p->pads[i] = pads[i]; }
    for (int i = 0; i < 2; ++i) { p->stride[i] = stride[i]; p->dil[i] = dil[i]; }
    p->group = group; p->n_wscale = n_wscale;
    p->x_scale = x_scale; p->y_scale = y_scale; p->act_alpha = act_alpha; p->act_scale = act_scale;
    p->x_zp = x_zp; p->y_zp = y_zp; p->act_zp = act_zp;
    p->act = act; p->x_layout = x_layout; p->y_layout = y_layout;
    p->w = w; p->w_zp = w_zp; p->w_scale = w_scale; p->bias = bias;
    *out = p;
    return ZANT_OK;
}

extern "C" int zant_hip_qlinearconv_u8i8_packed(zant_ctx *ctx, zant_qconv_plan *p, const uint8_t *x, uint8_t *y) {
    if (!ctx || !p || !x || !y) return ZANT_NullPointer;
    return zant_qlinearconv_layout_pool(ctx, x, p->xdim, p->x_scale, p->x_zp, p->w, p->wdim, p->w_scale, p->n_wscale, p->w_zp,
                                        p->y_scale, p->y_zp, p->bias, y, p->ydim, p->stride, p->pads, p->dil, p->group, p->act,
                                        p->act_alpha, p->act_scale, p->act_zp, p->x_layout, p->y_layout, 0, false, &p->slot);
}

extern "C" void zant_hip_qlinearconv_plan_destroy(zant_ctx *ctx, zant_qconv_plan *p) {
    if (!p) return;
    zant_pack_slot_free(ctx, &p->slot);
    delete p;
}

extern "C" int zant_hip_conv2d_f32_prepack(zant_ctx *ctx, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                                           const float *bias, const int64_t ydim[4], const int64_t *stride, int n_stride,
                                           const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                                           const char *auto_pad, int fuse_act, int fuse_pool, zant_conv_plan **out) {
    if (!out) return ZANT_NullPointer;
    *out = nullptr;
    if (!ctx || !xdim || !wdim || !ydim || !w) return ZANT_NullPointer;
    if (n_stride < 0 || n_stride > 2 || n_pads < 0 || n_pads > 4 || n_dil < 0 || n_dil > 2) return ZANT_InvalidInput;  // what a plan stores
    if ((n_stride && !stride) || (n_pads && !pads) || (n_dil && !dil)) return ZANT_NullPointer;
    if (fuse_act != ZANT_ACT_NONE && fuse_act != ZANT_ACT_RELU) return ZANT_InvalidInput;
    // the shape checks of conv_lean (op_convolution.zig:42-219, 228-250), as the plain entry point makes them
    int64_t s[2], d[2], pd[4];
    const int rc = zant_conv_resolve(xdim, wdim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad, s, d, pd);
    if (rc) return rc;
    for (int i = 0; i < 4; ++i)
        if (xdim[i] <= 0 || wdim[i] <= 0 || xdim[i] > INT32_MAX || wdim[i] > INT32_MAX) return ZANT_InvalidDimensions;
    const int64_t PH = xdim[2] + pd[0] + pd[2], PW = xdim[3] + pd[1] + pd[3];
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1;
    if (PH < dkh || PW < dkw) return ZANT_InvalidDimensions;
    if (xdim[1] != wdim[1]) return ZANT_InputTensorsWrongShape;
    const int64_t OH = (PH - dkh) / s[0] + 1, OW = (PW - dkw) / s[1] + 1;
    const int64_t OHo = fuse_pool ? OH / 2 : OH, OWo = fuse_pool ? OW / 2 : OW;
    if (ydim[0] != xdim[0] || ydim[1] != wdim[0] || ydim[2] != OHo || ydim[3] != OWo) return ZANT_InvalidDimensions;
    if (fuse_pool) {
        // only the shapes whose convolution kernel takes the pool in its epilogue (stride and dilation 1: the matrix-core
        // kernel from 8 input channels on, the few-channel first-layer kernels): others are refused here, not run unfused
        const int rc2 = zant_conv2d_f32_fused_pool(ctx, nullptr, xdim, w, wdim, bias, nullptr, ydim, stride, n_stride, pads, n_pads, dil,
                                                   n_dil, group, auto_pad, fuse_act == ZANT_ACT_RELU, true, nullptr, 0, 0);
        if (rc2 < 0) return rc2;
        if (rc2 > 0) return ZANT_InvalidInput;
    }
    zant_conv_plan *p = new (std::nothrow) zant_conv_plan();
    if (!p) return ZANT_MemError;
    for (int i = 0; i < 4; ++i) { p->xdim[i] = xdim[i]; p->wdim[i] = wdim[i]; p->ydim[i] = ydim[i]; }
    for (int i = 0; i < n_stride; ++i) p->stride[i] = stride[i];
    for (int i = 0; i < n_pads; ++i) p->pads[i] = pads[i];
    for (int i = 0; i < n_dil; ++i) p->dil[i] = dil[i];
    p->n_stride = n_stride; p->n_pads = pads ? n_pads : -1; p->n_dil = dil ? n_dil : -1;
    p->group = group; p->fuse_act = fuse_act; p->fuse_pool = fuse_pool ? 1 : 0;
    p->has_auto_pad = auto_pad != nullptr;
    if (auto_pad) {
        size_t n = 0;
        while (auto_pad[n] && n < sizeof(p->auto_pad) - 1) { p->auto_pad[n] = auto_pad[n]; ++n; }
        p->auto_pad[n] = 0;
    }
    p->w = w; p->bias = bias;
    *out = p;
    return ZANT_OK;
}

extern "C" int zant_hip_conv2d_f32_packed(zant_ctx *ctx, zant_conv_plan *p, const float *x, float *y) {
    if (!ctx || !p || !x || !y) return ZANT_NullPointer;
    if (p->fuse_pool)
        return zant_conv2d_f32_fused_pool(ctx, x, p->xdim, p->w, p->wdim, p->bias, y, p->ydim, p->stride, p->n_stride,
                                          p->n_pads < 0 ? nullptr : p->pads, p->n_pads < 0 ? 0 : p->n_pads,
                                          p->n_dil < 0 ? nullptr : p->dil, p->n_dil < 0 ? 0 : p->n_dil, p->group,
                                          p->has_auto_pad ? p->auto_pad : nullptr, p->fuse_act == ZANT_ACT_RELU, false, &p->slot, 0, 0);
    return zant_conv2d_f32_slot(ctx, x, p->xdim, p->w, p->wdim, p->bias, y, p->ydim, p->stride, p->n_stride,
                                p->n_pads < 0 ? nullptr : p->pads, p->n_pads < 0 ? 0 : p->n_pads,
                                p->n_dil < 0 ? nullptr : p->dil, p->n_dil < 0 ? 0 : p->n_dil, p->group,
                                p->has_auto_pad ? p->auto_pad : nullptr, p->fuse_act, &p->slot);
}

extern "C" void zant_hip_conv2d_plan_destroy(zant_ctx *ctx, zant_conv_plan *p) {
    if (!p) return;
    zant_pack_slot_free(ctx, &p->slot);
    delete p;
}
