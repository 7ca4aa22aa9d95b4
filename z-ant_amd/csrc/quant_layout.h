// Internal interface of the int8 kernels that work on the channel-blocked activation layout.
//
// ZANT_LAYOUT_BLOCKED16 stores a [N, C, H, W] u8 tensor as [N][ceil(C/16)][H][W][16] bytes, every byte holding
// value ^ 0x80 (the two's-complement int8 "value - 128").  Sixteen channels of one position are one 16-byte unit:
// one global->LDS copy, one int8 MFMA operand, one vector store.  Bytes of channels >= C are unspecified but
// initialised (every consumer multiplies them by zero weights or drops them).  The public C ABI only ever sees
// NCHW u8; the model executor keeps int8 activations in this layout between layers.
#pragma once
#include "common.h"

// ZANT_LAYOUT_C4 stores a [N, C, H, W] f32 tensor with C a multiple of 4 as [N][C/4][H][W][4] floats: the four channels
// of a quad at one position are one 16-byte unit -- one global->LDS copy of the f32 matrix-core convolution (which keeps
// its patch as [position][4 channels] in LDS and otherwise copies 4 bytes at a time) and one vector store of the kernel
// that writes it.  Same size as NCHW.  Only between two convolution nodes of a model; never seen outside the executor.
// (ZANT_LAYOUT_NCHW = 0 and ZANT_LAYOUT_BLOCKED16 = 1 are public: include/zant_hip.h)
constexpr int ZANT_LAYOUT_C4 = 2;

static inline size_t zant_blocked_bytes(const int64_t dim[4]) {
    return size_t(dim[0]) * size_t((dim[1] + 15) / 16) * size_t(dim[2]) * size_t(dim[3]) * 16;
}

// zant_hip_qlinearconv_u8i8 with the layout of x and y chosen by the caller.
// fuse_pool: also max-pool 2x2/2 (floor, no padding) in the same kernel; ydim is then the pooled shape.  The first-layer
// kernel (1..4 input channels, 3x3, NCHW input) and the matrix-core kernel (blocked x and y, an order-preserving
// activation) do that: other shapes return 1 and run nothing.
// query_only: validate and report eligibility (ZANT_OK / 1 / error status) without touching any pointer.
// slot: where weight-derived scratch is kept across calls (nullptr: repacked on every call).
int zant_qlinearconv_layout_pool(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], float x_scale, uint8_t x_zp,
                                 const int8_t *w, const int64_t wdim[4], const float *w_scale, int64_t n_wscale,
                                 const int8_t *w_zp, float y_scale, uint8_t y_zp, const int32_t *bias, uint8_t *y,
                                 const int64_t ydim[4], const int64_t stride[2], const int64_t pads[4], const int64_t dil[2],
                                 int64_t group, int act, float act_alpha, float act_scale, uint8_t act_zp, int x_layout,
                                 int y_layout, int fuse_pool, bool query_only, zant_pack_slot *slot);

// The patch-stationary int8 matrix-core convolution (qconv_ps_i8.hip): 3x3, stride 1, pads <= 1, group 1, at least 32
// channels on both sides; with `pool` (a fused 2x2/2 max pool of even-sized planes into a blocked y: g.OH / g.OW stay the
// convolution's, y has half of each) up to 128 output channels.  x / y are NCHW u8 or blocked as said; ZANT_OK when it ran (with plan_only: would run), 1 when
// the shape is left to the other kernels, a negative status on failure.
struct QConvArgs;
int zant_qconv_ps(zant_ctx *ctx, const uint8_t *x, const int8_t *w, const float *w_scale, const int32_t *bias, uint8_t *y,
                  const ConvGeom &g, const QConvArgs &q, bool x_blocked, bool y_blocked, zant_pack_slot *slot, bool plan_only,
                  bool pool = false);

// Layout conversions (HW = H * W).
int zant_to_blocked(zant_ctx *ctx, const uint8_t *x, int64_t N, int64_t C, int64_t HW, uint8_t *xb);
int zant_from_blocked(zant_ctx *ctx, const uint8_t *xb, int64_t N, int64_t C, int64_t HW, uint8_t *y);

// MaxPool 2x2 / stride 2 / no padding (floor) on a blocked tensor; ydim = [N, C, H/2, W/2].
int zant_maxpool2x2_blocked(zant_ctx *ctx, const uint8_t *xb, const int64_t xdim[4], uint8_t *yb);

// Elementwise operators on buffers whose bytes hold value ^ flip (flip = 0x80 for blocked tensors, 0 for NCHW).
int zant_qlinear_act_flip(zant_ctx *ctx, const uint8_t *x, int64_t n, float x_scale, uint8_t x_zp, int act, float alpha,
                          float y_scale, uint8_t y_zp, uint8_t *y, int flip);
int zant_qlinear_add_flip(zant_ctx *ctx, const uint8_t *a, float a_scale, uint8_t a_zp, const uint8_t *b, float b_scale,
                          uint8_t b_zp, float y_scale, uint8_t y_zp, uint8_t *y, int64_t n, int flip);

// Global average pool of a blocked tensor; y is [N, C, 1, 1] in y_layout.
int zant_qgap_blocked(zant_ctx *ctx, const uint8_t *xb, const int64_t xdim[4], float x_scale, uint8_t x_zp, float y_scale,
                      uint8_t y_zp, uint8_t *y, int y_layout);

// Weight packing shared by the int8 matrix-core kernels (device pointers; launches on the context's stream).
// Dense: [chunk of 32 input channels][block of k_blk output channels][tap][half][k_blk][16] int8, zero padded; per
// output channel the requantisation multiplier (x_scale * w_scale / y_scale) and the integer correction
// (bias + (128 - x_zp) * sum of weights); padvec = 16 bytes of x_zp - 128.
int zant_qpack_dense(zant_ctx *ctx, const int8_t *w, const float *w_scale, int64_t n_wscale, const int32_t *bias, int K, int C,
                     int T, int k_blk, float x_scale, int x_zp, float y_scale, int8_t *wp, float *mult, int32_t *corr,
                     int8_t *padvec);
// Depthwise 3x3: one dword per (channel, tap) with the weight in byte (channel % 4) and zeros elsewhere, at
// wm[((channel / 4) * 9 + tap) * 4 + channel % 4]; multipliers and corrections as above, for kpad channels.
int zant_qpack_depthwise(zant_ctx *ctx, const int8_t *w, const float *w_scale, int64_t n_wscale, const int32_t *bias, int K,
                         int kpad, float x_scale, int x_zp, float y_scale, uint32_t *wm, float *mult, int32_t *corr);

// One QLinearConv of a fused block: weights, requantisation and the optional fused activation (conv output quantised
// with y_scale / y_zp, the activation's output with act_scale / act_zp).
struct zant_qconv_desc {
    const int8_t *w;
    const float *w_scale;
    int64_t n_wscale;
    const int32_t *bias;
    int64_t K, C;          // output channels, input channels (depthwise: C == K)
    float x_scale; int x_zp;
    float y_scale; int y_zp;
    int act; float act_alpha; float act_scale; int act_zp;
};

// MobileNetV2's inverted residual block in one kernel, on blocked tensors: 1x1 expansion (+activation) -> depthwise 3x3,
// pads 1, stride 1 or 2 (+activation) -> 1x1 projection (-> QLinearAdd with the block input when `residual`).  The
// expanded tensors live only in LDS.  query_only: report eligibility (ZANT_OK / 1) without touching pointers.
// residual: y = sat(rne(((p - p_zp) * p_scale + (x - x_zp) * x_scale) / add_scale) + add_zp), p the projection output.
int zant_qblock_blocked(zant_ctx *ctx, const uint8_t *x, const int64_t xdim[4], const zant_qconv_desc *expand,
                        const zant_qconv_desc *dw, int64_t dw_stride, const zant_qconv_desc *project, int residual,
                        float add_scale, int add_zp, uint8_t *y, const int64_t ydim[4], bool query_only, zant_pack_slot *slot);

// One block of a chain: the arguments of zant_qblock_blocked.
struct zant_qblock_call {
    const uint8_t *x;
    const int64_t *xdim;
    const zant_qconv_desc *expand, *dw;
    int64_t dw_stride;
    const zant_qconv_desc *project;
    int residual;
    float add_scale;
    int add_zp;
    uint8_t *y;
    const int64_t *ydim;
    zant_pack_slot *slot;
};
// Consecutive blocks (each one's input is the one before's output) as one launch; 1 when they do not form a chain.
int zant_qblock_chain(zant_ctx *ctx, int n, const zant_qblock_call *calls, bool query_only);
