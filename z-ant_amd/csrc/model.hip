// zant_model: the GPU form of a generated library (reference src/codeGen/predict.zig:23-70, 265-377).
//
// The reference emits one zero-initialised static array per node output, memsets all of them at the
// top of every predict(), and calls one *_lean operator per ONNX node.  Here the node list is built
// once (ready order), then finalize():
//   - folds a constant per-channel Add into the preceding bias-less Conv (the mnist-8 pattern
//     Conv -> Add({M,1,1}) -> Relu, src/codeGen/hardcoded/hardcoded_mnist8.zig:186-209),
//   - fuses Relu into the Conv / Gemm that feeds it, and the Dequantize -> activation -> Quantize
//     step into the QLinearConv that feeds it (one kernel epilogue instead of a pass over HBM),
//   - turns Reshape into a view,
//   - assigns every remaining activation an offset in ONE device allocation by liveness
//     (first fit over [definition, last use] intervals), and uploads all parameters into one
//     allocation.
// run() then enqueues the operator kernels on arena pointers: no allocation, no memset (every
// kernel writes its whole output).
#include <algorithm>
#include <cmath>
#include <vector>

#include "common.h"
#include "quant_layout.h"

namespace {

enum OpKind {
    OP_CONV, OP_RELU, OP_LEAKY, OP_MAXPOOL, OP_RESHAPE, OP_GEMM, OP_MATMUL, OP_ADD_CONST, OP_ADD, OP_SOFTMAX,
    OP_QUANT, OP_DEQUANT, OP_QCONV, OP_QACT, OP_QADD, OP_QGAP, OP_QBLOCK,
    OP_SIGMOID, OP_REDUCE_MEAN, OP_CONCAT, OP_RESIZE, OP_AVGPOOL, OP_BATCHNORM
};

struct MTensor {
    int dtype = ZANT_F32;
    int rank = 0;
    int64_t dim[8] = {0};
    float scale = 1.0f;   // quantisation parameters of a u8 tensor
    int zp = 0;
    int layout = ZANT_LAYOUT_NCHW;  // how the storage root keeps a rank-4 u8 tensor (set by finalize)
    int alias_of = -1;    // shares storage with that tensor (views, fused activations)
    size_t offset = 0;    // in the arena, valid for storage roots after finalize
    int def = -1, last = -1;
    size_t bytes() const {
        size_t n = dtype == ZANT_F32 ? 4 : 1;
        for (int i = 0; i < rank; ++i) n *= size_t(dim[i]);
        return n;
    }
    size_t storage_bytes() const { return layout == ZANT_LAYOUT_BLOCKED16 ? zant_blocked_bytes(dim) : bytes(); }
};

struct Param {           // a host copy of a constant until finalize, then its place in the parameter block
    std::vector<char> host;
    size_t offset = 0;
};

struct MNode {
    int op = 0;
    int in0 = -1, in1 = -1, out = -1;
    bool skip = false;            // fused into its producer or turned into a view
    int fuse_act = ZANT_ACT_NONE; // activation applied in this node's epilogue
    bool fuse_pool = false;       // a following 2x2/2 MaxPool is computed in this node's kernel
    float act_alpha = 0.0f, act_scale = 1.0f;
    int act_zp = 0;
    int w = -1, b = -1, c = -1, ws = -1;  // parameter indices
    int64_t wdim[4] = {0}, cdim[4] = {0};
    int c_rank = 0;
    int64_t stride[2] = {1, 1}, pads[4] = {0, 0, 0, 0}, dil[2] = {1, 1}, kernel[2] = {1, 1};
    int n_stride = 2, n_pads = 0, n_dil = 0;
    bool has_pads = false, has_dil = false;
    int64_t group = 1;
    std::string auto_pad;
    bool has_auto_pad = false;
    int pool_pad = ZANT_PAD_NOTSET;
    float alpha = 1.0f, beta = 1.0f, slope = 0.0f;
    int trans_a = 0, trans_b = 0;
    int64_t n_wscale = 1;
    int act = ZANT_ACT_NONE;
    int b_rank = 0;
    int64_t bdim[8] = {0};
    mutable zant_pack_slot slot;  // packed weights / tables of this node, filled by its first launch
    // OP_QBLOCK (a fused inverted residual block): the expansion, depthwise, projection and residual Add nodes
    int blk_expand = -1, blk_dw = -1, blk_project = -1, blk_add = -1;
    // consecutive blocks run as one launch (zant_qblock_chain): the first one lists the others, which are skipped
    std::vector<int> chain;
    int chain_head = -1;
    std::vector<int> more;        // inputs of a Concat beyond the first two
    std::vector<int64_t> axes;    // ReduceMean axes / Resize sizes
    std::vector<float> scales;    // Resize scales
    int64_t axis = 0;             // Concat axis
    int keepdims = 1, coord_mode = 0;
};

}  // namespace

struct zant_model {
    zant_ctx *ctx = nullptr;
    std::vector<MTensor> t;
    std::vector<MNode> n;
    std::vector<Param> p;
    bool finalized = false;
    int input = -1, output = -1;
    void *params_dev = nullptr;
    size_t arena_bytes = 0, unfused_bytes = 0;
    int launches = 0;
    std::vector<char> result_host;  // what predict() hands out
    std::vector<std::string> launch_kernels;  // device function of each launch's main kernel, filled by zant_model_profile
    bool no_chain = false;  // run chained blocks one by one (zant_model_read_tensor: a chain overwrites its own intermediates)
};

namespace {

zant_model *g_predict_model = nullptr;

int root_of(const zant_model *m, int id) {
    while (m->t[id].alias_of >= 0) id = m->t[id].alias_of;
    return id;
}

int add_tensor(zant_model *m, int dtype, const int64_t *dims, int rank, float scale, int zp) {
    MTensor t;
    t.dtype = dtype; t.rank = rank; t.scale = scale; t.zp = zp;
    for (int i = 0; i < rank; ++i) t.dim[i] = dims[i];
    m->t.push_back(t);
    return int(m->t.size()) - 1;
}

int add_param(zant_model *m, const void *src, size_t bytes) {
    Param p;
    p.host.assign(static_cast<const char *>(src), static_cast<const char *>(src) + bytes);
    m->p.push_back(std::move(p));
    return int(m->p.size()) - 1;
}

bool valid_tensor(const zant_model *m, int id) { return m && id >= 0 && id < int(m->t.size()); }

void *tensor_ptr(zant_model *m, int id) {
    return static_cast<char *>(m->ctx->arena) + m->t[root_of(m, id)].offset;
}

const void *param_ptr(const zant_model *m, int idx) {
    return idx < 0 ? nullptr : static_cast<const char *>(m->params_dev) + m->p[idx].offset;
}

int consumers(const zant_model *m, int tensor, int *only) {
    int cnt = 0;
    for (size_t i = 0; i < m->n.size(); ++i)
        if (m->n[i].in0 == tensor || m->n[i].in1 == tensor ||
            std::find(m->n[i].more.begin(), m->n[i].more.end(), tensor) != m->n[i].more.end()) { ++cnt; *only = int(i); }
    return cnt;
}

int producer(const zant_model *m, int tensor) {
    for (size_t i = 0; i < m->n.size(); ++i)
        if (m->n[i].out == tensor) return int(i);
    return -1;
}

int append(zant_model *m, MNode &node, int dtype, const int64_t *dims, int rank, float scale, int zp) {
    if (m->finalized) return ZANT_InvalidInput;
    node.out = add_tensor(m, dtype, dims, rank, scale, zp);
    m->n.push_back(node);
    return node.out;
}

// One QLinearConv node as the fused block kernel takes it.  x_scale / x_zp: the tensor the node reads.
zant_qconv_desc qconv_desc(const zant_model *m, const MNode &cv, float x_scale, int x_zp) {
    const MTensor &to = m->t[cv.out];
    zant_qconv_desc d;
    d.w = static_cast<const int8_t *>(param_ptr(m, cv.w));
    d.w_scale = static_cast<const float *>(param_ptr(m, cv.ws));
    d.n_wscale = cv.n_wscale;
    d.bias = static_cast<const int32_t *>(param_ptr(m, cv.b));
    d.K = cv.wdim[0];
    d.C = cv.group > 1 ? cv.wdim[0] : cv.wdim[1];
    d.x_scale = x_scale; d.x_zp = x_zp;
    d.y_scale = cv.fuse_act ? cv.act_scale : to.scale;
    d.y_zp = cv.fuse_act ? cv.act_zp : to.zp;
    d.act = cv.fuse_act; d.act_alpha = cv.act_alpha;
    d.act_scale = to.scale; d.act_zp = to.zp;
    return d;
}

// The three convolutions of a fused block (each reads what the one before it stores) and the residual Add's output.
void fill_block_descs(const zant_model *m, const MNode &nd, zant_qconv_desc d[3], float *add_scale, int *add_zp) {
    const MNode &ex = m->n[nd.blk_expand], &dw = m->n[nd.blk_dw], &pj = m->n[nd.blk_project];
    const MTensor &ti = m->t[nd.in0];
    d[0] = qconv_desc(m, ex, ti.scale, ti.zp);
    d[1] = qconv_desc(m, dw, m->t[ex.out].scale, m->t[ex.out].zp);
    d[2] = qconv_desc(m, pj, m->t[dw.out].scale, m->t[dw.out].zp);
    if (nd.blk_add >= 0) {
        const MTensor &ao = m->t[m->n[nd.blk_add].out];
        *add_scale = ao.scale;
        *add_zp = ao.zp;
    }
}

// The block `head` and the blocks `more` after it (head.chain when null) as one launch; query_only: would they?
int run_block_chain(zant_model *m, const MNode &head, bool query_only, const std::vector<int> *more = nullptr) {
    const std::vector<int> &rest = more ? *more : head.chain;
    constexpr int kMax = 16;
    const int n = 1 + int(rest.size());
    if (n > kMax) return 1;
    zant_qconv_desc d[kMax][3];
    zant_qblock_call calls[kMax];
    for (int b = 0; b < n; ++b) {
        const MNode &nd = b == 0 ? head : m->n[rest[b - 1]];
        float add_scale = 1.0f;
        int add_zp = 0;
        fill_block_descs(m, nd, d[b], &add_scale, &add_zp);
        zant_qblock_call &c = calls[b];
        c.x = query_only ? nullptr : static_cast<const uint8_t *>(tensor_ptr(m, nd.in0));
        c.xdim = m->t[nd.in0].dim;
        c.expand = &d[b][0]; c.dw = &d[b][1]; c.project = &d[b][2];
        c.dw_stride = m->n[nd.blk_dw].stride[0];
        c.residual = nd.blk_add >= 0;
        c.add_scale = add_scale; c.add_zp = add_zp;
        c.y = query_only ? nullptr : static_cast<uint8_t *>(tensor_ptr(m, nd.out));
        c.ydim = m->t[nd.out].dim;
        c.slot = query_only ? nullptr : &nd.slot;
    }
    return zant_qblock_chain(m->ctx, n, calls, query_only);
}

int run_node(zant_model *m, const MNode &nd) {
    zant_ctx *ctx = m->ctx;
    const MTensor &ti = m->t[nd.in0];
    const MTensor &to = m->t[nd.out];
    const void *x = tensor_ptr(m, nd.in0);
    void *y = tensor_ptr(m, nd.out);
    const int lin = m->t[root_of(m, nd.in0)].layout, lout = m->t[root_of(m, nd.out)].layout;
    switch (nd.op) {
    case OP_CONV:
        if (nd.fuse_pool)
            return zant_conv2d_f32_fused_pool(ctx, static_cast<const float *>(x), ti.dim,
                                              static_cast<const float *>(param_ptr(m, nd.w)), nd.wdim,
                                              static_cast<const float *>(param_ptr(m, nd.b)), static_cast<float *>(y), to.dim,
                                              nd.stride, nd.n_stride, nd.has_pads ? nd.pads : nullptr, nd.n_pads,
                                              nd.has_dil ? nd.dil : nullptr, nd.n_dil, nd.group,
                                              nd.has_auto_pad ? nd.auto_pad.c_str() : nullptr, nd.fuse_act == ZANT_ACT_RELU, false, &nd.slot,
                                              lin == ZANT_LAYOUT_C4, lout == ZANT_LAYOUT_C4);
        if (lout == ZANT_LAYOUT_C4) return ZANT_InvalidInput;  // no unpooled kernel writes that layout (finalize never asks)
        return zant_conv2d_f32_slot(ctx, static_cast<const float *>(x), ti.dim, static_cast<const float *>(param_ptr(m, nd.w)),
                                    nd.wdim, static_cast<const float *>(param_ptr(m, nd.b)), static_cast<float *>(y), to.dim,
                                    nd.stride, nd.n_stride, nd.has_pads ? nd.pads : nullptr, nd.n_pads,
                                    nd.has_dil ? nd.dil : nullptr, nd.n_dil, nd.group,
                                    nd.has_auto_pad ? nd.auto_pad.c_str() : nullptr, nd.fuse_act, &nd.slot, lin == ZANT_LAYOUT_C4);
    case OP_RELU:
        return zant_hip_relu_f32(ctx, static_cast<const float *>(x), static_cast<float *>(y), int64_t(ti.bytes() / 4));
    case OP_LEAKY:
        return zant_hip_leaky_relu_f32(ctx, static_cast<const float *>(x), nd.slope, static_cast<float *>(y),
                                       int64_t(ti.bytes() / 4));
    case OP_MAXPOOL:
        if (ti.dtype == ZANT_U8 && lin == ZANT_LAYOUT_BLOCKED16)
            return zant_maxpool2x2_blocked(ctx, static_cast<const uint8_t *>(x), ti.dim, static_cast<uint8_t *>(y));
        if (ti.dtype == ZANT_U8)
            return zant_hip_maxpool2d_u8(ctx, static_cast<const uint8_t *>(x), ti.dim, static_cast<uint8_t *>(y), to.dim,
                                         nd.kernel, nd.stride, nd.dil, nd.pads, 4, nd.pool_pad);
        return zant_hip_maxpool2d_f32(ctx, static_cast<const float *>(x), ti.dim, static_cast<float *>(y), to.dim, nd.kernel,
                                      nd.stride, nd.dil, nd.pads, 4, nd.pool_pad);
    case OP_AVGPOOL:
        return zant_hip_avgpool2d_f32(ctx, static_cast<const float *>(x), ti.dim, static_cast<float *>(y), to.dim, nd.kernel,
                                      nd.stride, nd.pads, nd.keepdims /* count_include_pad */);
    case OP_BATCHNORM:
        return zant_hip_batchnorm_f32(ctx, static_cast<const float *>(x), ti.dim, ti.rank,
                                      static_cast<const float *>(param_ptr(m, nd.w)), static_cast<const float *>(param_ptr(m, nd.b)),
                                      static_cast<const float *>(param_ptr(m, nd.c)), static_cast<const float *>(param_ptr(m, nd.ws)),
                                      nd.alpha /* epsilon */, static_cast<float *>(y));
    case OP_GEMM:
        return zant_hip_gemm_f32(ctx, static_cast<const float *>(x), ti.dim, static_cast<const float *>(param_ptr(m, nd.w)),
                                 nd.wdim, static_cast<const float *>(param_ptr(m, nd.c)), nd.cdim, nd.c_rank, nd.alpha,
                                 nd.beta, nd.trans_a, nd.trans_b, static_cast<float *>(y), to.dim, nd.fuse_act);
    case OP_MATMUL:
        return zant_hip_matmul_f32(ctx, static_cast<const float *>(x), ti.dim, ti.rank,
                                   static_cast<const float *>(param_ptr(m, nd.w)), nd.bdim, nd.b_rank, static_cast<float *>(y));
    case OP_ADD_CONST:
        return zant_hip_add_f32(ctx, static_cast<const float *>(x), ti.dim, ti.rank,
                                static_cast<const float *>(param_ptr(m, nd.c)), nd.cdim, nd.c_rank, static_cast<float *>(y),
                                nullptr, nullptr);
    case OP_ADD: {
        const MTensor &tb = m->t[nd.in1];
        return zant_hip_add_f32(ctx, static_cast<const float *>(x), ti.dim, ti.rank,
                                static_cast<const float *>(tensor_ptr(m, nd.in1)), tb.dim, tb.rank, static_cast<float *>(y),
                                nullptr, nullptr);
    }
    case OP_SOFTMAX:
        return zant_hip_softmax_f32(ctx, static_cast<const float *>(x), static_cast<float *>(y), ti.dim[0], ti.dim[1]);
    case OP_SIGMOID:
        return zant_hip_sigmoid_f32(ctx, static_cast<const float *>(x), static_cast<float *>(y), int64_t(ti.bytes() / 4));
    case OP_REDUCE_MEAN: {
        int64_t ydim[8];
        int yr = 0;
        return zant_hip_reduce_mean_f32(ctx, static_cast<const float *>(x), ti.dim, ti.rank, nd.axes.data(), int(nd.axes.size()),
                                        nd.keepdims, 0, static_cast<float *>(y), ydim, &yr);
    }
    case OP_CONCAT: {
        const void *xs[16];
        const int64_t *dd[16];
        int rr[16], n = 0;
        for (int in : {nd.in0, nd.in1})
            if (in >= 0) { xs[n] = tensor_ptr(m, in); dd[n] = m->t[in].dim; rr[n++] = m->t[in].rank; }
        for (int in : nd.more) { xs[n] = tensor_ptr(m, in); dd[n] = m->t[in].dim; rr[n++] = m->t[in].rank; }
        int64_t ydim[8];
        int yr = 0;
        return zant_hip_concatenate(ctx, xs, dd, rr, n, nd.axis, ti.dtype == ZANT_F32 ? 4 : 1, y, ydim, &yr);
    }
    case OP_RESIZE: {
        int64_t ydim[8];
        const bool by_scale = !nd.scales.empty();
        return zant_hip_resize_nearest(ctx, x, ti.dim, ti.rank, ti.dtype == ZANT_F32 ? 4 : 1, by_scale ? nd.scales.data() : nullptr,
                                       by_scale ? nullptr : nd.axes.data(), ti.rank, nd.coord_mode, y, ydim);
    }
    case OP_QUANT:
        return zant_hip_quantize_linear_f32_u8(ctx, static_cast<const float *>(x), ti.dim, ti.rank,
                                               static_cast<const float *>(param_ptr(m, nd.ws)),
                                               static_cast<const uint8_t *>(param_ptr(m, nd.b)), 1, 1,
                                               static_cast<uint8_t *>(y));
    case OP_DEQUANT:
        return zant_hip_dequantize_linear_u8_f32(ctx, static_cast<const uint8_t *>(x), ti.dim, ti.rank,
                                                 static_cast<const float *>(param_ptr(m, nd.ws)),
                                                 static_cast<const uint8_t *>(param_ptr(m, nd.b)), 1, 1,
                                                 static_cast<float *>(y));
    case OP_QCONV:
        return zant_qlinearconv_layout_pool(ctx, static_cast<const uint8_t *>(x), ti.dim, ti.scale, uint8_t(ti.zp),
                                            static_cast<const int8_t *>(param_ptr(m, nd.w)), nd.wdim,
                                            static_cast<const float *>(param_ptr(m, nd.ws)), nd.n_wscale, nullptr,
                                            nd.fuse_act ? nd.act_scale : to.scale, uint8_t(nd.fuse_act ? nd.act_zp : to.zp),
                                            static_cast<const int32_t *>(param_ptr(m, nd.b)), static_cast<uint8_t *>(y), to.dim,
                                            nd.stride, nd.pads, nd.dil, nd.group, nd.fuse_act, nd.act_alpha, to.scale,
                                            uint8_t(to.zp), lin, lout, nd.fuse_pool ? 1 : 0, false, &nd.slot);
    case OP_QACT:
        return zant_qlinear_act_flip(ctx, static_cast<const uint8_t *>(x), int64_t(m->t[root_of(m, nd.in0)].storage_bytes()),
                                     ti.scale, uint8_t(ti.zp), nd.act, nd.act_alpha, to.scale, uint8_t(to.zp),
                                     static_cast<uint8_t *>(y), lin == ZANT_LAYOUT_BLOCKED16 ? 0x80 : 0);
    case OP_QADD: {
        const MTensor &tb = m->t[nd.in1];
        return zant_qlinear_add_flip(ctx, static_cast<const uint8_t *>(x), ti.scale, uint8_t(ti.zp),
                                     static_cast<const uint8_t *>(tensor_ptr(m, nd.in1)), tb.scale, uint8_t(tb.zp), to.scale,
                                     uint8_t(to.zp), static_cast<uint8_t *>(y),
                                     int64_t(m->t[root_of(m, nd.in0)].storage_bytes()), lin == ZANT_LAYOUT_BLOCKED16 ? 0x80 : 0);
    }
    case OP_QBLOCK: {
        zant_qconv_desc d[3];
        float add_scale = 1.0f;
        int add_zp = 0;
        const bool chained = !nd.chain.empty() && !m->no_chain;
        if (chained) {
            const int rc = run_block_chain(m, nd, false);
            if (rc != 1) return rc;  // (1: not a chain after all: the blocks one by one, this one first)
        }
        fill_block_descs(m, nd, d, &add_scale, &add_zp);
        int rc = zant_qblock_blocked(ctx, static_cast<const uint8_t *>(x), ti.dim, &d[0], &d[1], m->n[nd.blk_dw].stride[0], &d[2],
                                     nd.blk_add >= 0, add_scale, add_zp, static_cast<uint8_t *>(y), to.dim, false, &nd.slot);
        if (chained)
            for (size_t f = 0; f < nd.chain.size() && !rc; ++f) {
                m->no_chain = true;
                rc = run_node(m, m->n[nd.chain[f]]);
                m->no_chain = false;
            }
        return rc;
    }
    case OP_QGAP:
        if (lin == ZANT_LAYOUT_BLOCKED16)
            return zant_qgap_blocked(ctx, static_cast<const uint8_t *>(x), ti.dim, ti.scale, uint8_t(ti.zp), to.scale,
                                     uint8_t(to.zp), static_cast<uint8_t *>(y), lout);
        return zant_hip_qlinear_global_avgpool_u8(ctx, static_cast<const uint8_t *>(x), ti.dim, ti.scale, uint8_t(ti.zp),
                                                  to.scale, uint8_t(to.zp), static_cast<uint8_t *>(y));
    default:
        return ZANT_InvalidInput;
    }
}

}  // namespace

extern "C" int zant_model_create(zant_ctx *ctx, zant_model **out) {
    if (!out) return ZANT_NullPointer;  // ctx may be NULL: such a model validates nodes and answers shape queries only
    zant_model *m = new (std::nothrow) zant_model();
    if (!m) return ZANT_MemError;
    m->ctx = ctx;
    *out = m;
    return ZANT_OK;
}

extern "C" void zant_model_destroy(zant_model *m) {
    if (!m) return;
    if (g_predict_model == m) g_predict_model = nullptr;
    if (m->params_dev) {
        (void)hipStreamSynchronize(m->ctx->stream);
        (void)hipFree(m->params_dev);
    }
    for (MNode &nd : m->n) zant_pack_slot_free(m->ctx, &nd.slot);
    delete m;
}

extern "C" int zant_model_input(zant_model *m, int dtype, const int64_t *dims, int rank, float scale, int zp) {
    if (!m || !dims) return ZANT_NullPointer;
    if (m->finalized || m->input >= 0 || rank < 1 || rank > 8 || (dtype != ZANT_F32 && dtype != ZANT_U8)) return ZANT_InvalidInput;
    for (int i = 0; i < rank; ++i)
        if (dims[i] <= 0) return ZANT_InvalidDimensions;
    m->input = add_tensor(m, dtype, dims, rank, scale, zp);
    return m->input;
}

extern "C" int zant_model_conv(zant_model *m, int x, const float *w, const int64_t wdim[4], const float *bias,
                               const int64_t *stride, int n_stride, const int64_t *pads, int n_pads, const int64_t *dil,
                               int n_dil, int64_t group, const char *auto_pad) {
    if (!valid_tensor(m, x) || !w || !wdim || !stride) return ZANT_NullPointer;
    const MTensor &tx = m->t[x];
    if (tx.rank != 4 || tx.dtype != ZANT_F32) return ZANT_InvalidDimensions;
    if (n_stride < 1 || n_stride > 2 || n_pads > 4 || n_dil > 2) return ZANT_InvalidInput;
    // shape inference runs the operator's own rule; the generated code passes pads only with "NOTSET" in mind
    int64_t s[2], d[2], p[4];
    int rc = zant_conv_resolve(tx.dim, wdim, stride, n_stride, pads, n_pads, dil, n_dil, group, auto_pad, s, d, p);
    if (rc) return rc;
    const int64_t dkh = (wdim[2] - 1) * d[0] + 1, dkw = (wdim[3] - 1) * d[1] + 1;
    const int64_t PH = tx.dim[2] + p[0] + p[2], PW = tx.dim[3] + p[1] + p[3];
    if (PH < dkh || PW < dkw || tx.dim[1] != wdim[1]) return ZANT_InvalidDimensions;
    const int64_t ydim[4] = {tx.dim[0], wdim[0], (PH - dkh) / s[0] + 1, (PW - dkw) / s[1] + 1};
    MNode nd;
    nd.op = OP_CONV; nd.in0 = x;
    for (int i = 0; i < 4; ++i) nd.wdim[i] = wdim[i];
    nd.w = add_param(m, w, size_t(wdim[0] * wdim[1] * wdim[2] * wdim[3]) * 4);
    if (bias) nd.b = add_param(m, bias, size_t(wdim[0]) * 4);
    nd.n_stride = n_stride;
    for (int i = 0; i < n_stride; ++i) nd.stride[i] = stride[i];
    nd.has_pads = pads != nullptr; nd.n_pads = n_pads;
    for (int i = 0; pads && i < n_pads; ++i) nd.pads[i] = pads[i];
    nd.has_dil = dil != nullptr; nd.n_dil = n_dil;
    for (int i = 0; dil && i < n_dil; ++i) nd.dil[i] = dil[i];
    nd.group = group;
    nd.has_auto_pad = auto_pad != nullptr;
    if (auto_pad) nd.auto_pad = auto_pad;
    return append(m, nd, ZANT_F32, ydim, 4, 1.0f, 0);
}

static int unary_same_shape(zant_model *m, int x, int op, float slope) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_F32) return ZANT_InvalidInput;
    MNode nd;
    nd.op = op; nd.in0 = x; nd.slope = slope;
    return append(m, nd, ZANT_F32, tx.dim, tx.rank, 1.0f, 0);
}

extern "C" int zant_model_relu(zant_model *m, int x) { return unary_same_shape(m, x, OP_RELU, 0.0f); }
extern "C" int zant_model_leaky_relu(zant_model *m, int x, float slope) { return unary_same_shape(m, x, OP_LEAKY, slope); }

extern "C" int zant_model_maxpool(zant_model *m, int x, const int64_t kernel[2], const int64_t strides[2],
                                  const int64_t dil[2], const int64_t pads[4], int auto_pad, int ceil_mode) {
    if (!valid_tensor(m, x) || !kernel || !strides || !dil || !pads) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.rank != 4) return ZANT_InvalidDimensions;
    int64_t ydim[4];
    int rc = zant_hip_maxpool2d_out_shape(tx.dim, kernel, strides, dil, pads, auto_pad, ceil_mode, ydim);
    if (rc) return rc;
    MNode nd;
    nd.op = OP_MAXPOOL; nd.in0 = x; nd.pool_pad = auto_pad;
    for (int i = 0; i < 2; ++i) { nd.kernel[i] = kernel[i]; nd.stride[i] = strides[i]; nd.dil[i] = dil[i]; }
    for (int i = 0; i < 4; ++i) nd.pads[i] = pads[i];
    return append(m, nd, tx.dtype, ydim, 4, tx.scale, tx.zp);
}

extern "C" int zant_model_avgpool(zant_model *m, int x, const int64_t kernel[2], const int64_t strides[2],
                                  const int64_t pads[4], int ceil_mode, int count_include_pad) {
    if (!valid_tensor(m, x) || !kernel || !strides) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.rank != 4) return ZANT_InputTensorDimensionMismatch;  // op_pooling.zig:229-231
    if (tx.dtype != ZANT_F32) return ZANT_InvalidInput;
    int64_t ydim[4];
    int rc = zant_hip_avgpool2d_out_shape(tx.dim, kernel, strides, pads, ceil_mode, ydim);
    if (rc) return rc;
    if (pads)
        for (int i = 0; i < 4; ++i)
            if (pads[i] >= (i & 1 ? kernel[1] : kernel[0])) return ZANT_InvalidPadding;
    MNode nd;
    nd.op = OP_AVGPOOL; nd.in0 = x;
    nd.keepdims = count_include_pad != 0;  // (the field ReduceMean uses for its own flag)
    for (int i = 0; i < 2; ++i) { nd.kernel[i] = kernel[i]; nd.stride[i] = strides[i]; }
    for (int i = 0; i < 4; ++i) nd.pads[i] = pads ? pads[i] : 0;
    return append(m, nd, ZANT_F32, ydim, 4, 1.0f, 0);
}

extern "C" int zant_model_batchnorm(zant_model *m, int x, const float *gamma, const float *beta, const float *mean,
                                    const float *var, int64_t features, float epsilon) {
    if (!valid_tensor(m, x) || !gamma || !beta || !mean || !var) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_F32) return ZANT_InvalidInput;
    if (tx.rank < 2) return ZANT_InvalidDimensions;
    if (features != tx.dim[1]) return ZANT_InputTensorDimensionMismatch;
    MNode nd;
    nd.op = OP_BATCHNORM; nd.in0 = x;
    nd.alpha = epsilon;  // (the field Gemm uses for its own scalar)
    nd.w = add_param(m, gamma, size_t(features) * 4);
    nd.b = add_param(m, beta, size_t(features) * 4);
    nd.c = add_param(m, mean, size_t(features) * 4);
    nd.ws = add_param(m, var, size_t(features) * 4);
    return append(m, nd, ZANT_F32, tx.dim, tx.rank, 1.0f, 0);
}

extern "C" int zant_model_reshape(zant_model *m, int x, const int64_t *new_shape, int rank) {
    if (!valid_tensor(m, x) || !new_shape) return ZANT_NullPointer;
    if (rank < 1 || rank > 8) return ZANT_InvalidInput;
    const MTensor tx = m->t[x];
    int64_t ydim[8];
    // shape resolution of reshape_lean (0 copies, -1 infers); no data moves: the result is a view
    int rc = zant_hip_reshape(m->ctx, nullptr, tx.dim, tx.rank, 1, new_shape, rank, nullptr, ydim);
    if (rc) return rc;
    MNode nd;
    nd.op = OP_RESHAPE; nd.in0 = x;
    return append(m, nd, tx.dtype, ydim, rank, tx.scale, tx.zp);
}

extern "C" int zant_model_gemm(zant_model *m, int a, const float *b, const int64_t bdim[4], const float *c,
                               const int64_t *cdim, int c_rank, float alpha, float beta, int trans_a, int trans_b) {
    if (!valid_tensor(m, a) || !b || !bdim) return ZANT_NullPointer;
    const MTensor ta = m->t[a];
    if (ta.dtype != ZANT_F32) return ZANT_InvalidInput;
    int64_t ydim[4];
    int rc = zant_hip_gemm_check(ta.dim, ta.rank, bdim, 4, cdim, c_rank, c != nullptr, trans_a, trans_b, ydim);
    if (rc) return rc;
    // lean_gemm multiplies the first matrix only and leaves the other planes of the (zero filled) result alone
    // (op_gemm.zig:126-128, op_mat_mul.zig:95-97); the arena is not zero filled per pass, so batched shapes are refused
    if (ta.dim[0] * ta.dim[1] != 1) return ZANT_InvalidInput;
    MNode nd;
    nd.op = OP_GEMM; nd.in0 = a;
    for (int i = 0; i < 4; ++i) nd.wdim[i] = bdim[i];
    nd.w = add_param(m, b, size_t(bdim[0] * bdim[1] * bdim[2] * bdim[3]) * 4);
    if (c) {
        nd.c_rank = c_rank;
        size_t n = 4;
        for (int i = 0; i < c_rank; ++i) { nd.cdim[i] = cdim[i]; n *= size_t(cdim[i]); }
        nd.c = add_param(m, c, n);
    }
    nd.alpha = alpha; nd.beta = beta; nd.trans_a = trans_a; nd.trans_b = trans_b;
    return append(m, nd, ZANT_F32, ydim, 4, 1.0f, 0);
}

extern "C" int zant_model_matmul(zant_model *m, int a, const float *b, const int64_t *bdim, int b_rank) {
    if (!valid_tensor(m, a) || !b || !bdim) return ZANT_NullPointer;
    const MTensor ta = m->t[a];
    if (ta.dtype != ZANT_F32 || b_rank > 8) return ZANT_InvalidInput;
    int rc = zant_hip_matmul_check(ta.dim, ta.rank, bdim, b_rank);
    if (rc) return rc;
    MNode nd;
    nd.op = OP_MATMUL; nd.in0 = a; nd.b_rank = b_rank;
    size_t n = 4;
    for (int i = 0; i < b_rank; ++i) { nd.bdim[i] = bdim[i]; n *= size_t(bdim[i]); }
    nd.w = add_param(m, b, n);
    int64_t ydim[8];
    for (int i = 0; i < ta.rank; ++i) ydim[i] = ta.dim[i];
    ydim[ta.rank - 1] = bdim[b_rank - 1];
    return append(m, nd, ZANT_F32, ydim, ta.rank, 1.0f, 0);
}

extern "C" int zant_model_add_const(zant_model *m, int x, const float *c, const int64_t *cdim, int c_rank) {
    if (!valid_tensor(m, x) || !c || !cdim) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_F32 || c_rank > 4 || c_rank < 1) return ZANT_InvalidInput;
    int64_t ydim[8];
    int yr = 0;
    int rc = zant_hip_add_f32(m->ctx, nullptr, tx.dim, tx.rank, nullptr, cdim, c_rank, nullptr, ydim, &yr);
    if (rc != ZANT_OK && rc != ZANT_NullPointer) return rc;  // shapes are validated before pointers are looked at
    MNode nd;
    nd.op = OP_ADD_CONST; nd.in0 = x; nd.c_rank = c_rank;
    size_t n = 4;
    for (int i = 0; i < c_rank; ++i) { nd.cdim[i] = cdim[i]; n *= size_t(cdim[i]); }
    nd.c = add_param(m, c, n);
    return append(m, nd, ZANT_F32, ydim, yr, 1.0f, 0);
}

extern "C" int zant_model_add(zant_model *m, int a, int b) {
    if (!valid_tensor(m, a) || !valid_tensor(m, b)) return ZANT_NullPointer;
    const MTensor ta = m->t[a], tb = m->t[b];
    if (ta.dtype != ZANT_F32 || tb.dtype != ZANT_F32) return ZANT_InvalidInput;
    int64_t ydim[8];
    int yr = 0;
    int rc = zant_hip_add_f32(m->ctx, nullptr, ta.dim, ta.rank, nullptr, tb.dim, tb.rank, nullptr, ydim, &yr);
    if (rc != ZANT_OK && rc != ZANT_NullPointer) return rc;
    MNode nd;
    nd.op = OP_ADD; nd.in0 = a; nd.in1 = b;
    return append(m, nd, ZANT_F32, ydim, yr, 1.0f, 0);
}

extern "C" int zant_model_softmax(zant_model *m, int x) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_F32 || tx.rank < 2) return ZANT_InvalidInput;
    MNode nd;
    nd.op = OP_SOFTMAX; nd.in0 = x;
    return append(m, nd, ZANT_F32, tx.dim, tx.rank, 1.0f, 0);
}

extern "C" int zant_model_sigmoid(zant_model *m, int x) { return unary_same_shape(m, x, OP_SIGMOID, 0.0f); }

extern "C" int zant_model_reduce_mean(zant_model *m, int x, const int64_t *axes, int n_axes, int keepdims) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_F32) return ZANT_InvalidInput;
    int64_t ydim[8];
    int yr = 0;
    const int rc = zant_hip_reduce_mean_f32(nullptr, nullptr, tx.dim, tx.rank, axes, n_axes, keepdims, 0, nullptr, ydim, &yr);
    if (rc != ZANT_OK) return rc;
    MNode nd;
    nd.op = OP_REDUCE_MEAN; nd.in0 = x; nd.keepdims = keepdims;
    if (axes) nd.axes.assign(axes, axes + n_axes);
    return append(m, nd, ZANT_F32, ydim, yr, 1.0f, 0);
}

extern "C" int zant_model_concat(zant_model *m, const int *xs, int n, int64_t axis) {
    if (!m || !xs) return ZANT_NullPointer;
    if (n <= 0) return ZANT_EmptyTensorList;
    if (n > 16) return ZANT_InvalidDimensions;
    const int64_t *dd[16];
    int rr[16];
    for (int i = 0; i < n; ++i) {
        if (!valid_tensor(m, xs[i])) return ZANT_NullPointer;
        const MTensor &t = m->t[xs[i]], &t0 = m->t[xs[0]];
        // quantised inputs must already share their parameters: concatenation moves codes, it does not requantise
        if (t.dtype != t0.dtype || (t.dtype == ZANT_U8 && (t.scale != t0.scale || t.zp != t0.zp))) return ZANT_InvalidInput;
        dd[i] = t.dim; rr[i] = t.rank;
    }
    int64_t ydim[8];
    int yr = 0;
    const int rc = zant_hip_concatenate(nullptr, nullptr, dd, rr, n, axis, 1, nullptr, ydim, &yr);
    if (rc != ZANT_OK) return rc;
    const MTensor t0 = m->t[xs[0]];
    MNode nd;
    nd.op = OP_CONCAT; nd.in0 = xs[0]; nd.in1 = n > 1 ? xs[1] : -1; nd.axis = axis;
    for (int i = 2; i < n; ++i) nd.more.push_back(xs[i]);
    return append(m, nd, t0.dtype, ydim, yr, t0.scale, t0.zp);
}

extern "C" int zant_model_resize_nearest(zant_model *m, int x, const float *scales, const int64_t *sizes, int n_param,
                                         int coord_mode) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    int64_t ydim[8];
    const int rc = zant_hip_resize_nearest(nullptr, nullptr, tx.dim, tx.rank, 1, scales, sizes, n_param, coord_mode, nullptr, ydim);
    if (rc != ZANT_OK) return rc;
    MNode nd;
    nd.op = OP_RESIZE; nd.in0 = x; nd.coord_mode = coord_mode;
    if (scales) nd.scales.assign(scales, scales + n_param);
    else nd.axes.assign(sizes, sizes + n_param);
    return append(m, nd, tx.dtype, ydim, tx.rank, tx.scale, tx.zp);
}

extern "C" int zant_model_quantize(zant_model *m, int x, float y_scale, int y_zp) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_F32 || y_zp < 0 || y_zp > 255) return ZANT_InvalidInput;
    MNode nd;
    nd.op = OP_QUANT; nd.in0 = x;
    const uint8_t zp8 = uint8_t(y_zp);
    nd.ws = add_param(m, &y_scale, 4);
    nd.b = add_param(m, &zp8, 1);
    return append(m, nd, ZANT_U8, tx.dim, tx.rank, y_scale, y_zp);
}

extern "C" int zant_model_dequantize(zant_model *m, int x) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_U8) return ZANT_InvalidInput;
    MNode nd;
    nd.op = OP_DEQUANT; nd.in0 = x;
    const uint8_t zp8 = uint8_t(tx.zp);
    nd.ws = add_param(m, &tx.scale, 4);
    nd.b = add_param(m, &zp8, 1);
    return append(m, nd, ZANT_F32, tx.dim, tx.rank, 1.0f, 0);
}

extern "C" int zant_model_qlinearconv(zant_model *m, int x, const int8_t *w, const int64_t wdim[4], const float *w_scale,
                                      int64_t n_wscale, const int32_t *bias, float y_scale, int y_zp,
                                      const int64_t stride[2], const int64_t pads[4], const int64_t dil[2], int64_t group) {
    if (!valid_tensor(m, x) || !w || !wdim || !w_scale || !stride || !pads || !dil) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_U8 || tx.rank != 4 || y_zp < 0 || y_zp > 255) return ZANT_InvalidInput;
    if (group < 1 || tx.dim[1] % group || wdim[0] % group || tx.dim[1] / group != wdim[1]) return ZANT_InvalidDimensions;
    if (n_wscale != 1 && n_wscale != wdim[0]) return ZANT_InputTensorDimensionMismatch;
    if (stride[0] <= 0 || stride[1] <= 0 || dil[0] <= 0 || dil[1] <= 0) return ZANT_WrongStride;
    const int64_t dkh = (wdim[2] - 1) * dil[0] + 1, dkw = (wdim[3] - 1) * dil[1] + 1;
    const int64_t PH = tx.dim[2] + pads[0] + pads[2], PW = tx.dim[3] + pads[1] + pads[3];
    if (PH < dkh || PW < dkw) return ZANT_InvalidDimensions;
    const int64_t ydim[4] = {tx.dim[0], wdim[0], (PH - dkh) / stride[0] + 1, (PW - dkw) / stride[1] + 1};
    MNode nd;
    nd.op = OP_QCONV; nd.in0 = x; nd.group = group; nd.n_wscale = n_wscale;
    for (int i = 0; i < 4; ++i) { nd.wdim[i] = wdim[i]; nd.pads[i] = pads[i]; }
    for (int i = 0; i < 2; ++i) { nd.stride[i] = stride[i]; nd.dil[i] = dil[i]; }
    nd.w = add_param(m, w, size_t(wdim[0] * wdim[1] * wdim[2] * wdim[3]));
    nd.ws = add_param(m, w_scale, size_t(n_wscale) * 4);
    if (bias) nd.b = add_param(m, bias, size_t(wdim[0]) * 4);
    return append(m, nd, ZANT_U8, ydim, 4, y_scale, y_zp);
}

extern "C" int zant_model_qlinear_act(zant_model *m, int x, int act, float alpha, float y_scale, int y_zp) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_U8 || act < ZANT_ACT_NONE || act > ZANT_ACT_RELU6 || y_zp < 0 || y_zp > 255) return ZANT_InvalidInput;
    MNode nd;
    nd.op = OP_QACT; nd.in0 = x; nd.act = act; nd.act_alpha = alpha;
    return append(m, nd, ZANT_U8, tx.dim, tx.rank, y_scale, y_zp);
}

extern "C" int zant_model_qlinear_add(zant_model *m, int a, int b, float y_scale, int y_zp) {
    if (!valid_tensor(m, a) || !valid_tensor(m, b)) return ZANT_NullPointer;
    const MTensor ta = m->t[a], tb = m->t[b];
    if (ta.dtype != ZANT_U8 || tb.dtype != ZANT_U8 || y_zp < 0 || y_zp > 255) return ZANT_InvalidInput;
    if (ta.rank != tb.rank || ta.bytes() != tb.bytes()) return ZANT_InputTensorDifferentSize;
    MNode nd;
    nd.op = OP_QADD; nd.in0 = a; nd.in1 = b;
    return append(m, nd, ZANT_U8, ta.dim, ta.rank, y_scale, y_zp);
}

extern "C" int zant_model_qlinear_global_avgpool(zant_model *m, int x, float y_scale, int y_zp) {
    if (!valid_tensor(m, x)) return ZANT_NullPointer;
    const MTensor tx = m->t[x];
    if (tx.dtype != ZANT_U8 || tx.rank != 4 || y_zp < 0 || y_zp > 255) return ZANT_InvalidInput;
    const int64_t ydim[4] = {tx.dim[0], tx.dim[1], 1, 1};
    MNode nd;
    nd.op = OP_QGAP; nd.in0 = x;
    return append(m, nd, ZANT_U8, ydim, 4, y_scale, y_zp);
}

extern "C" int zant_model_finalize(zant_model *m) {
    if (!m) return ZANT_NullPointer;
    if (m->finalized) return ZANT_OK;
    if (!m->ctx) return ZANT_NullPointer;  // built without a context: a dry run
    if (m->input < 0 || m->n.empty()) return ZANT_InvalidInput;
    zant_ctx *ctx = m->ctx;
    const int nn = int(m->n.size());
    m->output = m->n.back().out;
    m->unfused_bytes = 0;  // what one static array per node output (the reference's layout) would take
    for (const MNode &nd : m->n) m->unfused_bytes += m->t[nd.out].bytes();

    // ---- peephole fusions -----------------------------------------------------------------------
    for (int i = 0; i < nn; ++i) {
        MNode &nd = m->n[i];
        if (nd.skip) continue;
        int only = -1;
        if (nd.op == OP_RESHAPE) {  // a view of its input
            m->t[nd.out].alias_of = nd.in0;
            nd.skip = true;
            continue;
        }
        if (nd.op == OP_CONV && nd.b < 0 && consumers(m, nd.out, &only) == 1 && m->n[only].op == OP_ADD_CONST &&
            m->n[only].in0 == nd.out) {
            // Conv -> Add(constant of one value per output channel): that constant is the bias
            MNode &ad = m->n[only];
            int64_t cnt = 1;
            for (int k = 0; k < ad.c_rank; ++k) cnt *= ad.cdim[k];
            const bool per_channel = cnt == nd.wdim[0] &&
                                     ((ad.c_rank == 3 && ad.cdim[0] == nd.wdim[0]) || (ad.c_rank == 4 && ad.cdim[1] == nd.wdim[0]) ||
                                      // {M} broadcasts against the LAST axis: a per-channel bias only for a [1, M, 1, 1]
                                      // result, where the Add is an equal-size flat add and keeps the shape
                                      (ad.c_rank == 1 && m->t[nd.out].dim[3] == 1 && m->t[nd.out].dim[2] == 1 &&
                                       m->t[nd.out].dim[0] == 1 && m->t[ad.out].rank == m->t[nd.out].rank &&
                                       m->t[ad.out].bytes() == m->t[nd.out].bytes()));
            if (per_channel) {
                nd.b = ad.c;
                m->t[ad.out].alias_of = nd.out;
                ad.skip = true;
            }
        }
        if (nd.op == OP_CONV) {
            // Conv (-> folded Add) -> BatchNormalization that nothing else reads the input of: the normalisation is a
            // per-channel scale and shift, folded into the weights and the bias on the host:
            //   w'[k] = w[k] * s[k],  b'[k] = (b[k] - mean[k]) * s[k] + beta[k],  s[k] = gamma[k] / sqrt(var[k] + eps)
            int out = nd.out, c1 = -1;
            while (consumers(m, out, &c1) == 1 && m->n[c1].skip && m->n[c1].op == OP_ADD_CONST) out = m->n[c1].out;
            if (consumers(m, out, &only) == 1 && m->n[only].op == OP_BATCHNORM && !m->n[only].skip && m->n[only].in0 == out &&
                m->t[out].rank == 4 && out != m->output) {
                MNode &bn = m->n[only];
                const int64_t K = nd.wdim[0], per_k = nd.wdim[1] * nd.wdim[2] * nd.wdim[3];
                float *w = reinterpret_cast<float *>(m->p[nd.w].host.data());
                const float *ga = reinterpret_cast<const float *>(m->p[bn.w].host.data());
                const float *be = reinterpret_cast<const float *>(m->p[bn.b].host.data());
                const float *mu = reinterpret_cast<const float *>(m->p[bn.c].host.data());
                const float *va = reinterpret_cast<const float *>(m->p[bn.ws].host.data());
                // The fold replaces the reference's order of operations ((x - mean) / sqrt(var + eps) * gamma + beta,
                // batchNormLayer.zig:143-145) by one scale folded into the weights: the two differ by rounding errors that
                // grow with |s|, and a non-finite s (var + eps <= 0, overflow) would poison every weight of the channel
                // where the operator itself yields NaN / inf only where the reference does.  So the fold is taken only when
                // every channel's scale is finite and moderate; otherwise the normalisation stays a node of its own.
                std::vector<float> scale(static_cast<size_t>(K));
                bool foldable = true;
                for (int64_t k = 0; k < K; ++k) {
                    const float sc = ga[k] / sqrtf(va[k] + bn.alpha);
                    scale[size_t(k)] = sc;
                    if (!std::isfinite(sc) || fabsf(sc) > 1024.0f || (sc != 0.0f && fabsf(sc) < 1.0f / 1024.0f)) foldable = false;
                }
                if (foldable) {
                    std::vector<float> bias(size_t(K), 0.0f);
                    if (nd.b >= 0) memcpy(bias.data(), m->p[nd.b].host.data(), size_t(K) * 4);
                    for (int64_t k = 0; k < K; ++k) {
                        const float sc = scale[size_t(k)];
                        for (int64_t e = 0; e < per_k; ++e) w[k * per_k + e] *= sc;
                        bias[size_t(k)] = (bias[size_t(k)] - mu[k]) * sc + be[k];
                    }
                    nd.b = add_param(m, bias.data(), size_t(K) * 4);  // (a bias shared with another node keeps its own copy)
                    m->t[bn.out].alias_of = out;
                    bn.skip = true;
                }
            }
        }
        if ((nd.op == OP_CONV || nd.op == OP_GEMM) && nd.fuse_act == ZANT_ACT_NONE) {
            int out = nd.out;
            // look through an Add that was just folded
            int c1 = -1;
            // ... or a normalisation, and through Reshape views (ReLU is elementwise: the view's shape does not matter)
            while (consumers(m, out, &c1) == 1 &&
                   ((m->n[c1].skip && (m->n[c1].op == OP_ADD_CONST || m->n[c1].op == OP_BATCHNORM)) || m->n[c1].op == OP_RESHAPE))
                out = m->n[c1].out;
            if (consumers(m, out, &only) == 1 && m->n[only].op == OP_RELU && !m->n[only].skip) {
                nd.fuse_act = ZANT_ACT_RELU;
                m->t[m->n[only].out].alias_of = out;
                m->n[only].skip = true;
            }
        }
        if (nd.op == OP_GEMM && nd.fuse_act == ZANT_ACT_NONE && !nd.trans_a) {
            // Gemm -> (Reshape views) -> Softmax over the same [rows, cols]: the classifier head in one kernel
            int out = nd.out, c1 = -1;
            while (consumers(m, out, &c1) == 1 && m->n[c1].op == OP_RESHAPE) out = m->n[c1].out;
            if (consumers(m, out, &only) == 1 && m->n[only].op == OP_SOFTMAX && !m->n[only].skip) {
                const MTensor &si = m->t[m->n[only].in0];
                const MTensor &go = m->t[nd.out];
                if (si.dim[0] == go.dim[2] && si.dim[1] == go.dim[3] && go.dim[3] <= 16) {
                    nd.fuse_act = ZANT_ACT_SOFTMAX;
                    m->t[m->n[only].out].alias_of = out;
                    m->n[only].skip = true;
                }
            }
        }
        if (nd.op == OP_CONV) {
            // Conv (+ReLU) -> MaxPool 2x2/2: one kernel, pooled output only (where the convolution kernels take the shape)
            int out = nd.out, c1 = -1;
            while (consumers(m, out, &c1) == 1 && m->n[c1].skip &&
                   (m->n[c1].op == OP_ADD_CONST || m->n[c1].op == OP_RELU || m->n[c1].op == OP_BATCHNORM))
                out = m->n[c1].out;
            if (consumers(m, out, &only) == 1 && m->n[only].op == OP_MAXPOOL && !m->n[only].skip) {
                MNode &pn = m->n[only];
                const bool pool22 = pn.kernel[0] == 2 && pn.kernel[1] == 2 && pn.stride[0] == 2 && pn.stride[1] == 2 &&
                                    pn.dil[0] == 1 && pn.dil[1] == 1 && pn.pads[0] == 0 && pn.pads[1] == 0 && pn.pads[2] == 0 &&
                                    pn.pads[3] == 0 && (pn.pool_pad == ZANT_PAD_NOTSET || pn.pool_pad == ZANT_PAD_VALID);
                const MTensor &tp = m->t[pn.out];
                if (pool22 && m->t[nd.in0].dtype == ZANT_F32 &&
                    zant_conv2d_f32_fused_pool(ctx, nullptr, m->t[nd.in0].dim, nullptr, nd.wdim, nullptr, nullptr, tp.dim, nd.stride,
                                               nd.n_stride, nd.has_pads ? nd.pads : nullptr, nd.n_pads,
                                               nd.has_dil ? nd.dil : nullptr, nd.n_dil, nd.group,
                                               nd.has_auto_pad ? nd.auto_pad.c_str() : nullptr, 0, true) == ZANT_OK) {
                    // the conv node now produces the pool's tensor; the intermediate tensors are never materialised
                    nd.fuse_pool = true;
                    const int conv_out = nd.out;
                    nd.out = pn.out;
                    pn.skip = true;
                    pn.out = conv_out;  // keeps every tensor id owned by exactly one node
                    pn.in0 = conv_out;
                }
            }
        }
        if (nd.op == OP_QCONV && nd.fuse_act == ZANT_ACT_NONE && consumers(m, nd.out, &only) == 1 &&
            m->n[only].op == OP_QACT && !m->n[only].skip && m->n[only].act != ZANT_ACT_NONE) {
            // (a plain requantisation node, act == none, stays a node of its own: fused, the kernel would take the
            // activation's parameters for its first stage and skip the rounding and saturation of the intermediate u8)
            // the activation's output parameters become the kernel's second requantisation stage
            const MNode &an = m->n[only];
            const MTensor &ao = m->t[an.out];
            nd.fuse_act = an.act;
            nd.act_alpha = an.act_alpha;
            // run_node passes (conv y_scale/zp) = this node's out tensor, (act scale/zp) = the activation's out tensor
            nd.act_scale = m->t[nd.out].scale;
            nd.act_zp = m->t[nd.out].zp;
            m->t[nd.out].scale = ao.scale;  // the stored tensor now holds the activation's result
            m->t[nd.out].zp = ao.zp;
            m->t[an.out].alias_of = nd.out;
            m->n[only].skip = true;
        }
    }
    (void)producer;

    // ---- first int8 layer: QLinearConv (+activation) -> MaxPool 2x2/2 in the few-channel kernel -------------------
    for (int i = 0; i < nn; ++i) {
        MNode &nd = m->n[i];
        int only = -1;
        if (nd.skip || nd.op != OP_QCONV || consumers(m, nd.out, &only) != 1) continue;
        // (a fused activation's tensor is an alias of nd.out, so its consumers count as consumers of nd.out's storage;
        //  look for the pool among the readers of either id)
        int out = nd.out, c1 = -1;
        while (consumers(m, out, &c1) == 1 && m->n[c1].skip && m->n[c1].op == OP_QACT) out = m->n[c1].out;
        if (consumers(m, out, &only) != 1 || m->n[only].op != OP_MAXPOOL || m->n[only].skip) continue;
        MNode &pn = m->n[only];
        const bool pool22 = pn.kernel[0] == 2 && pn.kernel[1] == 2 && pn.stride[0] == 2 && pn.stride[1] == 2 &&
                            pn.dil[0] == 1 && pn.dil[1] == 1 && pn.pads[0] == 0 && pn.pads[1] == 0 && pn.pads[2] == 0 &&
                            pn.pads[3] == 0 && (pn.pool_pad == ZANT_PAD_NOTSET || pn.pool_pad == ZANT_PAD_VALID);
        const MTensor &ti = m->t[nd.in0];
        const MTensor &tp = m->t[pn.out];
        if (!pool22 || root_of(m, nd.in0) != root_of(m, m->input)) continue;
        if (zant_qlinearconv_layout_pool(ctx, nullptr, ti.dim, ti.scale, uint8_t(ti.zp), nullptr, nd.wdim, nullptr, nd.n_wscale,
                                         nullptr, 1.0f, 0, nullptr, nullptr, tp.dim, nd.stride, nd.pads, nd.dil, nd.group,
                                         nd.fuse_act, 0.0f, 1.0f, 0, ZANT_LAYOUT_NCHW, ZANT_LAYOUT_NCHW, 1, true, nullptr) != ZANT_OK)
            continue;
        // the pool's tensor carries the same scale / zero point as the tensor it pooled
        m->t[pn.out].scale = m->t[nd.out].scale;
        m->t[pn.out].zp = m->t[nd.out].zp;
        nd.fuse_pool = true;
        const int conv_out = nd.out;
        nd.out = pn.out;
        pn.skip = true;
        pn.out = conv_out;
        pn.in0 = conv_out;
    }

    // ---- layouts: int8 activations stay channel-blocked between the operators that have blocked kernels ----------
    {
        const int ntl = int(m->t.size());
        auto blocked_op = [&](const MNode &nd) {
            return nd.op == OP_QCONV || nd.op == OP_QACT || nd.op == OP_QADD || nd.op == OP_QGAP ||
                   (nd.op == OP_MAXPOOL && m->t[nd.in0].dtype == ZANT_U8);
        };
        for (const MNode &nd : m->n) {
            if (nd.skip || !blocked_op(nd)) continue;
            MTensor &ro = m->t[root_of(m, nd.out)];
            if (ro.dtype == ZANT_U8 && ro.rank == 4) ro.layout = ZANT_LAYOUT_BLOCKED16;
        }
        auto demote = [&](int id, bool &changed) {
            MTensor &r = m->t[root_of(m, id)];
            if (r.layout != ZANT_LAYOUT_NCHW) { r.layout = ZANT_LAYOUT_NCHW; changed = true; }
        };
        bool changed = true;
        while (changed) {
            changed = false;
            demote(m->input, changed);
            demote(m->output, changed);
            for (const MNode &nd : m->n) {
                if (nd.op == OP_RESHAPE) { demote(nd.in0, changed); demote(nd.out, changed); continue; }  // views need NCHW
                if (nd.skip) continue;
                const int li = m->t[root_of(m, nd.in0)].layout, lo = m->t[root_of(m, nd.out)].layout;
                if (!blocked_op(nd)) {
                    demote(nd.in0, changed);
                    if (nd.in1 >= 0) demote(nd.in1, changed);
                    for (int in : nd.more) demote(in, changed);
                    demote(nd.out, changed);
                    continue;
                }
                if (nd.op == OP_QCONV) {
                    if (nd.fuse_pool) demote(nd.in0, changed);
                } else if (nd.op == OP_QGAP) {
                    if (li == ZANT_LAYOUT_NCHW) demote(nd.out, changed);
                } else if (nd.op == OP_QADD) {
                    const int l1 = m->t[root_of(m, nd.in1)].layout;
                    if (li == ZANT_LAYOUT_NCHW || l1 == ZANT_LAYOUT_NCHW || lo == ZANT_LAYOUT_NCHW) {
                        demote(nd.in0, changed); demote(nd.in1, changed); demote(nd.out, changed);
                    }
                } else if (nd.op == OP_MAXPOOL) {
                    const bool pool22 = nd.kernel[0] == 2 && nd.kernel[1] == 2 && nd.stride[0] == 2 && nd.stride[1] == 2 &&
                                        nd.dil[0] == 1 && nd.dil[1] == 1 && nd.pads[0] == 0 && nd.pads[1] == 0 &&
                                        nd.pads[2] == 0 && nd.pads[3] == 0 &&
                                        (nd.pool_pad == ZANT_PAD_NOTSET || nd.pool_pad == ZANT_PAD_VALID) &&
                                        m->t[nd.out].dim[2] == m->t[nd.in0].dim[2] / 2 &&
                                        m->t[nd.out].dim[3] == m->t[nd.in0].dim[3] / 2;
                    if (!pool22 || li == ZANT_LAYOUT_NCHW || lo == ZANT_LAYOUT_NCHW) { demote(nd.in0, changed); demote(nd.out, changed); }
                } else {  // OP_QACT: elementwise, same layout on both sides
                    if (li == ZANT_LAYOUT_NCHW || lo == ZANT_LAYOUT_NCHW) { demote(nd.in0, changed); demote(nd.out, changed); }
                }
            }
        }
        (void)ntl;
    }

    // ---- layouts: an f32 activation between convolution nodes stays quad-blocked ([N][C/4][H][W][4]) where the kernel
    // that writes it and every kernel that reads it take that layout: 16-byte stores on one side, a quarter of the
    // patch copies on the other.  Same bytes as NCHW, so the arena plan does not change. ----
    {
        auto caps = [&](const MNode &nd, int *in_ok, int *out_ok) {
            zant_conv2d_f32_c4_caps(m->t[nd.in0].dim, nd.wdim, m->t[nd.out].dim, nd.stride, nd.n_stride,
                                    nd.has_pads ? nd.pads : nullptr, nd.n_pads, nd.has_dil ? nd.dil : nullptr, nd.n_dil, nd.group,
                                    nd.has_auto_pad ? nd.auto_pad.c_str() : nullptr, nd.fuse_pool, in_ok, out_ok);
        };
        const int in_root = root_of(m, m->input), out_root = root_of(m, m->output);
        for (const MNode &nd : m->n) {
            if (nd.skip || nd.op != OP_CONV) continue;
            const int root = root_of(m, nd.out);
            MTensor &ro = m->t[root];
            if (ro.dtype != ZANT_F32 || ro.rank != 4 || root == in_root || root == out_root || ro.layout != ZANT_LAYOUT_NCHW) continue;
            int in_ok = 0, out_ok = 0;
            caps(nd, &in_ok, &out_ok);
            if (!out_ok) continue;
            bool all = true;
            int readers = 0;
            for (const MNode &c : m->n) {
                if (c.skip && c.op != OP_RESHAPE) continue;  // fused away; a view, though, would need NCHW
                bool reads = root_of(m, c.in0) == root || (c.in1 >= 0 && root_of(m, c.in1) == root);
                for (int in : c.more) reads = reads || root_of(m, in) == root;
                if (!reads) continue;
                ++readers;
                if (c.skip || c.op != OP_CONV || root_of(m, c.in0) != root) { all = false; break; }
                int cin = 0, cout = 0;
                caps(c, &cin, &cout);
                if (!cin) { all = false; break; }
            }
            if (all && readers > 0) ro.layout = ZANT_LAYOUT_C4;
        }
    }

    // ---- QLinearConv (+activation) -> MaxPool 2x2/2 between blocked tensors: the pool rides in the matrix-core kernel ----
    for (int i = 0; i < nn; ++i) {
        MNode &nd = m->n[i];
        if (nd.skip || nd.op != OP_QCONV || nd.fuse_pool) continue;
        int out = nd.out, c1 = -1, only = -1;
        while (consumers(m, out, &c1) == 1 && m->n[c1].skip && m->n[c1].op == OP_QACT) out = m->n[c1].out;
        if (consumers(m, out, &only) != 1 || m->n[only].op != OP_MAXPOOL || m->n[only].skip) continue;
        MNode &pn = m->n[only];
        const bool pool22 = pn.kernel[0] == 2 && pn.kernel[1] == 2 && pn.stride[0] == 2 && pn.stride[1] == 2 &&
                            pn.dil[0] == 1 && pn.dil[1] == 1 && pn.pads[0] == 0 && pn.pads[1] == 0 && pn.pads[2] == 0 &&
                            pn.pads[3] == 0 && (pn.pool_pad == ZANT_PAD_NOTSET || pn.pool_pad == ZANT_PAD_VALID);
        const MTensor &ti = m->t[nd.in0];
        const MTensor &to = m->t[nd.out];
        const MTensor &tp = m->t[pn.out];
        if (!pool22 || m->t[root_of(m, nd.in0)].layout != ZANT_LAYOUT_BLOCKED16 ||
            m->t[root_of(m, pn.out)].layout != ZANT_LAYOUT_BLOCKED16)
            continue;
        if (zant_qlinearconv_layout_pool(ctx, nullptr, ti.dim, ti.scale, uint8_t(ti.zp), nullptr, nd.wdim, nullptr, nd.n_wscale,
                                         nullptr, nd.fuse_act ? nd.act_scale : to.scale, uint8_t(nd.fuse_act ? nd.act_zp : to.zp),
                                         nullptr, nullptr, tp.dim, nd.stride, nd.pads, nd.dil, nd.group, nd.fuse_act, nd.act_alpha,
                                         to.scale, uint8_t(to.zp), ZANT_LAYOUT_BLOCKED16, ZANT_LAYOUT_BLOCKED16, 1, true,
                                         nullptr) != ZANT_OK)
            continue;
        m->t[pn.out].scale = m->t[nd.out].scale;
        m->t[pn.out].zp = m->t[nd.out].zp;
        nd.fuse_pool = true;
        const int conv_out = nd.out;
        nd.out = pn.out;
        pn.skip = true;
        pn.out = conv_out;
        pn.in0 = conv_out;
    }

    // ---- inverted residual blocks: 1x1 expansion -> depthwise 3x3 -> 1x1 projection (-> Add with the block input) in one
    // kernel; the expanded tensors are never materialised -------------------------------------------------------------
    {
        auto is_1x1 = [](const MNode &c) {
            return c.op == OP_QCONV && !c.skip && !c.fuse_pool && c.group == 1 && c.wdim[2] == 1 && c.wdim[3] == 1 &&
                   c.stride[0] == 1 && c.stride[1] == 1 && c.pads[0] == 0 && c.pads[1] == 0 && c.pads[2] == 0 && c.pads[3] == 0;
        };
        // the single live reader of a tensor, looking through the activation nodes already folded into their producers
        auto next_reader = [&](int tensor) {
            int only = -1;
            while (consumers(m, tensor, &only) == 1 && m->n[only].skip && m->n[only].op == OP_QACT) tensor = m->n[only].out;
            return consumers(m, tensor, &only) == 1 && !m->n[only].skip ? only : -1;
        };
        for (int i = 0; i < nn; ++i) {
            MNode &ex = m->n[i];
            if (!is_1x1(ex) || m->t[root_of(m, ex.in0)].layout != ZANT_LAYOUT_BLOCKED16) continue;
            const int id = next_reader(ex.out);
            if (id < 0) continue;
            MNode &dw = m->n[id];
            if (dw.op != OP_QCONV || dw.fuse_pool || dw.group != dw.wdim[0] || dw.wdim[1] != 1 || dw.wdim[2] != 3 ||
                dw.wdim[3] != 3 || dw.group != ex.wdim[0] || dw.stride[0] != dw.stride[1] || dw.stride[0] < 1 ||
                dw.stride[0] > 2 || dw.dil[0] != 1 || dw.dil[1] != 1 || dw.pads[0] != 1 || dw.pads[1] != 1 || dw.pads[2] != 1 ||
                dw.pads[3] != 1)
                continue;
            const int ip = next_reader(dw.out);
            if (ip < 0 || !is_1x1(m->n[ip]) || m->n[ip].fuse_act != ZANT_ACT_NONE) continue;
            MNode &pj = m->n[ip];
            int ia = next_reader(pj.out);
            if (ia >= 0) {
                const MNode &ad = m->n[ia];
                const int other = ad.in0 == pj.out ? ad.in1 : ad.in0;
                if (ad.op != OP_QADD || other < 0 || root_of(m, other) != root_of(m, ex.in0)) ia = -1;
            }
            const int last = ia >= 0 ? ia : ip;
            if (m->t[root_of(m, m->n[last].out)].layout != ZANT_LAYOUT_BLOCKED16) continue;
            MNode blk;
            blk.op = OP_QBLOCK;
            blk.in0 = ex.in0;
            blk.out = m->n[last].out;
            blk.blk_expand = i; blk.blk_dw = id; blk.blk_project = ip; blk.blk_add = ia;
            zant_qconv_desc d[3];
            float add_scale = 1.0f;
            int add_zp = 0;
            fill_block_descs(m, blk, d, &add_scale, &add_zp);
            if (zant_qblock_blocked(ctx, nullptr, m->t[ex.in0].dim, &d[0], &d[1], dw.stride[0], &d[2], ia >= 0, add_scale, add_zp,
                                    nullptr, m->t[blk.out].dim, true, nullptr) != ZANT_OK)
                continue;
            // the block node takes the place of its last member (ready order); the members keep their tensor ids
            ex.skip = true; dw.skip = true; pj.skip = true;
            if (ia >= 0) m->n[ia].skip = true;
            MNode &slot_node = m->n[last];
            const MNode keep = slot_node;
            slot_node.op = OP_QBLOCK;
            slot_node.skip = false;
            slot_node.in0 = blk.in0; slot_node.in1 = -1;
            slot_node.blk_expand = i; slot_node.blk_dw = id; slot_node.blk_project = ip; slot_node.blk_add = ia;
            // the member's own fields move to a spare node appended at the end (skipped, never run)
            MNode spare = keep;
            spare.skip = true;
            spare.in0 = -1; spare.in1 = -1;  // no longer a reader of anything
            spare.slot = zant_pack_slot();
            m->n.push_back(spare);
            const int moved = int(m->n.size()) - 1;
            if (last == ip) m->n[last].blk_project = moved; else m->n[last].blk_add = moved;
        }
    }

    // ---- chains of inverted residual blocks: blocks that follow each other directly, each reading the one before's output,
    // become one launch where the kernel can keep a workgroup on the same images through all of them.  A chain stores
    // every block's output as before, but its workgroups are at different blocks at the same time: the tensors it reads
    // and writes are all planned as alive at the chain's launch, so none of them shares storage with another.
    {
        std::vector<int> live;
        for (int i = 0; i < nn; ++i)
            if (!m->n[i].skip) live.push_back(i);
        for (size_t k = 0; k < live.size();) {
            MNode &head = m->n[live[k]];
            size_t j = k + 1;
            if (head.op == OP_QBLOCK) {
                std::vector<int> rest;
                while (j < live.size()) {
                    const MNode &cand = m->n[live[j]], &prev = m->n[live[j - 1]];
                    if (cand.op != OP_QBLOCK || root_of(m, cand.in0) != root_of(m, prev.out)) break;
                    rest.push_back(live[j]);
                    if (run_block_chain(m, head, true, &rest) != ZANT_OK) { rest.pop_back(); break; }
                    ++j;
                }
                if (!rest.empty()) {
                    head.chain = rest;
                    for (int f : rest) m->n[f].chain_head = live[k];
                }
            }
            k = std::max(j, k + 1);
        }
    }

    // ---- liveness and first-fit arena planning --------------------------------------------------
    const int nt = int(m->t.size());
    for (int i = 0; i < nt; ++i) { m->t[i].def = -1; m->t[i].last = -1; }
    m->t[root_of(m, m->input)].def = 0;
    m->launches = 0;
    for (int i = 0; i < nn; ++i) {
        const MNode &nd = m->n[i];
        if (nd.skip) continue;  // fused away: its tensors are views of live ones or are never materialised
        if (nd.chain_head < 0) ++m->launches;
        const int when = (nd.chain_head >= 0 ? nd.chain_head : i) + 1;  // a chain's blocks all run at its first block's launch
        const int ro = root_of(m, nd.out);
        if (m->t[ro].def < 0) m->t[ro].def = when;
        m->t[ro].last = std::max(m->t[ro].last, when);
        for (int in : {nd.in0, nd.in1})
            if (in >= 0) { const int r = root_of(m, in); m->t[r].last = std::max(m->t[r].last, when); }
        for (int in : nd.more) { const int r = root_of(m, in); m->t[r].last = std::max(m->t[r].last, when); }
    }
    for (int i = 0; i < nn; ++i)
        if (m->n[i].chain_head >= 0) m->n[i].skip = true;  // from here on the chain's first block stands for them
    m->t[root_of(m, m->output)].last = nn + 1;  // the output outlives the pass
    // The input keeps its storage for the whole pass: a caller that uploads it once to zant_model_input_ptr() may run
    // the model any number of times (the reference's predict() copies its input on every call, predict.zig:339-366)
    m->t[root_of(m, m->input)].last = nn + 1;
    struct Placed { size_t off, size; int def, last; };
    std::vector<Placed> placed;
    size_t arena = 0;
    std::vector<int> order;
    for (int i = 0; i < nt; ++i)
        if (m->t[i].alias_of < 0 && m->t[i].def >= 0) order.push_back(i);
    std::sort(order.begin(), order.end(), [&](int a, int b) { return m->t[a].def < m->t[b].def; });
    for (int id : order) {
        MTensor &t = m->t[id];
        // the storage of a view chain must hold the largest member (they are all the same size here)
        const size_t size = (t.storage_bytes() + 255) & ~size_t(255);
        const int last = std::max(t.last, t.def);
        std::vector<std::pair<size_t, size_t>> busy;  // arena ranges alive during [def, last]
        for (const Placed &p : placed)
            if (!(p.last < t.def || p.def > last)) busy.emplace_back(p.off, p.off + p.size);
        std::sort(busy.begin(), busy.end());
        size_t off = 0;
        for (const auto &b : busy) {
            if (off + size <= b.first) break;
            off = std::max(off, b.second);
        }
        t.offset = off;
        placed.push_back({off, size, t.def, last});
        arena = std::max(arena, off + size);
    }
    m->arena_bytes = arena;
    int rc = zant_hip_arena_reserve(ctx, arena);
    if (rc) return rc;

    // ---- wide Gemm weights are kept k-contiguous ([N][K], i.e. transB): both operands of the matrix-core kernel are then
    // staged with 16-byte copies, half as many copy instructions per chunk as with a row-major B ---------------------
    for (MNode &nd : m->n) {
        if (nd.skip || nd.op != OP_GEMM || nd.trans_b || nd.wdim[0] != 1 || nd.wdim[1] != 1 || nd.wdim[3] <= 32) continue;
        const int64_t K = nd.wdim[2], N = nd.wdim[3];
        if (K % 4) continue;  // 16-byte copies need k-rows of a multiple of 4 floats
        std::vector<char> &h = m->p[nd.w].host;
        std::vector<char> tr(h.size());
        const float *src = reinterpret_cast<const float *>(h.data());
        float *dst = reinterpret_cast<float *>(tr.data());
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) dst[n * K + k] = src[k * N + n];
        h.swap(tr);
        nd.wdim[2] = N; nd.wdim[3] = K;
        nd.trans_b = 1;
    }

    // ---- parameters: one allocation, one upload each ---------------------------------------------
    size_t pbytes = 0;
    for (Param &p : m->p) { p.offset = pbytes; pbytes += (p.host.size() + 255) & ~size_t(255); }
    if (pbytes) {
        hipError_t e = hipMalloc(&m->params_dev, pbytes);
        if (e != hipSuccess) { zant_fail_hip(ctx, e, "hipMalloc(parameters)"); return ZANT_MemError; }
        for (Param &p : m->p) {
            rc = zant_hip_upload(ctx, static_cast<char *>(m->params_dev) + p.offset, p.host.data(), p.host.size());
            if (rc) return rc;
            std::vector<char>().swap(p.host);
        }
    }
    m->result_host.resize(m->t[m->output].bytes());
    // One pass over whatever the arena holds: every node packs its weights and sizes its scratch now, so that
    // zant_model_run allocates nothing and launches no packing kernels.
    ZANT_HIP_TRY(ctx, hipMemsetAsync(ctx->arena, 0, arena, ctx->stream));
    for (const MNode &nd : m->n) {
        if (nd.skip) continue;
        rc = run_node(m, nd);
        if (rc) return rc;
    }
    ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    m->finalized = true;
    return ZANT_OK;
}

extern "C" int zant_model_output_dims(zant_model *m, int64_t *dims, int *rank, int *dtype) {
    if (!m || !dims || !rank) return ZANT_NullPointer;
    if (m->n.empty()) return ZANT_InvalidInput;
    // before finalize the last node added; afterwards the recorded output (fusions may re-home a node's tensor)
    const MTensor &t = m->t[m->finalized ? m->output : m->n.back().out];
    *rank = t.rank;
    for (int i = 0; i < t.rank; ++i) dims[i] = t.dim[i];
    if (dtype) *dtype = t.dtype;
    return ZANT_OK;
}

extern "C" int zant_model_tensor_dims(zant_model *m, int tensor, int64_t *dims, int *rank, int *dtype) {
    if (!valid_tensor(m, tensor) || !dims || !rank) return ZANT_NullPointer;
    const MTensor &t = m->t[tensor];
    *rank = t.rank;
    for (int i = 0; i < t.rank; ++i) dims[i] = t.dim[i];
    if (dtype) *dtype = t.dtype;
    return ZANT_OK;
}

extern "C" size_t zant_model_arena_bytes(zant_model *m) { return m ? m->arena_bytes : 0; }
extern "C" size_t zant_model_unfused_bytes(zant_model *m) { return m ? m->unfused_bytes : 0; }
extern "C" int zant_model_num_launches(zant_model *m) { return m ? m->launches : 0; }

extern "C" void *zant_model_input_ptr(zant_model *m) { return (m && m->finalized) ? tensor_ptr(m, m->input) : nullptr; }
extern "C" void *zant_model_output_ptr(zant_model *m) { return (m && m->finalized) ? tensor_ptr(m, m->output) : nullptr; }

extern "C" int zant_model_run(zant_model *m, const void *input_dev, void *output_dev) {
    if (!m) return ZANT_NullPointer;
    if (!m->finalized) return ZANT_NotFinalized;
    zant_ctx *ctx = m->ctx;
    if (m->arena_bytes > ctx->arena_bytes) return ZANT_ArenaOverflow;  // another model shrank nothing, but be explicit
    const MTensor &tin = m->t[m->input];
    if (input_dev && input_dev != tensor_ptr(m, m->input))
        ZANT_HIP_TRY(ctx, hipMemcpyAsync(tensor_ptr(m, m->input), input_dev, tin.bytes(), hipMemcpyDeviceToDevice, ctx->stream));
    for (const MNode &nd : m->n) {
        if (nd.skip) continue;
        const int rc = run_node(m, nd);
        if (rc) return rc;
    }
    if (output_dev)
        ZANT_HIP_TRY(ctx, hipMemcpyAsync(output_dev, tensor_ptr(m, m->output), m->t[m->output].bytes(), hipMemcpyDeviceToDevice,
                                         ctx->stream));
    return ZANT_OK;
}

extern "C" int zant_model_predict_host(zant_model *m, const void *input_host, void *output_host) {
    if (!m || !input_host || !output_host) return ZANT_NullPointer;
    if (!m->finalized) return ZANT_NotFinalized;
    zant_ctx *ctx = m->ctx;
    int rc = zant_hip_upload(ctx, tensor_ptr(m, m->input), input_host, m->t[m->input].bytes());
    if (rc) return rc;
    for (const MNode &nd : m->n) {
        if (nd.skip) continue;
        rc = run_node(m, nd);
        if (rc) return rc;
    }
    return zant_hip_download(ctx, output_host, tensor_ptr(m, m->output), m->t[m->output].bytes());
}

namespace {

const char *op_name(const MNode &nd) {
    switch (nd.op) {
    case OP_CONV:
        if (nd.fuse_pool) return nd.fuse_act ? "Conv+Relu+MaxPool" : "Conv+MaxPool";
        return nd.fuse_act ? "Conv+Relu" : "Conv";
    case OP_RELU: return "Relu";
    case OP_LEAKY: return "LeakyRelu";
    case OP_MAXPOOL: return "MaxPool";
    case OP_RESHAPE: return "Reshape";
    case OP_GEMM: return nd.fuse_act == ZANT_ACT_SOFTMAX ? "Gemm+Softmax" : nd.fuse_act ? "Gemm+Relu" : "Gemm";
    case OP_MATMUL: return "MatMul";
    case OP_ADD_CONST: return "Add(const)";
    case OP_ADD: return "Add";
    case OP_SOFTMAX: return "Softmax";
    case OP_SIGMOID: return "Sigmoid";
    case OP_REDUCE_MEAN: return "ReduceMean";
    case OP_CONCAT: return "Concat";
    case OP_RESIZE: return "Resize";
    case OP_AVGPOOL: return "AveragePool";
    case OP_BATCHNORM: return "BatchNormalization";
    case OP_QUANT: return "QuantizeLinear";
    case OP_DEQUANT: return "DequantizeLinear";
    case OP_QCONV:
        if (nd.fuse_pool) return nd.fuse_act ? "QLinearConv+Act+MaxPool" : "QLinearConv+MaxPool";
        if (nd.group > 1) return nd.fuse_act ? "QLinearConv(depthwise)+Act" : "QLinearConv(depthwise)";
        return nd.fuse_act ? "QLinearConv+Act" : "QLinearConv";
    case OP_QACT: return "QLinearAct";
    case OP_QADD: return "QLinearAdd";
    case OP_QGAP: return "QLinearGlobalAveragePool";
    case OP_QBLOCK:
        if (!nd.chain.empty()) return "InvertedResidualChain";
        return nd.blk_add >= 0 ? "InvertedResidual(1x1+dw3x3+1x1+Add)" : "InvertedResidual(1x1+dw3x3+1x1)";
    default: return "?";
    }
}

void node_work(const zant_model *m, const MNode &nd, double *ops, double *bytes) {
    const MTensor &ti = m->t[nd.in0];
    const MTensor &to = m->t[nd.out];
    double b = double(ti.bytes()) + double(to.bytes());
    if (nd.in1 >= 0) b += double(m->t[nd.in1].bytes());
    for (int in : nd.more) b += double(m->t[in].bytes());
    double o = 0.0;
    switch (nd.op) {
    case OP_CONV:
    case OP_QCONV: {
        // ops count the convolution's own output (before any fused pooling)
        double outs = double(to.bytes()) / (nd.op == OP_CONV ? 4.0 : 1.0);
        if (nd.fuse_pool) outs *= 4.0;
        o = 2.0 * outs * double(nd.wdim[1] * nd.wdim[2] * nd.wdim[3]);
        b += double(nd.wdim[0] * nd.wdim[1] * nd.wdim[2] * nd.wdim[3]) * (nd.op == OP_CONV ? 4.0 : 1.0);
        break;
    }
    case OP_GEMM: {
        const double K = double(nd.trans_a ? ti.dim[2] : ti.dim[3]);
        o = 2.0 * double(to.dim[2]) * double(to.dim[3]) * K;
        b += double(nd.wdim[2] * nd.wdim[3]) * 4.0;
        break;
    }
    case OP_MATMUL: {
        const double K = double(ti.dim[ti.rank - 1]);
        o = 2.0 * double(to.dim[to.rank - 2]) * double(to.dim[to.rank - 1]) * K;
        b += double(nd.bdim[nd.b_rank - 2] * nd.bdim[nd.b_rank - 1]) * 4.0;
        break;
    }
    case OP_QBLOCK: {
        const MNode &ex = m->n[nd.blk_expand], &dw = m->n[nd.blk_dw], &pj = m->n[nd.blk_project];
        const double pos_in = double(ti.dim[0] * ti.dim[2] * ti.dim[3]), pos_out = double(to.dim[0] * to.dim[2] * to.dim[3]);
        o = 2.0 * (pos_in * double(ex.wdim[0] * ex.wdim[1]) + pos_out * double(dw.wdim[0]) * 9.0 +
                   pos_out * double(pj.wdim[0] * pj.wdim[1]));
        b += double(ex.wdim[0] * ex.wdim[1] + dw.wdim[0] * 9 + pj.wdim[0] * pj.wdim[1]);
        break;
    }
    default: break;
    }
    for (int f : nd.chain) {  // a chain's launch does the work of all its blocks
        double fo = 0, fb = 0;
        node_work(m, m->n[f], &fo, &fb);
        o += fo;
        b += fb;
    }
    *ops = o;
    *bytes = b;
}

}  // namespace

extern "C" int zant_model_profile(zant_model *m, float *ms, double *ops, double *bytes, int capacity) {
    if (!m || !ms) return ZANT_NullPointer;
    if (!m->finalized) return ZANT_NotFinalized;
    zant_ctx *ctx = m->ctx;
    const bool was = ctx->kernel_timing;
    ctx->kernel_timing = true;
    int cnt = 0, rc = ZANT_OK;
    for (const MNode &nd : m->n) {
        if (nd.skip) continue;
        rc = run_node(m, nd);
        if (rc) break;
        if (cnt < capacity) {
            rc = zant_hip_kernel_ms(ctx, &ms[cnt]);
            if (rc) break;
            if (cnt >= int(m->launch_kernels.size())) m->launch_kernels.resize(cnt + 1);
            m->launch_kernels[cnt] = ctx->last_kernel;
            double o = 0, b = 0;
            node_work(m, nd, &o, &b);
            if (ops) ops[cnt] = o;
            if (bytes) bytes[cnt] = b;
            ++cnt;
        }
    }
    ctx->kernel_timing = was;
    return rc ? rc : cnt;
}

extern "C" const char *zant_model_launch_name(zant_model *m, int i) {
    if (!m) return "";
    int cnt = 0;
    for (const MNode &nd : m->n) {
        if (nd.skip) continue;
        if (cnt++ == i) return op_name(nd);
    }
    return "";
}

extern "C" const char *zant_model_launch_kernel(zant_model *m, int i) {
    if (!m || i < 0 || i >= int(m->launch_kernels.size())) return "";
    return m->launch_kernels[i].c_str();
}

extern "C" int zant_model_read_tensor(zant_model *m, int id, void *dst_host, size_t bytes) {
    if (!valid_tensor(m, id) || !dst_host) return ZANT_NullPointer;
    if (!m->finalized) return ZANT_NotFinalized;
    if (bytes > m->t[id].bytes()) return ZANT_InvalidDimensions;
    if (m->t[root_of(m, id)].def < 0) return ZANT_InvalidInput;  // fused away: the tensor is never materialised
    const MTensor &t = m->t[id];
    // A later node may have been planned over this tensor's storage once its last reader was done, so the pass is
    // replayed up to the node that produces it (the input still sits in its slot: a pass never writes there), the tensor
    // is copied out, and the rest of the pass is replayed so that the arena -- the output at zant_model_output_ptr()
    // included -- again holds what the last zant_model_run left.
    // (chained blocks run one by one here: a chain may be planned over its own intermediate tensors)
    const int root = root_of(m, id);
    auto runs = [&](int i) { return !m->n[i].skip || m->n[i].chain_head >= 0; };
    struct Unchain {
        zant_model *m;
        explicit Unchain(zant_model *mm) : m(mm) { m->no_chain = true; }
        ~Unchain() { m->no_chain = false; }
    } unchain(m);
    int last_writer = -1;
    for (int i = 0; i < int(m->n.size()); ++i)
        if (runs(i) && root_of(m, m->n[i].out) == root) last_writer = i;
    for (int i = 0; i <= last_writer; ++i) {
        if (!runs(i)) continue;
        const int rc = run_node(m, m->n[i]);
        if (rc) return rc;
    }
    int rc;
    if (m->t[root].layout == ZANT_LAYOUT_BLOCKED16) {  // hand out NCHW u8 like everywhere outside the executor
        void *ws = nullptr;
        rc = zant_workspace(m->ctx, t.bytes(), &ws);
        if (rc) return rc;
        rc = zant_from_blocked(m->ctx, static_cast<const uint8_t *>(tensor_ptr(m, id)), t.dim[0], t.dim[1], t.dim[2] * t.dim[3],
                               static_cast<uint8_t *>(ws));
        if (rc) return rc;
        rc = zant_hip_download(m->ctx, dst_host, ws, bytes);
    } else if (m->t[root].layout == ZANT_LAYOUT_C4) {  // likewise NCHW f32
        void *ws = nullptr;
        rc = zant_workspace(m->ctx, t.bytes(), &ws);
        if (rc) return rc;
        rc = zant_from_c4_f32(m->ctx, static_cast<const float *>(tensor_ptr(m, id)), t.dim[0], t.dim[1], t.dim[2] * t.dim[3],
                              static_cast<float *>(ws));
        if (rc) return rc;
        rc = zant_hip_download(m->ctx, dst_host, ws, bytes);
    } else {
        rc = zant_hip_download(m->ctx, dst_host, tensor_ptr(m, id), bytes);
    }
    if (rc) return rc;
    for (int i = last_writer + 1; i < int(m->n.size()); ++i) {
        if (!runs(i)) continue;
        rc = run_node(m, m->n[i]);
        if (rc) return rc;
    }
    return ZANT_OK;
}

extern "C" int zant_model_bind_predict(zant_model *m) {
    if (m && !m->finalized) return ZANT_NotFinalized;
    g_predict_model = m;
    return ZANT_OK;
}

// predict's body; predict_batched calls it directly so that a generated library's own `predict` symbol, which comes
// first in a process that links both, is never reached from here.
static void predict_bound(float *input, uint32_t *input_shape, uint32_t shape_len, float **result) {
    zant_log("Starting prediction...\n");
    zant_model *m = g_predict_model;
    if (!m || !input || !input_shape || !result) return;
    const MTensor &tin = m->t[m->input];
    if (shape_len == 0) return;                      // src/codeGen/predict.zig:324
    if (shape_len != uint32_t(tin.rank)) return;     // :325
    for (int i = 0; i < tin.rank; ++i)
        if (int64_t(input_shape[i]) != tin.dim[i]) return;  // :329-334
    if (tin.dtype != ZANT_F32 || m->t[m->output].dtype != ZANT_F32) return;
    if (zant_model_predict_host(m, input, m->result_host.data()) != ZANT_OK) return;  // `catch return`: result untouched
    *result = reinterpret_cast<float *>(m->result_host.data());
    zant_log("Prediction completed.\n");
}

extern "C" void predict(float *input, uint32_t *input_shape, uint32_t shape_len, float **result) {
    predict_bound(input, input_shape, shape_len, result);
}

extern "C" void predict_batched(float *input, uint32_t n, float **result) {
    zant_model *m = g_predict_model;
    if (!m || !input || !result) return;
    const MTensor &tin = m->t[m->input];
    if (tin.rank < 1 || int64_t(n) != tin.dim[0]) return;
    uint32_t shape[8];
    for (int i = 0; i < tin.rank; ++i) shape[i] = uint32_t(tin.dim[i]);
    predict_bound(input, shape, uint32_t(tin.rank), result);
}
