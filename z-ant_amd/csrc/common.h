// Shared internals of libzant_hip.so: the context, status helpers and launch utilities.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "zant_hip.h"

struct zant_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    // activation arena: one allocation, bump/plan addressed by offset
    void *arena = nullptr;
    size_t arena_bytes = 0;
    // scratch for per-call packed weights / multiplier tables (grown on demand, never shrunk)
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    hipEvent_t ev_k0 = nullptr, ev_k1 = nullptr;  // bracket the last main kernel when kernel_timing is on
    bool kernel_timing = false;
    char last_kernel[96] = {0};  // device function of the last main kernel, template arguments included where the launch site knows them
    int num_cus = 256;
    std::string last_error;
};

extern void (*g_zant_log)(char *);
static inline void zant_log(const char *msg) {
    if (g_zant_log) g_zant_log(const_cast<char *>(msg));
}

// Records a failed HIP call on the context and yields ZANT_HipError.
int zant_fail_hip(zant_ctx *ctx, hipError_t e, const char *what);

#define ZANT_HIP_TRY(ctx, expr)                                      \
    do {                                                             \
        hipError_t _e = (expr);                                      \
        if (_e != hipSuccess) return zant_fail_hip((ctx), _e, #expr); \
    } while (0)

// Checks the launch that was just enqueued.
#define ZANT_LAUNCH_CHECK(ctx) ZANT_HIP_TRY(ctx, hipGetLastError())

// Opts `kernel` into `bytes` of dynamic LDS (more than 64 KB has to be asked for) on the context's device.  Done once per
// (kernel, device) under a lock; a failure is not cached, is recorded on the context and leaves the HIP runtime's last
// error set, so the launch site's ZANT_LAUNCH_CHECK reports it.  Returns false when the limit is not in place: the
// caller then does not launch.
bool zant_raise_lds_limit(zant_ctx *ctx, const void *kernel, int bytes);

// Names the main kernel a launch site is about to enqueue (what a profiler's kernel trace shows for it).
#define ZANT_KERNEL_NAME(ctx, ...) snprintf((ctx)->last_kernel, sizeof((ctx)->last_kernel), __VA_ARGS__)

// Brackets the main kernel of an operator with events when per-kernel timing is enabled.
struct KernelTimer {
    zant_ctx *ctx;
    explicit KernelTimer(zant_ctx *c) : ctx(c) {
        ctx->last_kernel[0] = 0;
        if (ctx->kernel_timing) (void)hipEventRecord(ctx->ev_k0, ctx->stream);
    }
    ~KernelTimer() {
        if (ctx->kernel_timing) (void)hipEventRecord(ctx->ev_k1, ctx->stream);
    }
};

// Grows the context's workspace to at least `bytes` (stream-ordered use only).
int zant_workspace(zant_ctx *ctx, size_t bytes, void **out);

// Weight-derived scratch of one operator instance (packed weights, requantisation tables, tile counters).  The model
// executor owns one per node, so packing happens once; calls through the C ABI pass none and pack on every call
// (the caller may have changed the weights).
struct zant_pack_slot {
    void *dev = nullptr;
    size_t bytes = 0;
    bool ready = false;   // the packed contents are valid
    unsigned runs = 0;    // launches so far; its parity selects the tile counter of a launch
    bool fixed = false;   // `dev` is memory the slot does not own and must not grow: a request beyond `bytes` fails
    // What the launcher that last used this slot derived from the call's geometry (tile shape, LDS layout, kernel
    // choice), and the geometry it derived it from: a model node or a prepared plan calls with the same geometry every
    // time, and the search for a tile shape costs the host 10-40 us, as much as a small layer takes on the GPU.
    std::vector<unsigned char> plan_key, plan_val;
};
// The cached plan of `slot` when it was made for the geometry `key` (byte-wise equal; fill keys over a zeroed struct).
template <class K, class V>
inline bool zant_plan_cached(const zant_pack_slot *slot, const K &key, V *val) {
    static_assert(std::is_trivially_copyable<K>::value && std::is_trivially_copyable<V>::value, "plain data only");
    if (!slot || slot->fixed || slot->plan_key.size() != sizeof(K) || slot->plan_val.size() != sizeof(V)) return false;
    if (std::memcmp(slot->plan_key.data(), &key, sizeof(K)) != 0) return false;
    std::memcpy(val, slot->plan_val.data(), sizeof(V));
    return true;
}
template <class K, class V>
inline void zant_plan_remember(zant_pack_slot *slot, const K &key, const V &val) {
    if (!slot || slot->fixed) return;
    slot->plan_key.assign(reinterpret_cast<const unsigned char *>(&key), reinterpret_cast<const unsigned char *>(&key) + sizeof(K));
    slot->plan_val.assign(reinterpret_cast<const unsigned char *>(&val), reinterpret_cast<const unsigned char *>(&val) + sizeof(V));
}
void zant_pack_slot_free(zant_ctx *ctx, zant_pack_slot *slot);
// Hands out `static_bytes` of weight-derived scratch (the slot's own allocation, or the front of the context
// workspace when slot == nullptr) and `dyn_bytes` of per-call scratch (always workspace).  *need_pack says whether
// the static part must be (re)filled; *parity which of the two tile counters this launch draws from.
int zant_pack_region(zant_ctx *ctx, zant_pack_slot *slot, size_t static_bytes, size_t dyn_bytes, void **stat, void **dyn,
                     bool *need_pack, int *parity);

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Streaming pattern of the HBM-bound elementwise kernels: a workgroup of 256 threads handles ZANT_STREAM_U x 256
// consecutive vectors, issuing all its loads before its stores, with nontemporal hints on both (measured on a
// 354 MB f32 stream: 6.7 TB/s against 5.0 TB/s for a grid-stride loop of plain 16-byte accesses).
constexpr int ZANT_STREAM_U = 4;
static inline unsigned zant_stream_grid(int64_t vectors) {
    const int64_t b = ceil_div64(vectors, int64_t(256) * ZANT_STREAM_U);
    return unsigned(b < 1 ? 1 : b);
}
#include "fastdiv.h"

static inline int64_t prod_dims(const int64_t *d, int rank) {
    int64_t p = 1;
    for (int i = 0; i < rank; ++i) p *= d[i];
    return p;
}

// Geometry every 2-D convolution kernel takes (already validated, int32 safe).
struct ConvGeom {
    int N, C, H, W;      // input
    int K, CG, KH, KW;   // filters, channels per group, kernel
    int OH, OW;
    int sh, sw, dh, dw;
    int pt, pl;          // pad top / left (bottom/right are implied by OH/OW)
    int groups;
};

// Resolves OnnxConvLean's stride / dilation defaults and pads; host only.
int zant_conv_resolve(const int64_t xdim[4], const int64_t wdim[4], const int64_t *stride, int n_stride,
                      const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                      const char *auto_pad, int64_t s[2], int64_t d[2], int64_t p[4]);

// Internal (not part of the C ABI): Conv (+ReLU) + MaxPool 2x2/2 fused into the convolution kernels.
// Returns ZANT_OK, a negative status, or 1 when the shape is not eligible.  query_only: just say whether it is.
int zant_conv2d_f32_fused_pool(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                               const float *bias, float *y, const int64_t ydim[4], const int64_t *stride, int n_stride,
                               const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                               const char *auto_pad, int relu, bool query_only, zant_pack_slot *slot = nullptr,
                               int x_c4 = 0, int y_c4 = 0);

// Which of a convolution node's tensors may be kept in the quad-blocked f32 layout ([N][C/4][H][W][4], quant_layout.h):
// *in_ok when the kernel that will run the node (with the fused pool or without) reads it, *out_ok when it writes it.
void zant_conv2d_f32_c4_caps(const int64_t xdim[4], const int64_t wdim[4], const int64_t ydim[4], const int64_t *stride,
                             int n_stride, const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group,
                             const char *auto_pad, bool fuse_pool, int *in_ok, int *out_ok);

// [N][C/4][HW][4] f32 -> NCHW f32 (for handing a quad-blocked tensor out of the executor).
int zant_from_c4_f32(zant_ctx *ctx, const float *x, int64_t N, int64_t C, int64_t HW, float *y);

// Resolves, once per device, the device address of the static scratch array behind zant_hip_conv2d_f32_static
// (conv_f32.hip).  Called by zant_hip_ctx_create with the context's device current; a failure is remembered and
// reported by the entry point.
void zant_conv_static_scratch_init(int device);

// zant_hip_conv2d_f32 with a pack slot (see above).
int zant_conv2d_f32_slot(zant_ctx *ctx, const float *x, const int64_t xdim[4], const float *w, const int64_t wdim[4],
                         const float *bias, float *y, const int64_t ydim[4], const int64_t *stride, int n_stride,
                         const int64_t *pads, int n_pads, const int64_t *dil, int n_dil, int64_t group, const char *auto_pad,
                         int fuse_act, zant_pack_slot *slot, int x_c4 = 0);
