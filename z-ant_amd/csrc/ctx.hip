// Context, arena, transfers, timing and status names of libzant_hip.so.
#include <map>
#include <mutex>
#include <utility>

#include "common.h"

void (*g_zant_log)(char *) = nullptr;

extern "C" void setLogFunctionC(void (*func)(char *)) { g_zant_log = func; }
extern "C" void setLogFunction(void (*func)(char *)) { g_zant_log = func; }

// Failures with no context to hold them (context creation itself) are kept per thread.
static thread_local std::string g_create_error;

static int create_failed(hipError_t e, const char *what) {
    g_create_error = std::string(what) + ": " + hipGetErrorString(e);
    zant_log(g_create_error.c_str());
    return ZANT_HipError;
}

int zant_fail_hip(zant_ctx *ctx, hipError_t e, const char *what) {
    if (ctx) {
        ctx->last_error = std::string(what) + ": " + hipGetErrorString(e);
        zant_log(ctx->last_error.c_str());
    }
    return ZANT_HipError;
}

bool zant_raise_lds_limit(zant_ctx *ctx, const void *kernel, int bytes) {
    static std::mutex lock;
    static std::map<std::pair<const void *, int>, int> raised;  // (kernel, device) -> bytes granted so far
    std::lock_guard<std::mutex> guard(lock);
    int &have = raised[{kernel, ctx->device}];
    if (have >= bytes) return true;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) {
        (void)zant_fail_hip(ctx, e, "hipFuncSetAttribute(MaxDynamicSharedMemorySize)");
        return false;
    }
    have = bytes;
    return true;
}

int zant_workspace(zant_ctx *ctx, size_t bytes, void **out) {
    if (bytes > ctx->workspace_bytes) {
        // The old buffer may still be read by queued kernels: drain before replacing it.
        ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
        if (ctx->workspace) ZANT_HIP_TRY(ctx, hipFree(ctx->workspace));
        ctx->workspace = nullptr;
        ctx->workspace_bytes = 0;
        size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes;
        ZANT_HIP_TRY(ctx, hipMalloc(&ctx->workspace, want));
        ctx->workspace_bytes = want;
    }
    *out = ctx->workspace;
    return ZANT_OK;
}

void zant_pack_slot_free(zant_ctx *ctx, zant_pack_slot *slot) {
    if (!slot || !slot->dev || slot->fixed) return;
    if (ctx && ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(slot->dev);
    slot->dev = nullptr; slot->bytes = 0; slot->ready = false; slot->runs = 0;
}

int zant_pack_region(zant_ctx *ctx, zant_pack_slot *slot, size_t static_bytes, size_t dyn_bytes, void **stat, void **dyn,
                     bool *need_pack, int *parity) {
    const size_t sa = (static_bytes + 255) & ~size_t(255);
    if (!slot) {
        void *ws = nullptr;
        const int rc = zant_workspace(ctx, sa + dyn_bytes, &ws);
        if (rc) return rc;
        *stat = ws;
        *dyn = static_cast<char *>(ws) + sa;
        *need_pack = true;
        *parity = 0;
        return ZANT_OK;
    }
    if (slot->fixed) {
        // borrowed memory of a fixed size: nothing is allocated, larger requests are refused
        if (!slot->dev) return ZANT_NullPointer;
        if (sa > slot->bytes || dyn_bytes) {
            ctx->last_error = "static scratch too small: " + std::to_string(sa + dyn_bytes) + " bytes needed, " +
                              std::to_string(slot->bytes) + " available";
            zant_log(ctx->last_error.c_str());
            return ZANT_ArenaOverflow;
        }
        *stat = slot->dev;
        *dyn = nullptr;
        *need_pack = true;  // the array is shared by every call on the device and the weights may have changed
        *parity = 0;
        return ZANT_OK;
    }
    if (!slot->dev || slot->bytes < sa) {
        zant_pack_slot_free(ctx, slot);
        ZANT_HIP_TRY(ctx, hipMalloc(&slot->dev, sa));
        slot->bytes = sa;
    }
    *dyn = nullptr;
    if (dyn_bytes) {
        const int rc = zant_workspace(ctx, dyn_bytes, dyn);
        if (rc) return rc;
    }
    *stat = slot->dev;
    *need_pack = !slot->ready;
    slot->ready = true;  // the caller packs in stream order before the first consumer
    *parity = int(slot->runs & 1u);
    ++slot->runs;
    return ZANT_OK;
}

extern "C" int zant_hip_ctx_create(zant_ctx **out, int device, void *stream) {
    if (!out) return ZANT_NullPointer;
    *out = nullptr;
    zant_ctx *ctx = new (std::nothrow) zant_ctx();
    if (!ctx) return ZANT_MemError;
    ctx->device = device;
    hipError_t e = hipSetDevice(device);
    if (e != hipSuccess) { delete ctx; return create_failed(e, "hipSetDevice"); }
    if (stream) {
        ctx->stream = static_cast<hipStream_t>(stream);
    } else {
        e = hipStreamCreate(&ctx->stream);  // default priority
        if (e != hipSuccess) { delete ctx; return create_failed(e, "hipStreamCreate"); }
        ctx->owns_stream = true;
    }
    zant_conv_static_scratch_init(device);
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->num_cus = prop.multiProcessorCount;
    hipEvent_t *evs[4] = {&ctx->ev_start, &ctx->ev_stop, &ctx->ev_k0, &ctx->ev_k1};
    for (hipEvent_t *ev : evs) {
        e = hipEventCreate(ev);
        if (e != hipSuccess) {
            zant_hip_ctx_destroy(ctx);
            return create_failed(e, "hipEventCreate");
        }
    }
    *out = ctx;
    return ZANT_OK;
}

extern "C" void zant_hip_ctx_destroy(zant_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->arena) (void)hipFree(ctx->arena);
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    if (ctx->ev_start) (void)hipEventDestroy(ctx->ev_start);
    if (ctx->ev_stop) (void)hipEventDestroy(ctx->ev_stop);
    if (ctx->ev_k0) (void)hipEventDestroy(ctx->ev_k0);
    if (ctx->ev_k1) (void)hipEventDestroy(ctx->ev_k1);
    if (ctx->owns_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

extern "C" int zant_hip_sync(zant_ctx *ctx) {
    if (!ctx) return ZANT_NullPointer;
    ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return ZANT_OK;
}

extern "C" const char *zant_hip_last_error(zant_ctx *ctx) { return ctx ? ctx->last_error.c_str() : g_create_error.c_str(); }
extern "C" const char *zant_hip_version(void) { return "zant-hip 0.1 (gfx950)"; }

extern "C" const char *zant_hip_status_name(int s) {
    switch (s) {
    case ZANT_OK: return "OK";
    case ZANT_InvalidDimensions: return "InvalidDimensions";
    case ZANT_InvalidPadding: return "InvalidPadding";
    case ZANT_InputTensorsWrongShape: return "InputTensorsWrongShape";
    case ZANT_InputTensorDifferentShape: return "InputTensorDifferentShape";
    case ZANT_InputTensorDimensionMismatch: return "InputTensorDimensionMismatch";
    case ZANT_IncompatibleBroadcastShapes: return "IncompatibleBroadcastShapes";
    case ZANT_InputTensorDifferentSize: return "InputTensorDifferentSize";
    case ZANT_EmptyTensor: return "EmptyTensor";
    case ZANT_ZeroSizeTensor: return "ZeroSizeTensor";
    case ZANT_InvalidInput: return "InvalidInput";
    case ZANT_InputArrayWrongSize: return "InputArrayWrongSize";
    case ZANT_WrongStride: return "WrongStride";
    case ZANT_MemError: return "MemError";
    case ZANT_InvalidAxes: return "InvalidAxes";
    case ZANT_AxisOutOfBounds: return "AxisOutOfBounds";
    case ZANT_MismatchedShape: return "MismatchedShape";
    case ZANT_MismatchedRank: return "MismatchedRank";
    case ZANT_EmptyTensorList: return "EmptyTensorList";
    case ZANT_UnsupportedMode: return "UnsupportedMode";
    case ZANT_HipError: return "HipError";
    case ZANT_NullPointer: return "NullPointer";
    case ZANT_ArenaOverflow: return "ArenaOverflow";
    case ZANT_NotFinalized: return "NotFinalized";
    default: return "Unknown";
    }
}

extern "C" int zant_hip_arena_reserve(zant_ctx *ctx, size_t bytes) {
    if (!ctx) return ZANT_NullPointer;
    if (bytes <= ctx->arena_bytes) return ZANT_OK;
    ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    if (ctx->arena) ZANT_HIP_TRY(ctx, hipFree(ctx->arena));
    ctx->arena = nullptr;
    ctx->arena_bytes = 0;
    hipError_t e = hipMalloc(&ctx->arena, bytes);
    if (e != hipSuccess) { zant_fail_hip(ctx, e, "hipMalloc(arena)"); return ZANT_MemError; }
    ctx->arena_bytes = bytes;
    return ZANT_OK;
}

extern "C" void *zant_hip_arena_ptr(zant_ctx *ctx, size_t offset) {
    if (!ctx || !ctx->arena || offset >= ctx->arena_bytes) return nullptr;
    return static_cast<char *>(ctx->arena) + offset;
}

extern "C" size_t zant_hip_arena_size(zant_ctx *ctx) { return ctx ? ctx->arena_bytes : 0; }

extern "C" int zant_hip_malloc(zant_ctx *ctx, void **dev_ptr, size_t bytes) {
    if (!ctx || !dev_ptr) return ZANT_NullPointer;
    hipError_t e = hipMalloc(dev_ptr, bytes ? bytes : 1);
    if (e != hipSuccess) { zant_fail_hip(ctx, e, "hipMalloc"); return ZANT_MemError; }
    return ZANT_OK;
}

extern "C" int zant_hip_free(zant_ctx *ctx, void *dev_ptr) {
    if (!ctx) return ZANT_NullPointer;
    if (!dev_ptr) return ZANT_OK;
    ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    ZANT_HIP_TRY(ctx, hipFree(dev_ptr));
    return ZANT_OK;
}

extern "C" int zant_hip_upload(zant_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    if (!ctx || (bytes && (!dst_dev || !src_host))) return ZANT_NullPointer;
    if (!bytes) return ZANT_OK;
    ZANT_HIP_TRY(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));  // the host buffer may be pageable and reused
    return ZANT_OK;
}

extern "C" int zant_hip_download(zant_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if (!ctx || (bytes && (!dst_host || !src_dev))) return ZANT_NullPointer;
    if (!bytes) return ZANT_OK;
    ZANT_HIP_TRY(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    ZANT_HIP_TRY(ctx, hipStreamSynchronize(ctx->stream));
    return ZANT_OK;
}

__global__ void zant_fill_bytes_kernel(uint8_t *p, uint8_t v, size_t n) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const size_t step = size_t(gridDim.x) * blockDim.x;
    for (; i < n; i += step) p[i] = v;
}

extern "C" int zant_hip_memset(zant_ctx *ctx, void *dst_dev, int byte_value, size_t bytes) {
    if (!ctx || (bytes && !dst_dev)) return ZANT_NullPointer;
    if (!bytes) return ZANT_OK;
    // A fill kernel rather than hipMemsetAsync so the call stays safe under graph capture.
    size_t blocks = (bytes + 255) / 256;
    if (blocks > 65535) blocks = 65535;
    hipLaunchKernelGGL(zant_fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       static_cast<uint8_t *>(dst_dev), (uint8_t)byte_value, bytes);
    ZANT_LAUNCH_CHECK(ctx);
    return ZANT_OK;
}

extern "C" int zant_hip_timer_start(zant_ctx *ctx) {
    if (!ctx) return ZANT_NullPointer;
    ZANT_HIP_TRY(ctx, hipEventRecord(ctx->ev_start, ctx->stream));
    return ZANT_OK;
}

extern "C" int zant_hip_timer_stop(zant_ctx *ctx, float *elapsed_ms) {
    if (!ctx || !elapsed_ms) return ZANT_NullPointer;
    ZANT_HIP_TRY(ctx, hipEventRecord(ctx->ev_stop, ctx->stream));
    ZANT_HIP_TRY(ctx, hipEventSynchronize(ctx->ev_stop));
    ZANT_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_start, ctx->ev_stop));
    return ZANT_OK;
}

extern "C" int zant_hip_kernel_timing(zant_ctx *ctx, int enable) {
    if (!ctx) return ZANT_NullPointer;
    ctx->kernel_timing = enable != 0;
    return ZANT_OK;
}

extern "C" const char *zant_hip_kernel_name(zant_ctx *ctx) { return ctx ? ctx->last_kernel : ""; }

extern "C" int zant_hip_kernel_ms(zant_ctx *ctx, float *elapsed_ms) {
    if (!ctx || !elapsed_ms) return ZANT_NullPointer;
    ZANT_HIP_TRY(ctx, hipEventSynchronize(ctx->ev_k1));
    ZANT_HIP_TRY(ctx, hipEventElapsedTime(elapsed_ms, ctx->ev_k0, ctx->ev_k1));
    return ZANT_OK;
}
