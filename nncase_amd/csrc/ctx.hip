// Context, device memory and stream entry points of libnncase_hip.so.
#include "common.hpp"

#include <mutex>
#include <new>

using namespace nnhip;

extern "C" int nncase_hip_version(void) { return (0 << 16) | 1; }

extern "C" int nncase_hip_ctx_create(int device, nncase_hip_ctx_t **out) {
    if (!out) return -EINVAL;
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) return -ENODEV;
    if (device < 0 || device >= count) return -ENODEV;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return -ENODEV;
    // The kernels are built for gfx950 only; any other part cannot run them.
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return -ENODEV;
    if (hipSetDevice(device) != hipSuccess) return -ENODEV;
    nncase_hip_ctx *ctx = new (std::nothrow) nncase_hip_ctx();
    if (!ctx) return -ENOMEM;
    ctx->device = device;
    ctx->compute_units = prop.multiProcessorCount;
    ctx->clock_khz = prop.clockRate;
    ctx->hbm_bytes = prop.totalGlobalMem;
    e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete ctx;
        return -(NNCASE_HIP_ERR_HIP_BASE + (int)e);
    }
    ctx->owns_stream = true;
    e = nnhip::attn_static_scratch_address(&ctx->attn_static); // (the device is current)
    if (e != hipSuccess || !ctx->attn_static) {
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return e != hipSuccess ? -(NNCASE_HIP_ERR_HIP_BASE + (int)e) : -ENOMEM;
    }
    *out = ctx;
    return 0;
}

// HIP multiplexes streams over at most GPU_MAX_HW_QUEUES hardware queues (4 unless the environment says otherwise): a
// new stream opens a new queue until that many exist and joins the least shared one after that, and kernels of streams
// that share a queue run one after the other.  Idle streams created here, once per device, fill the pool, so that the
// streams of the contexts created afterwards are dealt out one per queue in turn.  They are kept until
// nncase_hip_release_queue_pool destroys them (a host that unloads the library) or the process ends.
namespace {
constexpr int kPoolMaxDevices = 64, kPoolMaxQueues = 32;
std::mutex g_pool_lock;
int g_pool_filled[kPoolMaxDevices] = {0};
hipStream_t g_pool_streams[kPoolMaxDevices][kPoolMaxQueues] = {};
} // namespace

extern "C" int nncase_hip_fill_queue_pool(int device) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count || device >= kPoolMaxDevices) return -ENODEV;
    std::lock_guard<std::mutex> guard(g_pool_lock);
    if (g_pool_filled[device]) return g_pool_filled[device];
    int queues = 4;
    if (const char *env = getenv("GPU_MAX_HW_QUEUES")) {
        const int v = atoi(env);
        if (v >= 1 && v <= kPoolMaxQueues) queues = v;
    }
    if (hipSetDevice(device) != hipSuccess) return -ENODEV;
    for (int i = 0; i < queues; i++) {
        const hipError_t e = hipStreamCreateWithFlags(&g_pool_streams[device][i], hipStreamNonBlocking);
        if (e != hipSuccess) {
            for (int j = 0; j < i; j++) (void)hipStreamDestroy(g_pool_streams[device][j]);
            return -(NNCASE_HIP_ERR_HIP_BASE + (int)e);
        }
    }
    g_pool_filled[device] = queues;
    return queues;
}

extern "C" int nncase_hip_release_queue_pool(int device) {
    if (device < 0 || device >= kPoolMaxDevices) return -ENODEV;
    std::lock_guard<std::mutex> guard(g_pool_lock);
    const int queues = g_pool_filled[device];
    if (!queues) return 0;
    if (hipSetDevice(device) != hipSuccess) return -ENODEV;
    for (int i = 0; i < queues; i++) {
        (void)hipStreamDestroy(g_pool_streams[device][i]);
        g_pool_streams[device][i] = nullptr;
    }
    g_pool_filled[device] = 0;
    return queues;
}

extern "C" int nncase_hip_ctx_destroy(nncase_hip_ctx_t *ctx) {
    NNHIP_CHECK_CTX(ctx);
    if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
    if (ctx->attn_ws) (void)hipFree(ctx->attn_ws);
    if (ctx->attn_done) (void)hipFree(ctx->attn_done);
    if (ctx->owns_stream && ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return 0;
}

extern "C" int nncase_hip_ctx_get_stream(nncase_hip_ctx_t *ctx, void **hip_stream) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, hip_stream, -EINVAL, "get_stream: null out pointer");
    *hip_stream = (void *)ctx->stream;
    return 0;
}

extern "C" int nncase_hip_ctx_set_stream(nncase_hip_ctx_t *ctx, void *hip_stream) {
    NNHIP_CHECK_CTX(ctx);
    if (ctx->stream) NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (ctx->owns_stream && ctx->stream) NNHIP_HIP(ctx, hipStreamDestroy(ctx->stream));
    ctx->stream = (hipStream_t)hip_stream;
    ctx->owns_stream = false;
    return 0;
}

extern "C" const char *nncase_hip_last_error_string(nncase_hip_ctx_t *ctx) { return ctx ? ctx->last_error : ""; }

extern "C" int nncase_hip_device_info(nncase_hip_ctx_t *ctx, int *compute_units, int *clock_khz, size_t *hbm_bytes) {
    NNHIP_CHECK_CTX(ctx);
    if (compute_units) *compute_units = ctx->compute_units;
    if (clock_khz) *clock_khz = ctx->clock_khz;
    if (hbm_bytes) *hbm_bytes = ctx->hbm_bytes;
    return 0;
}

extern "C" int nncase_hip_malloc(nncase_hip_ctx_t *ctx, size_t bytes, void **dptr) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, dptr, -EINVAL, "malloc: null out pointer");
    *dptr = nullptr;
    if (bytes == 0) bytes = 1;
    hipError_t e = hipMalloc(dptr, bytes);
    if (e == hipErrorOutOfMemory) return fail(ctx, -ENOMEM, "malloc: out of device memory (%zu bytes)", bytes);
    NNHIP_HIP(ctx, e);
    return 0;
}

extern "C" int nncase_hip_free(nncase_hip_ctx_t *ctx, void *dptr) {
    NNHIP_CHECK_CTX(ctx);
    if (!dptr) return 0;
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    NNHIP_HIP(ctx, hipFree(dptr));
    return 0;
}

extern "C" int nncase_hip_memcpy_h2d(nncase_hip_ctx_t *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, (dst_dev && src_host) || bytes == 0, -EINVAL, "memcpy_h2d: null pointer");
    if (!bytes) return 0;
    NNHIP_HIP(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return 0;
}

extern "C" int nncase_hip_memcpy_d2h(nncase_hip_ctx_t *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, (dst_host && src_dev) || bytes == 0, -EINVAL, "memcpy_d2h: null pointer");
    if (!bytes) return 0;
    NNHIP_HIP(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return 0;
}

extern "C" int nncase_hip_memset(nncase_hip_ctx_t *ctx, void *dptr, int byte, size_t bytes) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, dptr || bytes == 0, -EINVAL, "memset: null pointer");
    if (!bytes) return 0;
    NNHIP_HIP(ctx, hipMemsetAsync(dptr, byte, bytes, ctx->stream));
    return 0;
}

extern "C" int nncase_hip_stream_sync(nncase_hip_ctx_t *ctx) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    return 0;
}
