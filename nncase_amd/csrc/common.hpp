// Shared host-side plumbing of libnncase_hip.so: context object, error
// recording, argument checks, small device helpers.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>

#include <cerrno>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/nncase_hip.h"

struct nncase_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool owns_stream = false;
    int compute_units = 0;
    int clock_khz = 0;
    size_t hbm_bytes = 0;
    // paged-attention partials and completion counters, owned by the context (calls on one context
    // are ordered on its stream, so they can share them).  Sized when an attention operator is
    // recorded into a function or first called eagerly; never moved while a captured graph holds
    // their addresses (attn_pins = captured functions with an attention operator).
    void *attn_ws = nullptr;
    size_t attn_ws_bytes = 0;
    void *attn_done = nullptr; // counters live apart from the partials: they must stay zero between calls
    size_t attn_done_bytes = 0;
    int attn_pins = 0;
    // this GPU's copy of the static scratch of nncase_hip_paged_attention_decode_noalloc (its device address, taken
    // when the context is created so that the entry point itself makes no runtime call but launches)
    void *attn_static = nullptr;
    char last_error[512] = {0};
};

namespace nnhip {

// Device address of the static scratch array of the attention entry point that allocates nothing, on `device`
// (which must be current).  attn.hip, where the array lives.
hipError_t attn_static_scratch_address(void **ptr);

inline int fail(nncase_hip_ctx *ctx, int code, const char *fmt, ...) {
    if (ctx) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(ctx->last_error, sizeof(ctx->last_error), fmt, ap);
        va_end(ap);
    }
    return code;
}

inline int hip_fail(nncase_hip_ctx *ctx, hipError_t e, const char *what) {
    return fail(ctx, -(NNCASE_HIP_ERR_HIP_BASE + (int)e), "%s: %s", what, hipGetErrorString(e));
}

#define NNHIP_CHECK_CTX(ctx)                                                                                           \
    do {                                                                                                               \
        if (!(ctx)) return -EINVAL;                                                                                    \
    } while (0)

#define NNHIP_REQUIRE(ctx, cond, code, ...)                                                                            \
    do {                                                                                                               \
        if (!(cond)) return ::nnhip::fail((ctx), (code), __VA_ARGS__);                                                 \
    } while (0)

#define NNHIP_HIP(ctx, expr)                                                                                           \
    do {                                                                                                               \
        hipError_t e__ = (expr);                                                                                       \
        if (e__ != hipSuccess) return ::nnhip::hip_fail((ctx), e__, #expr);                                            \
    } while (0)

// Checks the launch itself (bad configuration etc.); execution errors surface
// at the next synchronising call.
#define NNHIP_LAUNCH_CHECK(ctx, name)                                                                                  \
    do {                                                                                                               \
        hipError_t e__ = hipGetLastError();                                                                            \
        if (e__ != hipSuccess) return ::nnhip::hip_fail((ctx), e__, name);                                             \
    } while (0)

inline int dtype_size(int dt) {
    switch (dt) {
    case NNCASE_HIP_DT_I8:
    case NNCASE_HIP_DT_U8: return 1;
    case NNCASE_HIP_DT_I16:
    case NNCASE_HIP_DT_F16: return 2;
    case NNCASE_HIP_DT_I32:
    case NNCASE_HIP_DT_F32: return 4;
    default: return 0;
    }
}

// src/Native/include/nncase/kernels/kernel_utils.h:86-93
inline int32_t windowed_output_size(int32_t size, int32_t filter, int32_t stride, int32_t dilation, int32_t before,
                                    int32_t after) {
    const int32_t eff = (filter - 1) * dilation + 1;
    return (size + before + after - eff + stride) / stride;
}

// Division of a 31-bit numerator by a runtime constant as multiply-high +
// shift (round-up method): q = (n * mul) >> (32 + shift).
struct FastDiv {
    uint32_t mul;
    uint32_t shift;
    uint32_t div;
};

inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.div = d;
    if (d == 1) {
        f.mul = 0;
        f.shift = 0;
        return f;
    }
    uint32_t l = 0;
    while ((1u << l) < d) l++;
    // mul = ceil(2^(32+l) / d) - 2^32, used as q = (umulhi(n, mul) + n) >> l
    const uint64_t m = ((uint64_t(1) << 32) * ((uint64_t(1) << l) - d)) / d + 1;
    f.mul = (uint32_t)m;
    f.shift = l;
    return f;
}

__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv &f) {
    // exact for n < 2^31 (Granlund-Montgomery / Hacker's Delight 10-9 form)
    // (a select, not a branch, for the divisor 1: callers count on straight-line code around their loads)
    const uint32_t t = __umulhi(n, f.mul);
    const uint32_t q = (t + ((n - t) >> 1)) >> ((f.shift - 1) & 31u);
    return f.div == 1 ? n : q;
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

template <typename TQ> struct QLimits;
template <> struct QLimits<uint8_t> { static constexpr float lo = 0.f, hi = 255.f; };
template <> struct QLimits<int8_t> { static constexpr float lo = -128.f, hi = 127.f; };
template <> struct QLimits<int16_t> { static constexpr float lo = -32768.f, hi = 32767.f; };

// rne(v) then saturate.  The clamp is done on the float before rounding: the
// limits are integers, so clamp and round-half-even commute, and values
// beyond the int32 range saturate instead of wrapping.
template <typename TQ> __device__ __forceinline__ TQ quantize_one(float x, float scale, float bias) {
    float v = x / scale + bias;
    v = fminf(fmaxf(v, QLimits<TQ>::lo), QLimits<TQ>::hi); // NaN -> lo
    return (TQ)(int32_t)rintf(v);
}


// attn.hip: checks the geometry and sizes the context's paged-attention workspace for it
// (-EBUSY if that needs a reallocation while a captured graph refers to it or the stream is capturing).
int attn_reserve(nncase_hip_ctx *ctx, const nncase_hip_paged_attn_args_t *geometry);
// Bytes of split partials and of counters paged attention needs for a geometry, and the launch on areas the caller
// brings (the counters zero before the first launch; every launch leaves them zero again).
int attn_scratch_sizes(nncase_hip_ctx *ctx, const nncase_hip_paged_attn_args_t *geometry, size_t *partial_bytes, size_t *counter_bytes);
int attn_decode_on(nncase_hip_ctx *ctx, const void *q_dev, const void *k_cache_dev, const void *v_cache_dev, const int32_t *block_table_dev,
                   const int32_t *ctx_lens_dev, void *out_dev, const nncase_hip_paged_attn_args_t *geometry, void *partials,
                   size_t partial_bytes, void *counters, size_t counter_bytes);

} // namespace nnhip
