// u8 glue operators that keep a quantized graph resident on the device between the
// convolutions: byte-table unary operators (requantisation, swish), channel concat with
// requantisation to a common scale, nearest-neighbour resize.  All are bound by HBM
// bandwidth; the arithmetic that decides a byte is done once per table entry on the host
// (256 evaluations with the same fp32 operations the CPU kernels use), so the device only
// moves bytes and the result is bit-exact by construction.
#include "common.hpp"

#include <cmath>

namespace nnhip {

constexpr int kGlueThreads = 256;

struct ByteTable {
    uint32_t w[64]; // 256 entries, little-endian packed
};

__device__ __forceinline__ uint32_t lut4(const uint8_t *t, uint32_t v) {
    return (uint32_t)t[v & 0xffu] | ((uint32_t)t[(v >> 8) & 0xffu] << 8) | ((uint32_t)t[(v >> 16) & 0xffu] << 16) |
           ((uint32_t)t[v >> 24] << 24);
}

__device__ __forceinline__ void stage_table(uint8_t *t, const ByteTable &lut) {
    if (threadIdx.x < 64) reinterpret_cast<uint32_t *>(t)[threadIdx.x] = lut.w[threadIdx.x];
    __syncthreads();
}

// out[i] = table[in[i]], 16 bytes per thread per step.
__global__ __launch_bounds__(kGlueThreads) void lut_u8_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                             size_t count, const ByteTable lut, int vec_ok) {
    __shared__ __align__(16) uint8_t t[256];
    stage_table(t, lut);
    const size_t tid = (size_t)blockIdx.x * kGlueThreads + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * kGlueThreads;
    const size_t nvec = vec_ok ? count / 16 : 0;
    for (size_t i = tid; i < nvec; i += nthreads) {
        const uint4 v = *reinterpret_cast<const uint4 *>(in + i * 16);
        *reinterpret_cast<uint4 *>(out + i * 16) = uint4{lut4(t, v.x), lut4(t, v.y), lut4(t, v.z), lut4(t, v.w)};
    }
    for (size_t j = nvec * 16 + tid; j < count; j += nthreads) out[j] = t[in[j]];
}

// One input of a channel concat: out[p, c_off + c] = table[in[p, c]] for c < c_in.
// VEC = bytes per thread: 16 when every channel count (hence every offset and the output's pixel stride) is a multiple
// of 16 and the buffers are 16-byte aligned, 4 likewise, else 1.
template <int VEC>
__global__ __launch_bounds__(kGlueThreads) void concat_lut_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
                                                                 uint32_t total, FastDiv d_cv, uint32_t c_in,
                                                                 uint32_t c_out, uint32_t c_off, const ByteTable lut) {
    __shared__ __align__(16) uint8_t t[256];
    stage_table(t, lut);
    const uint32_t gid = blockIdx.x * kGlueThreads + threadIdx.x;
    if (gid >= total) return;
    const uint32_t p = fastdiv(gid, d_cv);
    const uint32_t c = (gid - p * d_cv.div) * VEC;
    const size_t src = (size_t)p * c_in + c, dst = (size_t)p * c_out + c_off + c;
    if (VEC == 16) {
        const uint4 v = *reinterpret_cast<const uint4 *>(in + src);
        *reinterpret_cast<uint4 *>(out + dst) = uint4{lut4(t, v.x), lut4(t, v.y), lut4(t, v.z), lut4(t, v.w)};
    } else if (VEC == 4) {
        *reinterpret_cast<uint32_t *>(out + dst) = lut4(t, *reinterpret_cast<const uint32_t *>(in + src));
    } else {
        out[dst] = t[in[src]];
    }
}

// Every input of a channel concat in one launch (vector widths of 16 or 4 bytes): a thread owns VEC channels of one output
// pixel, finds the input they come from and applies that input's table; channels of an input that is already in place
// (a null pointer: written there by its producer) are left alone.
struct ConcatArgs {
    const uint8_t *in[NNCASE_HIP_MAX_CONCAT];
    uint32_t c_in[NNCASE_HIP_MAX_CONCAT], c_end[NNCASE_HIP_MAX_CONCAT]; // channels of input i; first output channel behind it
    ByteTable lut[NNCASE_HIP_MAX_CONCAT];
    uint8_t *out;
    uint32_t total, c_out;
    int n;
    FastDiv d_cv; // vectors per output pixel
};
template <int VEC> __global__ __launch_bounds__(kGlueThreads) void concat_all_kernel(const ConcatArgs a) {
    __shared__ __align__(16) uint8_t t[NNCASE_HIP_MAX_CONCAT][256];
    for (int i = threadIdx.x; i < a.n * 64; i += kGlueThreads) reinterpret_cast<uint32_t *>(t[i >> 6])[i & 63] = a.lut[i >> 6].w[i & 63];
    __syncthreads();
    const uint32_t gid = blockIdx.x * kGlueThreads + threadIdx.x;
    if (gid >= a.total) return;
    const uint32_t p = fastdiv(gid, a.d_cv);
    const uint32_t c = (gid - p * a.d_cv.div) * VEC;
    int i = 0;
    while (i + 1 < a.n && c >= a.c_end[i]) i++;
    if (!a.in[i]) return;
    const uint32_t c0 = i == 0 ? 0u : a.c_end[i - 1];
    const size_t src = (size_t)p * a.c_in[i] + (c - c0), dst = (size_t)p * a.c_out + c;
    if (VEC == 16) {
        const uint4 v = *reinterpret_cast<const uint4 *>(a.in[i] + src);
        *reinterpret_cast<uint4 *>(a.out + dst) = uint4{lut4(t[i], v.x), lut4(t[i], v.y), lut4(t[i], v.z), lut4(t[i], v.w)};
    } else {
        *reinterpret_cast<uint32_t *>(a.out + dst) = lut4(t[i], *reinterpret_cast<const uint32_t *>(a.in[i] + src));
    }
}

// Coordinate of an output index in the input (get_coordinate_from_resized,
// src/Native/include/nncase/kernels/stackvm/resize_image.h:30-66) and the rounding to a pixel
// (get_nearest_pixel_from_origin, :68-92): the same single fp32 operations in the same order.
__device__ __forceinline__ float resize_coordinate(int mode, float x_resized, float x_scale, float length_resized,
                                                   float length_original) {
    switch (mode) {
    case 3: return x_resized * x_scale;
    case 1: return length_resized > 1 ? (x_resized + 0.5f) * x_scale - 0.5f : 0.0f;
    case 2: return length_resized == 1 ? 0.f : x_resized * (length_original - 1) / (length_resized - 1);
    case 4: return 0.f; // tfcrop_and_resize: the nearest kernel passes roi (0, 0), which maps every index to 0
    default: return ((x_resized + 0.5f) * x_scale) - 0.5f;
    }
}

__device__ __forceinline__ int resize_nearest_pixel(int mode, float x, int length) {
    float r;
    switch (mode) {
    case 1: r = roundf(x); break;
    case 2: r = floorf(x); break;
    case 3: r = ceilf(x); break;
    default: r = (x == truncf(x) + 0.5f) ? floorf(x) : roundf(x); break; // halves prefer the floor
    }
    // the reference clamps after the conversion to int64; clamping the float first gives the same index
    r = fminf(fmaxf(r, 0.f), (float)(length - 1));
    return (int)r;
}

struct ResizeArgs {
    const uint8_t *in;
    uint8_t *out;
    int in_h, in_w, out_h, out_w;
    uint32_t row_vecs; // vectors per pixel (channels * element size / VEC)
    FastDiv d_vecs, d_ow, d_oh;
    uint32_t total;
    float h_scale, w_scale;
    int tmode, nmode;
};

// NHWC: every output pixel copies the channel vector of its source pixel.
template <typename V> __global__ __launch_bounds__(kGlueThreads) void resize_nearest_kernel(const ResizeArgs a) {
    const uint32_t gid = blockIdx.x * kGlueThreads + threadIdx.x;
    if (gid >= a.total) return;
    uint32_t q = fastdiv(gid, a.d_vecs);
    const uint32_t v = gid - q * a.d_vecs.div;
    uint32_t t = q;
    q = fastdiv(t, a.d_ow);
    const int ox = (int)(t - q * a.d_ow.div);
    t = q;
    q = fastdiv(t, a.d_oh);
    const int oy = (int)(t - q * a.d_oh.div);
    const uint32_t n = q;
    const int iy = resize_nearest_pixel(a.nmode, resize_coordinate(a.tmode, (float)oy, a.h_scale, (float)a.out_h, (float)a.in_h), a.in_h);
    const int ix = resize_nearest_pixel(a.nmode, resize_coordinate(a.tmode, (float)ox, a.w_scale, (float)a.out_w, (float)a.in_w), a.in_w);
    const size_t src = (((size_t)n * a.in_h + iy) * a.in_w + ix) * a.row_vecs + v;
    reinterpret_cast<V *>(a.out)[gid] = reinterpret_cast<const V *>(a.in)[src];
}

struct PoolArgs {
    const uint8_t *in;
    uint8_t *out;
    int in_h, in_w, out_h, out_w, kh, kw, stride_h, stride_w, pad_h, pad_w;
    uint32_t cvecs; // channel vectors per pixel
    FastDiv d_cvecs, d_ow, d_oh;
    uint32_t total;
    uint32_t zero_code; // Q(0.0) with the output's quant params, replicated in the four bytes
};

__device__ __forceinline__ uint32_t max_u8x4(uint32_t a, uint32_t b) {
    // bytewise unsigned max of two packed dwords (v_pk_max_u8 does not exist; compare bytes)
    uint32_t r = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t x = (a >> (8 * i)) & 0xffu, y = (b >> (8 * i)) & 0xffu;
        r |= (x > y ? x : y) << (8 * i);
    }
    return r;
}

// reduce_window2d(max) on NHWC u8, then a byte table (the requantisation to the output's quant
// params; the maximum commutes with the increasing maps Dequantize and Quantize, so it is taken
// on the codes).  The reference folds the value 0 into the result once per window position that
// lies in the padding (src/Native/src/kernels/stackvm/reference/reduce_window.cpp:88-91), so a
// window that overlaps the border yields max(values, 0): here max(table[m], Q(0)).
template <int VEC> __global__ __launch_bounds__(kGlueThreads) void maxpool_u8_kernel(const PoolArgs a, const ByteTable lut) {
    __shared__ __align__(16) uint8_t t[256];
    stage_table(t, lut);
    const uint32_t gid = blockIdx.x * kGlueThreads + threadIdx.x;
    if (gid >= a.total) return;
    uint32_t q = fastdiv(gid, a.d_cvecs);
    const uint32_t v = gid - q * a.d_cvecs.div;
    uint32_t r = q;
    q = fastdiv(r, a.d_ow);
    const int ox = (int)(r - q * a.d_ow.div);
    r = q;
    q = fastdiv(r, a.d_oh);
    const int oy = (int)(r - q * a.d_oh.div);
    const uint32_t n = q;
    const int y0 = max(oy * a.stride_h - a.pad_h, 0), y1 = min(oy * a.stride_h - a.pad_h + a.kh, a.in_h);
    const int x0 = max(ox * a.stride_w - a.pad_w, 0), x1 = min(ox * a.stride_w - a.pad_w + a.kw, a.in_w);
    const bool padded = (y1 - y0) * (x1 - x0) < a.kh * a.kw;
    if (VEC == 16) { // 16 channels per thread: a quarter of the loads for the same bytes
        uint4 m4 = uint4{0u, 0u, 0u, 0u};
        for (int y = y0; y < y1; y++)
            for (int x = x0; x < x1; x++) {
                const uint4 d = reinterpret_cast<const uint4 *>(a.in)[(((size_t)n * a.in_h + y) * a.in_w + x) * a.cvecs + v];
                m4 = uint4{max_u8x4(m4.x, d.x), max_u8x4(m4.y, d.y), max_u8x4(m4.z, d.z), max_u8x4(m4.w, d.w)};
            }
        uint4 o = uint4{lut4(t, m4.x), lut4(t, m4.y), lut4(t, m4.z), lut4(t, m4.w)};
        if (padded) o = uint4{max_u8x4(o.x, a.zero_code), max_u8x4(o.y, a.zero_code), max_u8x4(o.z, a.zero_code), max_u8x4(o.w, a.zero_code)};
        reinterpret_cast<uint4 *>(a.out)[gid] = o;
        return;
    }
    uint32_t m = 0;
    for (int y = y0; y < y1; y++)
        for (int x = x0; x < x1; x++) {
            const size_t src = (((size_t)n * a.in_h + y) * a.in_w + x) * a.cvecs + v;
            if (VEC == 4) m = max_u8x4(m, reinterpret_cast<const uint32_t *>(a.in)[src]);
            else m = max(m, (uint32_t)a.in[src]);
        }
    if (VEC == 4) {
        uint32_t o = lut4(t, m);
        if (padded) o = max_u8x4(o, a.zero_code);
        reinterpret_cast<uint32_t *>(a.out)[gid] = o;
    } else {
        uint32_t o = t[m];
        if (padded) o = max(o, a.zero_code & 0xffu);
        a.out[gid] = (uint8_t)o;
    }
}

inline ByteTable pack_table(const uint8_t *lut) {
    ByteTable t;
    memcpy(t.w, lut, 256);
    return t;
}

} // namespace nnhip

using namespace nnhip;

extern "C" int nncase_hip_make_unary_lut(int32_t kind, nncase_hip_quant_param_t x_qp, nncase_hip_quant_param_t y_qp,
                                         uint8_t *lut) {
    if (!lut || (kind != NNCASE_HIP_LUT_REQUANT && kind != NNCASE_HIP_LUT_SWISH)) return -EINVAL;
    if (!(y_qp.scale != 0.f)) return -EINVAL;
    for (int v = 0; v < 256; v++) {
        const float x = ((float)v - (float)x_qp.zero_point) * x_qp.scale;
        float f = x;
        if (kind == NNCASE_HIP_LUT_SWISH) f = x / (1 + expf(-x));
        const float t = f / y_qp.scale + (float)y_qp.zero_point;
        float r = nearbyintf(t); // round half to even (default rounding mode)
        if (!(r >= 0.f)) r = 0.f; // also NaN
        if (r > 255.f) r = 255.f;
        lut[v] = (uint8_t)r;
    }
    return 0;
}

extern "C" int nncase_hip_lut_u8(nncase_hip_ctx_t *ctx, const uint8_t *in_dev, uint8_t *out_dev, size_t count,
                                 const uint8_t *lut_host) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, lut_host, -EINVAL, "lut_u8: null table");
    if (count == 0) return 0;
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "lut_u8: null buffer");
    const int vec_ok = ((reinterpret_cast<uintptr_t>(in_dev) | reinterpret_cast<uintptr_t>(out_dev)) & 15u) == 0;
    const size_t vecs = (count + 15) / 16;
    const size_t want = (vecs + kGlueThreads - 1) / kGlueThreads;
    const size_t cap = (size_t)ctx->compute_units * 16;
    const int grid = (int)(want < cap ? (want ? want : 1) : cap);
    hipLaunchKernelGGL(lut_u8_kernel, dim3(grid), dim3(kGlueThreads), 0, ctx->stream, in_dev, out_dev, count,
                       pack_table(lut_host), vec_ok);
    NNHIP_LAUNCH_CHECK(ctx, "lut_u8_kernel");
    return 0;
}

extern "C" int nncase_hip_qconcat_channels(nncase_hip_ctx_t *ctx, int32_t n_inputs, const uint8_t *const *in_dev,
                                           const int32_t *channels, const nncase_hip_quant_param_t *in_qps,
                                           uint8_t *out_dev, nncase_hip_quant_param_t out_qp, int64_t pixels) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, n_inputs > 0 && n_inputs <= NNCASE_HIP_MAX_CONCAT && in_dev && channels && in_qps && out_dev, -EINVAL,
                  "qconcat_channels: bad argument (1..%d inputs)", NNCASE_HIP_MAX_CONCAT);
    NNHIP_REQUIRE(ctx, pixels >= 0, -EINVAL, "qconcat_channels: negative pixel count");
    NNHIP_REQUIRE(ctx, out_qp.scale != 0.f, -EINVAL, "qconcat_channels: output scale is zero");
    int64_t c_out = 0;
    bool vec = (reinterpret_cast<uintptr_t>(out_dev) & 3u) == 0, vec16 = (reinterpret_cast<uintptr_t>(out_dev) & 15u) == 0;
    for (int i = 0; i < n_inputs; i++) {
        NNHIP_REQUIRE(ctx, channels[i] > 0, -EINVAL, "qconcat_channels: input %d is empty", i);
        vec = vec && channels[i] % 4 == 0 && (reinterpret_cast<uintptr_t>(in_dev[i]) & 3u) == 0; // (a skipped input is null)
        vec16 = vec16 && channels[i] % 16 == 0 && (reinterpret_cast<uintptr_t>(in_dev[i]) & 15u) == 0;
        c_out += channels[i];
    }
    if (pixels == 0) return 0;
    int live = 0;
    for (int i = 0; i < n_inputs; i++) live += in_dev[i] != nullptr;
    if (vec && live > 1) { // one launch for all the inputs (a single one that is not in place yet keeps the launch that covers its channels only)
        const int v = vec16 ? 16 : 4;
        const int64_t total = pixels * (c_out / v);
        if (total < ((int64_t)1 << 31)) {
            ConcatArgs a;
            memset(&a, 0, sizeof(a));
            uint32_t end = 0;
            bool any = false;
            for (int i = 0; i < n_inputs; i++) {
                end += (uint32_t)channels[i];
                a.in[i] = in_dev[i], a.c_in[i] = (uint32_t)channels[i], a.c_end[i] = end;
                if (!in_dev[i]) continue;
                any = true;
                uint8_t lut[256];
                const int rc = nncase_hip_make_unary_lut(NNCASE_HIP_LUT_REQUANT, in_qps[i], out_qp, lut);
                NNHIP_REQUIRE(ctx, rc == 0, rc, "qconcat_channels: cannot build the requantisation table of input %d", i);
                a.lut[i] = pack_table(lut);
            }
            if (!any) return 0;
            a.out = out_dev, a.total = (uint32_t)total, a.c_out = (uint32_t)c_out, a.n = n_inputs, a.d_cv = make_fastdiv((uint32_t)(c_out / v));
            const dim3 grid((unsigned)((total + kGlueThreads - 1) / kGlueThreads));
            if (vec16) hipLaunchKernelGGL(concat_all_kernel<16>, grid, dim3(kGlueThreads), 0, ctx->stream, a);
            else hipLaunchKernelGGL(concat_all_kernel<4>, grid, dim3(kGlueThreads), 0, ctx->stream, a);
            NNHIP_LAUNCH_CHECK(ctx, "concat_all_kernel");
            return 0;
        }
    }
    uint32_t c_off = 0;
    for (int i = 0; i < n_inputs; i++) {
        if (!in_dev[i]) { // already in place: written by its producer
            c_off += (uint32_t)channels[i];
            continue;
        }
        uint8_t lut[256];
        const int rc = nncase_hip_make_unary_lut(NNCASE_HIP_LUT_REQUANT, in_qps[i], out_qp, lut);
        NNHIP_REQUIRE(ctx, rc == 0, rc, "qconcat_channels: cannot build the requantisation table of input %d", i);
        const int v = vec16 ? 16 : (vec ? 4 : 1);
        const int64_t total = pixels * (channels[i] / v);
        NNHIP_REQUIRE(ctx, total < ((int64_t)1 << 31), -EINVAL, "qconcat_channels: input %d too large", i);
        const FastDiv d_cv = make_fastdiv((uint32_t)(channels[i] / v));
        const dim3 grid((unsigned)((total + kGlueThreads - 1) / kGlueThreads));
        if (vec16)
            hipLaunchKernelGGL(concat_lut_kernel<16>, grid, dim3(kGlueThreads), 0, ctx->stream, in_dev[i], out_dev, (uint32_t)total,
                               d_cv, (uint32_t)channels[i], (uint32_t)c_out, c_off, pack_table(lut));
        else if (vec)
            hipLaunchKernelGGL(concat_lut_kernel<4>, grid, dim3(kGlueThreads), 0, ctx->stream, in_dev[i], out_dev, (uint32_t)total,
                               d_cv, (uint32_t)channels[i], (uint32_t)c_out, c_off, pack_table(lut));
        else
            hipLaunchKernelGGL(concat_lut_kernel<1>, grid, dim3(kGlueThreads), 0, ctx->stream, in_dev[i], out_dev, (uint32_t)total,
                               d_cv, (uint32_t)channels[i], (uint32_t)c_out, c_off, pack_table(lut));
        NNHIP_LAUNCH_CHECK(ctx, "concat_lut_kernel");
        c_off += (uint32_t)channels[i];
    }
    return 0;
}

extern "C" int nncase_hip_resize_nearest(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size,
                                         int32_t batch, int32_t in_h, int32_t in_w, int32_t channels, int32_t out_h,
                                         int32_t out_w, int32_t transformation_mode, int32_t nearest_mode) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "resize_nearest: null buffer");
    NNHIP_REQUIRE(ctx, elem_size == 1 || elem_size == 2 || elem_size == 4, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                  "resize_nearest: element size %d", elem_size);
    NNHIP_REQUIRE(ctx, batch > 0 && in_h > 0 && in_w > 0 && channels > 0 && out_h > 0 && out_w > 0, -EINVAL,
                  "resize_nearest: non-positive dimension");
    NNHIP_REQUIRE(ctx, transformation_mode >= 0 && transformation_mode <= 4 && nearest_mode >= 0 && nearest_mode <= 3, -EINVAL,
                  "resize_nearest: unknown mode (%d, %d)", transformation_mode, nearest_mode);
    NNHIP_REQUIRE(ctx, in_h < (1 << 24) && in_w < (1 << 24) && out_h < (1 << 24) && out_w < (1 << 24), -EINVAL,
                  "resize_nearest: extent beyond 2^24 (indices are computed in fp32, as in the CPU kernel)");
    const int64_t row_bytes = (int64_t)channels * elem_size;
    const uintptr_t addr = reinterpret_cast<uintptr_t>(in_dev) | reinterpret_cast<uintptr_t>(out_dev);
    int vec = 1;
    if (row_bytes % 16 == 0 && (addr & 15u) == 0) vec = 16;
    else if (row_bytes % 4 == 0 && (addr & 3u) == 0) vec = 4;
    ResizeArgs a;
    a.in = (const uint8_t *)in_dev;
    a.out = (uint8_t *)out_dev;
    a.in_h = in_h, a.in_w = in_w, a.out_h = out_h, a.out_w = out_w;
    a.row_vecs = (uint32_t)(row_bytes / vec);
    const int64_t total = (int64_t)batch * out_h * out_w * a.row_vecs;
    NNHIP_REQUIRE(ctx, total < ((int64_t)1 << 31), -EINVAL, "resize_nearest: too many work items");
    a.total = (uint32_t)total;
    a.d_vecs = make_fastdiv(a.row_vecs);
    a.d_ow = make_fastdiv((uint32_t)out_w);
    a.d_oh = make_fastdiv((uint32_t)out_h);
    // get_resize_scales, src/Native/include/nncase/kernels/kernel_utils.h:224-233
    const bool align = transformation_mode == 2;
    a.h_scale = (float)in_h / out_h;
    a.w_scale = (float)in_w / out_w;
    if (align && out_h > 1) a.h_scale = (float)(in_h - 1) / (out_h - 1);
    if (align && out_w > 1) a.w_scale = (float)(in_w - 1) / (out_w - 1);
    a.tmode = transformation_mode, a.nmode = nearest_mode;
    const dim3 grid((unsigned)((total + kGlueThreads - 1) / kGlueThreads));
    if (vec == 16) hipLaunchKernelGGL(resize_nearest_kernel<uint4>, grid, dim3(kGlueThreads), 0, ctx->stream, a);
    else if (vec == 4) hipLaunchKernelGGL(resize_nearest_kernel<uint32_t>, grid, dim3(kGlueThreads), 0, ctx->stream, a);
    else hipLaunchKernelGGL(resize_nearest_kernel<uint8_t>, grid, dim3(kGlueThreads), 0, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "resize_nearest_kernel");
    return 0;
}

extern "C" int nncase_hip_qmaxpool2d(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, uint8_t *out_dev, int32_t batch, int32_t in_h,
                                     int32_t in_w, int32_t channels, int32_t kernel_h, int32_t kernel_w, int32_t stride_h,
                                     int32_t stride_w, int32_t pad_h_before, int32_t pad_h_after, int32_t pad_w_before,
                                     int32_t pad_w_after, nncase_hip_quant_param_t x_qp, nncase_hip_quant_param_t y_qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && out_dev, -EINVAL, "qmaxpool2d: null buffer");
    NNHIP_REQUIRE(ctx, batch > 0 && in_h > 0 && in_w > 0 && channels > 0 && kernel_h > 0 && kernel_w > 0 && stride_h > 0 &&
                           stride_w > 0 && pad_h_before >= 0 && pad_h_after >= 0 && pad_w_before >= 0 && pad_w_after >= 0,
                  -EINVAL, "qmaxpool2d: bad shape");
    // every window must contain at least one pixel of the image
    NNHIP_REQUIRE(ctx, pad_h_before < kernel_h && pad_h_after < kernel_h && pad_w_before < kernel_w && pad_w_after < kernel_w,
                  -EINVAL, "qmaxpool2d: padding not smaller than the window");
    const int out_h = windowed_output_size(in_h, kernel_h, stride_h, 1, pad_h_before, pad_h_after);
    const int out_w = windowed_output_size(in_w, kernel_w, stride_w, 1, pad_w_before, pad_w_after);
    NNHIP_REQUIRE(ctx, out_h > 0 && out_w > 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH, "qmaxpool2d: empty output");
    uint8_t lut[256];
    const int rc = nncase_hip_make_unary_lut(NNCASE_HIP_LUT_REQUANT, x_qp, y_qp, lut);
    NNHIP_REQUIRE(ctx, rc == 0, rc, "qmaxpool2d: cannot build the requantisation table (zero output scale?)");
    const bool vec = channels % 4 == 0 && ((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(out_dev)) & 3u) == 0;
    const bool vec16 = channels % 16 == 0 && ((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(out_dev)) & 15u) == 0;
    PoolArgs a;
    a.in = x_dev, a.out = out_dev;
    a.in_h = in_h, a.in_w = in_w, a.out_h = out_h, a.out_w = out_w, a.kh = kernel_h, a.kw = kernel_w;
    a.stride_h = stride_h, a.stride_w = stride_w, a.pad_h = pad_h_before, a.pad_w = pad_w_before;
    a.cvecs = (uint32_t)(vec16 ? channels / 16 : (vec ? channels / 4 : channels));
    const int64_t total = (int64_t)batch * out_h * out_w * a.cvecs;
    NNHIP_REQUIRE(ctx, total < ((int64_t)1 << 31), -EINVAL, "qmaxpool2d: too many work items");
    a.total = (uint32_t)total;
    a.d_cvecs = make_fastdiv(a.cvecs), a.d_ow = make_fastdiv((uint32_t)out_w), a.d_oh = make_fastdiv((uint32_t)out_h);
    {
        float r = nearbyintf(0.f / y_qp.scale + (float)y_qp.zero_point);
        r = r < 0.f ? 0.f : (r > 255.f ? 255.f : r);
        a.zero_code = (uint32_t)r * 0x01010101u;
    }
    const dim3 grid((unsigned)((total + kGlueThreads - 1) / kGlueThreads));
    if (vec16) hipLaunchKernelGGL(maxpool_u8_kernel<16>, grid, dim3(kGlueThreads), 0, ctx->stream, a, pack_table(lut));
    else if (vec) hipLaunchKernelGGL(maxpool_u8_kernel<4>, grid, dim3(kGlueThreads), 0, ctx->stream, a, pack_table(lut));
    else hipLaunchKernelGGL(maxpool_u8_kernel<1>, grid, dim3(kGlueThreads), 0, ctx->stream, a, pack_table(lut));
    NNHIP_LAUNCH_CHECK(ctx, "maxpool_u8_kernel");
    return 0;
}
