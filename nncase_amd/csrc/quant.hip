// Quantize / Dequantize streaming kernels and the u8 elementwise glue
// (residual add, global average pool).  All HBM-bound: every thread moves
// 4 elements per step with one vector load and one vector store, the grid is
// a few waves per SIMD deep and walks the tensor with a grid stride so the
// loads of several steps are in flight together.
//
// Arithmetic contracts (each fp32 step is a single IEEE operation; the file
// is compiled with -ffp-contract=off):
//   quantize    q = sat_T((int32) rne(x / scale + bias))          reference/quantize.cpp:36-43
//   dequantize  y = ((float) q - bias) * scale                    reference/dequantize.cpp:36-39
#include "qconv.hpp"

#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>

namespace nnhip {

constexpr int kEwThreads = 256;
constexpr int kEwVec = 4;
constexpr int kEwUnroll = 4;

template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float4 type; };
template <> struct Vec4<int32_t> { typedef int4 type; };
template <> struct Vec4<__half> { typedef uint2 type; };
template <> struct Vec4<int16_t> { typedef uint2 type; };
template <> struct Vec4<uint8_t> { typedef uint32_t type; };
template <> struct Vec4<int8_t> { typedef uint32_t type; };

template <typename T> __device__ __forceinline__ void load4(const T *p, T (&v)[4]) {
    typename Vec4<T>::type raw = *reinterpret_cast<const typename Vec4<T>::type *>(p);
    __builtin_memcpy(v, &raw, sizeof(raw));
}
template <typename T> __device__ __forceinline__ void store4(T *p, const T (&v)[4]) {
    typename Vec4<T>::type raw;
    __builtin_memcpy(&raw, v, sizeof(raw));
    *reinterpret_cast<typename Vec4<T>::type *>(p) = raw;
}

template <typename T> __device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <> __device__ __forceinline__ float to_f32<__half>(__half v) { return __half2float(v); }

template <typename TIn, typename TQ>
__global__ __launch_bounds__(kEwThreads) void quantize_kernel(const TIn *__restrict__ in, TQ *__restrict__ out,
                                                              size_t count, float scale, float bias, int vec_ok) {
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    const size_t nvec = vec_ok ? count / kEwVec : 0;
    // a block owns kEwUnroll * kEwThreads neighbouring vectors (see ew_block_grid)
    const size_t i = (size_t)blockIdx.x * (kEwUnroll * kEwThreads) + threadIdx.x;
    if (i + (kEwUnroll - 1) * kEwThreads < nvec) {
        TIn v[kEwUnroll][4];
#pragma unroll
        for (int u = 0; u < kEwUnroll; u++) load4(in + (i + u * kEwThreads) * kEwVec, v[u]);
#pragma unroll
        for (int u = 0; u < kEwUnroll; u++) {
            TQ q[4];
#pragma unroll
            for (int e = 0; e < 4; e++) q[e] = quantize_one<TQ>(to_f32(v[u][e]), scale, bias);
            store4(out + (i + u * kEwThreads) * kEwVec, q);
        }
    } else {
        for (size_t k = i; k < nvec && k < i + kEwUnroll * kEwThreads; k += kEwThreads) {
            TIn v[4];
            TQ q[4];
            load4(in + k * kEwVec, v);
#pragma unroll
            for (int e = 0; e < 4; e++) q[e] = quantize_one<TQ>(to_f32(v[e]), scale, bias);
            store4(out + k * kEwVec, q);
        }
    }
    for (size_t j = nvec * kEwVec + tid; j < count; j += nthreads) out[j] = quantize_one<TQ>(to_f32(in[j]), scale, bias);
}

template <typename TOut> __device__ __forceinline__ TOut from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
// (the fp32 value is hidden from the optimiser first: where it sees the multiply that produced it, it may merge
// multiply and conversion into one mixed-precision instruction that rounds once, and does so in some copies of a
// loop body and not in others; the result is defined as the fp16 nearest to the rounded fp32 product)
template <> __device__ __forceinline__ __half from_f32<__half>(float v) {
    asm volatile("" : "+v"(v));
    return __float2half_rn(v);
}

template <typename TQ, typename TOut>
__global__ __launch_bounds__(kEwThreads) void dequantize_kernel(const TQ *__restrict__ in, TOut *__restrict__ out,
                                                                size_t count, float scale, float bias, int vec_ok) {
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    const size_t nvec = vec_ok ? count / kEwVec : 0;
    const size_t i = (size_t)blockIdx.x * (kEwUnroll * kEwThreads) + threadIdx.x;
    if (i + (kEwUnroll - 1) * kEwThreads < nvec) {
        TQ v[kEwUnroll][4];
#pragma unroll
        for (int u = 0; u < kEwUnroll; u++) load4(in + (i + u * kEwThreads) * kEwVec, v[u]);
#pragma unroll
        for (int u = 0; u < kEwUnroll; u++) {
            TOut y[4];
#pragma unroll
            for (int e = 0; e < 4; e++) y[e] = from_f32<TOut>(((float)v[u][e] - bias) * scale);
            store4(out + (i + u * kEwThreads) * kEwVec, y);
        }
    } else {
        for (size_t k = i; k < nvec && k < i + kEwUnroll * kEwThreads; k += kEwThreads) {
            TQ v[4];
            TOut y[4];
            load4(in + k * kEwVec, v);
#pragma unroll
            for (int e = 0; e < 4; e++) y[e] = from_f32<TOut>(((float)v[e] - bias) * scale);
            store4(out + k * kEwVec, y);
        }
    }
    for (size_t j = nvec * kEwVec + tid; j < count; j += nthreads) out[j] = from_f32<TOut>(((float)in[j] - bias) * scale);
}

// Strided forms: element `index` of a tensor of `rank` dimensions is read at sum(index[d] * in_strides[d]) and
// written at sum(index[d] * out_strides[d]) (strides in elements), as the reference's kernels address their
// operands (apply(in_shape, ...) with offset(strides, index), reference/quantize.cpp:36-47, dequantize.cpp:36-44).
// One element per thread and trip, innermost dimension fastest, so dense inner rows still coalesce.
constexpr int kMaxStridedRank = 6;
struct StridedArgs {
    int rank;
    uint32_t count;
    FastDiv dim[kMaxStridedRank];          // innermost first
    uint32_t in_stride[kMaxStridedRank];   // innermost first
    uint32_t out_stride[kMaxStridedRank];
};

__device__ __forceinline__ void strided_offsets(const StridedArgs &a, uint32_t i, uint32_t *in_off, uint32_t *out_off) {
    uint32_t io = 0, oo = 0;
#pragma unroll
    for (int d = 0; d < kMaxStridedRank; d++) {
        if (d < a.rank) {
            const uint32_t q = fastdiv(i, a.dim[d]);
            const uint32_t r = i - q * a.dim[d].div;
            io += r * a.in_stride[d];
            oo += r * a.out_stride[d];
            i = q;
        }
    }
    *in_off = io, *out_off = oo;
}

template <typename TIn, typename TQ>
__global__ __launch_bounds__(kEwThreads) void quantize_strided_kernel(const TIn *__restrict__ in, TQ *__restrict__ out, const StridedArgs a,
                                                                      float scale, float bias) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < a.count; i += gridDim.x * blockDim.x) {
        uint32_t io, oo;
        strided_offsets(a, i, &io, &oo);
        out[oo] = quantize_one<TQ>(to_f32(in[io]), scale, bias);
    }
}

template <typename TQ, typename TOut>
__global__ __launch_bounds__(kEwThreads) void dequantize_strided_kernel(const TQ *__restrict__ in, TOut *__restrict__ out, const StridedArgs a,
                                                                        float scale, float bias) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < a.count; i += gridDim.x * blockDim.x) {
        uint32_t io, oo;
        strided_offsets(a, i, &io, &oo);
        out[oo] = from_f32<TOut>(((float)in[io] - bias) * scale);
    }
}

// out = Q(clamp(DQ(a) + DQ(b))) on bytes; the clamp and the u8 saturation are folded into
// one clamp on the requantised value, the division is the exact FMA form (see qconv.hpp).
__global__ __launch_bounds__(kEwThreads) void qadd_kernel(const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                          uint8_t *__restrict__ out, size_t count, float za, float sa,
                                                          float zb, float sb, const Epilogue ep, int vec_ok) {
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t nthreads = (size_t)gridDim.x * blockDim.x;
    // the requantised sum before rounding to a byte
    auto value = [&](uint32_t qa, uint32_t qb) -> float {
        const float fa = ((float)qa - za) * sa;
        const float fb = ((float)qb - zb) * sb;
        return __builtin_amdgcn_fmed3f(div_rn(fa + fb, ep.sy, ep.rsy) + ep.zy, ep.qlo, ep.qhi);
    };
    auto one = [&](uint32_t qa, uint32_t qb) -> uint32_t { return __builtin_amdgcn_cvt_pk_u8_f32(value(qa, qb), 0, 0u); };
    // 16 bytes per thread per step
    const size_t nvec = vec_ok ? count / 16 : 0;
    for (size_t i = tid; i < nvec; i += nthreads) {
        const uint4 va = *reinterpret_cast<const uint4 *>(a + i * 16);
        const uint4 vb = *reinterpret_cast<const uint4 *>(b + i * 16);
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
        uint32_t wo[4];
#pragma unroll
        for (int d = 0; d < 4; d++) {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) w = __builtin_amdgcn_cvt_pk_u8_f32(value((wa[d] >> (8 * e)) & 0xffu, (wb[d] >> (8 * e)) & 0xffu), e, w);
            wo[d] = w;
        }
        *reinterpret_cast<uint4 *>(out + i * 16) = uint4{wo[0], wo[1], wo[2], wo[3]};
    }
    for (size_t j = nvec * 16 + tid; j < count; j += nthreads) out[j] = (uint8_t)one(a[j], b[j]);
}

// Global average pool over NHWC u8.  One thread per (image, channel): the sum
// runs over the pixels in (y, x) order with a float accumulator, exactly the
// order of the reference's window loop, so the result is bit-identical.
// Adjacent threads read adjacent channels, so every load is coalesced.
__global__ __launch_bounds__(kEwThreads) void qglobal_avgpool_kernel(const uint8_t *__restrict__ x,
                                                                     uint8_t *__restrict__ out, int batch, int hw,
                                                                     int channels, float zx, float sx, float zy,
                                                                     float sy) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= batch * channels) return;
    const int n = idx / channels, c = idx - n * channels;
    const uint8_t *p = x + (size_t)n * hw * channels + c;
    float value = 0.f;
    for (int i = 0; i < hw; i++) value = value + ((float)p[(size_t)i * channels] - zx) * sx;
    const float mean = value / (float)hw;
    float t = mean / sy + zy;
    t = fminf(fmaxf(t, 0.f), 255.f);
    out[idx] = (uint8_t)(int32_t)rintf(t);
}

// The same for 4 adjacent channels per thread (dword loads), the loads of 64 pixels (a whole 7x7 map) issued before
// their values are added: with one or two waves per SIMD the kernel is a chain of memory round trips, and this
// leaves one per 64 pixels.  Each channel's additions keep their order.
__global__ __launch_bounds__(kEwThreads) void qglobal_avgpool4_kernel(const uint8_t *__restrict__ x, uint8_t *__restrict__ out,
                                                                      int batch, int hw, int channels, float zx, float sx,
                                                                      float zy, float sy) {
    const int cq = channels >> 2;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= batch * cq) return;
    const int n = idx / cq, c = (idx - n * cq) * 4;
    const uint32_t q = global_avgpool4(x + (size_t)n * hw * channels + c, hw, channels, zx, sx, zy, sy);
    *reinterpret_cast<uint32_t *>(out + (size_t)n * channels + c) = q;
}

inline int ew_grid(const nncase_hip_ctx *ctx, size_t work_items) {
    size_t blocks = (work_items + kEwThreads - 1) / kEwThreads;
    const size_t cap = (size_t)ctx->compute_units * 16; // 16 blocks of 4 waves per CU
    if (blocks > cap) blocks = cap;
    if (blocks == 0) blocks = 1;
    return (int)blocks;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Quantize / dequantize: a block per kEwUnroll * kEwThreads neighbouring vectors, however many that makes.  Blocks that
// run at the same time then read and write neighbouring addresses (measured on 100 M elements against a capped grid that
// strides over the tensor: quantize f32 -> u8 114 -> 96 us, dequantize i32 -> f32 202 -> 136 us).  Without vectors (an
// unaligned buffer) the capped grid walks the elements.
inline int ew_block_grid(const nncase_hip_ctx *ctx, size_t count, bool vec_ok) {
    if (!vec_ok) return ew_grid(ctx, count);
    const size_t per_block = (size_t)kEwUnroll * kEwThreads * kEwVec;
    return (int)std::max<size_t>(1, (count + per_block - 1) / per_block);
}

template <typename TIn, typename TQ>
int launch_quantize(nncase_hip_ctx *ctx, const void *in, void *out, size_t count, float scale, float bias) {
    const int vec_ok = aligned16(in) && aligned16(out);
    const int grid = ew_block_grid(ctx, count, vec_ok);
    hipLaunchKernelGGL((quantize_kernel<TIn, TQ>), dim3(grid), dim3(kEwThreads), 0, ctx->stream, (const TIn *)in,
                       (TQ *)out, count, scale, bias, vec_ok);
    NNHIP_LAUNCH_CHECK(ctx, "quantize_kernel");
    return 0;
}

template <typename TQ, typename TOut>
int launch_dequantize(nncase_hip_ctx *ctx, const void *in, void *out, size_t count, float scale, float bias) {
    const int vec_ok = aligned16(in) && aligned16(out);
    const int grid = ew_block_grid(ctx, count, vec_ok);
    hipLaunchKernelGGL((dequantize_kernel<TQ, TOut>), dim3(grid), dim3(kEwThreads), 0, ctx->stream, (const TQ *)in,
                       (TOut *)out, count, scale, bias, vec_ok);
    NNHIP_LAUNCH_CHECK(ctx, "dequantize_kernel");
    return 0;
}

// Validates a strided operand pair and fills the kernel's arguments.  *dense is set when both sides are the
// plain row-major layout of the shape (the caller then takes the vector kernels).
int make_strided(nncase_hip_ctx *ctx, const char *what, int32_t rank, const int64_t *shape, const int64_t *in_strides,
                 const int64_t *out_strides, StridedArgs *a, bool *dense) {
    NNHIP_REQUIRE(ctx, rank >= 1 && rank <= kMaxStridedRank, -EINVAL, "%s: rank %d (1..%d are supported)", what, rank, kMaxStridedRank);
    NNHIP_REQUIRE(ctx, shape && in_strides && out_strides, -EINVAL, "%s: null shape or strides", what);
    memset(a, 0, sizeof(*a));
    a->rank = rank;
    int64_t count = 1, in_extent = 0, out_extent = 0, row_major = 1;
    *dense = true;
    for (int d = rank - 1; d >= 0; d--) { // innermost first
        NNHIP_REQUIRE(ctx, shape[d] >= 0 && in_strides[d] >= 0 && out_strides[d] >= 0, -EINVAL, "%s: negative extent or stride", what);
        NNHIP_REQUIRE(ctx, shape[d] < ((int64_t)1 << 31) && in_strides[d] < ((int64_t)1 << 31) && out_strides[d] < ((int64_t)1 << 31),
                      -EINVAL, "%s: extent or stride of 2^31 or more", what);
        count *= shape[d];
        NNHIP_REQUIRE(ctx, count < ((int64_t)1 << 31), -EINVAL, "%s: 2^31 elements or more", what);
        if (shape[d] > 0) {
            in_extent += (shape[d] - 1) * in_strides[d];
            out_extent += (shape[d] - 1) * out_strides[d];
        }
        NNHIP_REQUIRE(ctx, in_extent < ((int64_t)1 << 31) && out_extent < ((int64_t)1 << 31), -EINVAL, "%s: operand spans 2^31 elements or more", what);
        const int k = rank - 1 - d;
        a->dim[k] = make_fastdiv((uint32_t)std::max<int64_t>(shape[d], 1));
        a->in_stride[k] = (uint32_t)in_strides[d];
        a->out_stride[k] = (uint32_t)out_strides[d];
        if (shape[d] != 1 && (in_strides[d] != row_major || out_strides[d] != row_major)) *dense = false;
        row_major *= shape[d];
    }
    a->count = (uint32_t)count;
    return 0;
}

} // namespace nnhip

using namespace nnhip;

extern "C" int nncase_hip_quantize(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev,
                                   int out_dtype, size_t count, nncase_hip_quant_param_t qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, (in_dev && out_dev) || count == 0, -EINVAL, "quantize: null buffer");
    NNHIP_REQUIRE(ctx, qp.scale != 0.f, -EINVAL, "quantize: scale is zero");
    if (count == 0) return 0;
    const float bias = (float)qp.zero_point;
#define NNHIP_Q_CASE(IN_DT, TIn, OUT_DT, TQ)                                                                           \
    if (in_dtype == IN_DT && out_dtype == OUT_DT)                                                                      \
    return launch_quantize<TIn, TQ>(ctx, in_dev, out_dev, count, qp.scale, bias)
    NNHIP_Q_CASE(NNCASE_HIP_DT_F32, float, NNCASE_HIP_DT_U8, uint8_t);
    NNHIP_Q_CASE(NNCASE_HIP_DT_F32, float, NNCASE_HIP_DT_I8, int8_t);
    NNHIP_Q_CASE(NNCASE_HIP_DT_F32, float, NNCASE_HIP_DT_I16, int16_t);
    NNHIP_Q_CASE(NNCASE_HIP_DT_F16, __half, NNCASE_HIP_DT_U8, uint8_t);
    NNHIP_Q_CASE(NNCASE_HIP_DT_F16, __half, NNCASE_HIP_DT_I8, int8_t);
    NNHIP_Q_CASE(NNCASE_HIP_DT_F16, __half, NNCASE_HIP_DT_I16, int16_t);
#undef NNHIP_Q_CASE
    return fail(ctx, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "quantize: unsupported types in=0x%x out=0x%x", in_dtype,
                out_dtype);
}

extern "C" int nncase_hip_dequantize(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev,
                                     int out_dtype, size_t count, nncase_hip_quant_param_t qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, (in_dev && out_dev) || count == 0, -EINVAL, "dequantize: null buffer");
    if (count == 0) return 0;
    const float bias = (float)qp.zero_point;
#define NNHIP_DQ_CASE(IN_DT, TQ, OUT_DT, TOut)                                                                         \
    if (in_dtype == IN_DT && out_dtype == OUT_DT)                                                                      \
    return launch_dequantize<TQ, TOut>(ctx, in_dev, out_dev, count, qp.scale, bias)
    NNHIP_DQ_CASE(NNCASE_HIP_DT_U8, uint8_t, NNCASE_HIP_DT_F32, float);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_I8, int8_t, NNCASE_HIP_DT_F32, float);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_I16, int16_t, NNCASE_HIP_DT_F32, float);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_I32, int32_t, NNCASE_HIP_DT_F32, float);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_U8, uint8_t, NNCASE_HIP_DT_F16, __half);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_I8, int8_t, NNCASE_HIP_DT_F16, __half);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_I16, int16_t, NNCASE_HIP_DT_F16, __half);
    NNHIP_DQ_CASE(NNCASE_HIP_DT_I32, int32_t, NNCASE_HIP_DT_F16, __half);
#undef NNHIP_DQ_CASE
    return fail(ctx, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "dequantize: unsupported types in=0x%x out=0x%x", in_dtype,
                out_dtype);
}

extern "C" int nncase_hip_quantize_strided(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev, int out_dtype,
                                           int32_t rank, const int64_t *shape, const int64_t *in_strides, const int64_t *out_strides,
                                           nncase_hip_quant_param_t qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, qp.scale != 0.f, -EINVAL, "quantize: scale is zero");
    StridedArgs a;
    bool dense;
    const int rc = make_strided(ctx, "quantize", rank, shape, in_strides, out_strides, &a, &dense);
    if (rc) return rc;
    if (a.count == 0) return 0;
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "quantize: null buffer");
    if (dense) return nncase_hip_quantize(ctx, in_dev, in_dtype, out_dev, out_dtype, a.count, qp);
    const float bias = (float)qp.zero_point;
    const int grid = ew_grid(ctx, a.count);
#define NNHIP_QS_CASE(IN_DT, TIn, OUT_DT, TQ)                                                                          \
    if (in_dtype == IN_DT && out_dtype == OUT_DT) {                                                                    \
        hipLaunchKernelGGL((quantize_strided_kernel<TIn, TQ>), dim3(grid), dim3(kEwThreads), 0, ctx->stream,           \
                           (const TIn *)in_dev, (TQ *)out_dev, a, qp.scale, bias);                                     \
        NNHIP_LAUNCH_CHECK(ctx, "quantize_strided_kernel");                                                            \
        return 0;                                                                                                      \
    }
    NNHIP_QS_CASE(NNCASE_HIP_DT_F32, float, NNCASE_HIP_DT_U8, uint8_t)
    NNHIP_QS_CASE(NNCASE_HIP_DT_F32, float, NNCASE_HIP_DT_I8, int8_t)
    NNHIP_QS_CASE(NNCASE_HIP_DT_F32, float, NNCASE_HIP_DT_I16, int16_t)
    NNHIP_QS_CASE(NNCASE_HIP_DT_F16, __half, NNCASE_HIP_DT_U8, uint8_t)
    NNHIP_QS_CASE(NNCASE_HIP_DT_F16, __half, NNCASE_HIP_DT_I8, int8_t)
    NNHIP_QS_CASE(NNCASE_HIP_DT_F16, __half, NNCASE_HIP_DT_I16, int16_t)
#undef NNHIP_QS_CASE
    return fail(ctx, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "quantize: unsupported types in=0x%x out=0x%x", in_dtype, out_dtype);
}

extern "C" int nncase_hip_dequantize_strided(nncase_hip_ctx_t *ctx, const void *in_dev, int in_dtype, void *out_dev, int out_dtype,
                                             int32_t rank, const int64_t *shape, const int64_t *in_strides, const int64_t *out_strides,
                                             nncase_hip_quant_param_t qp) {
    NNHIP_CHECK_CTX(ctx);
    StridedArgs a;
    bool dense;
    const int rc = make_strided(ctx, "dequantize", rank, shape, in_strides, out_strides, &a, &dense);
    if (rc) return rc;
    if (a.count == 0) return 0;
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "dequantize: null buffer");
    if (dense) return nncase_hip_dequantize(ctx, in_dev, in_dtype, out_dev, out_dtype, a.count, qp);
    const float bias = (float)qp.zero_point;
    const int grid = ew_grid(ctx, a.count);
#define NNHIP_DQS_CASE(IN_DT, TQ, OUT_DT, TOut)                                                                        \
    if (in_dtype == IN_DT && out_dtype == OUT_DT) {                                                                    \
        hipLaunchKernelGGL((dequantize_strided_kernel<TQ, TOut>), dim3(grid), dim3(kEwThreads), 0, ctx->stream,        \
                           (const TQ *)in_dev, (TOut *)out_dev, a, qp.scale, bias);                                    \
        NNHIP_LAUNCH_CHECK(ctx, "dequantize_strided_kernel");                                                          \
        return 0;                                                                                                      \
    }
    NNHIP_DQS_CASE(NNCASE_HIP_DT_U8, uint8_t, NNCASE_HIP_DT_F32, float)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_I8, int8_t, NNCASE_HIP_DT_F32, float)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_I16, int16_t, NNCASE_HIP_DT_F32, float)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_I32, int32_t, NNCASE_HIP_DT_F32, float)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_U8, uint8_t, NNCASE_HIP_DT_F16, __half)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_I8, int8_t, NNCASE_HIP_DT_F16, __half)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_I16, int16_t, NNCASE_HIP_DT_F16, __half)
    NNHIP_DQS_CASE(NNCASE_HIP_DT_I32, int32_t, NNCASE_HIP_DT_F16, __half)
#undef NNHIP_DQS_CASE
    return fail(ctx, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "dequantize: unsupported types in=0x%x out=0x%x", in_dtype, out_dtype);
}

extern "C" int nncase_hip_qadd(nncase_hip_ctx_t *ctx, const uint8_t *a_dev, nncase_hip_quant_param_t a_qp,
                               const uint8_t *b_dev, nncase_hip_quant_param_t b_qp, uint8_t *out_dev,
                               nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max, size_t count) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, (a_dev && b_dev && out_dev) || count == 0, -EINVAL, "qadd: null buffer");
    if (count == 0) return 0;
    NNHIP_REQUIRE(ctx, std::isfinite(a_qp.scale) && std::isfinite(b_qp.scale) && std::fabs(a_qp.scale) <= 0x1p20f &&
                           std::fabs(b_qp.scale) <= 0x1p20f,
                  -ERANGE, "qadd: input scale outside the supported range");
    Epilogue ep;
    // the sum's magnitude is bounded by 255 * (|sa| + |sb|); mult is unused here
    const int rc = make_epilogue(ctx, &ep, 1.f, 1.f, y_qp, clamp_min, clamp_max, NNCASE_HIP_DT_U8, "qadd");
    if (rc) return rc;
    const int vec_ok = aligned16(a_dev) && aligned16(b_dev) && aligned16(out_dev);
    const int grid = ew_grid(ctx, (count + 15) / 16);
    hipLaunchKernelGGL(qadd_kernel, dim3(grid), dim3(kEwThreads), 0, ctx->stream, a_dev, b_dev, out_dev, count,
                       (float)a_qp.zero_point, a_qp.scale, (float)b_qp.zero_point, b_qp.scale, ep, vec_ok);
    NNHIP_LAUNCH_CHECK(ctx, "qadd_kernel");
    return 0;
}

extern "C" int nncase_hip_qglobal_avgpool(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, uint8_t *out_dev, int32_t batch,
                                          int32_t h, int32_t w, int32_t channels, nncase_hip_quant_param_t x_qp,
                                          nncase_hip_quant_param_t y_qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && out_dev, -EINVAL, "qglobal_avgpool: null buffer");
    NNHIP_REQUIRE(ctx, batch > 0 && h > 0 && w > 0 && channels > 0, -EINVAL, "qglobal_avgpool: bad shape");
    NNHIP_REQUIRE(ctx, (int64_t)batch * channels < (int64_t)1 << 31, -EINVAL, "qglobal_avgpool: too large");
    NNHIP_REQUIRE(ctx, y_qp.scale != 0.f, -EINVAL, "qglobal_avgpool: output scale is zero");
    if (channels % 4 == 0 && (reinterpret_cast<uintptr_t>(x_dev) & 3u) == 0 && (reinterpret_cast<uintptr_t>(out_dev) & 3u) == 0) {
        const int total4 = batch * (channels / 4);
        hipLaunchKernelGGL(qglobal_avgpool4_kernel, dim3((total4 + kEwThreads - 1) / kEwThreads), dim3(kEwThreads), 0, ctx->stream,
                           x_dev, out_dev, batch, h * w, channels, (float)x_qp.zero_point, x_qp.scale, (float)y_qp.zero_point,
                           y_qp.scale);
        NNHIP_LAUNCH_CHECK(ctx, "qglobal_avgpool4_kernel");
        return 0;
    }
    const int total = batch * channels;
    hipLaunchKernelGGL(qglobal_avgpool_kernel, dim3((total + kEwThreads - 1) / kEwThreads), dim3(kEwThreads), 0,
                       ctx->stream, x_dev, out_dev, batch, h * w, channels, (float)x_qp.zero_point, x_qp.scale,
                       (float)y_qp.zero_point, y_qp.scale);
    NNHIP_LAUNCH_CHECK(ctx, "qglobal_avgpool_kernel");
    return 0;
}
