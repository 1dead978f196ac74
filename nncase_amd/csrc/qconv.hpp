// Pre-packed constant block shared by the u8/u8 convolution / matmul kernels.
#pragma once

#include "common.hpp"

struct nncase_hip_weights {
    enum Kind { kIgemm = 0, kDepthwise = 1 };
    int kind = kIgemm;
    int in_channels = 0, out_channels = 0, kernel_h = 0, kernel_w = 0, groups = 1;
    int g_ic = 0, g_oc = 0; // channels per group
    int k = 0;              // reduction length per group: kernel_h * kernel_w * g_ic
    int ksteps = 0;         // ceil(k / 64)
    int tiles = 0;          // 16-channel MFMA tiles per channel chunk (T)
    int nchunks = 0;        // channel chunks per group
    int kc_steps = 0;       // k-steps staged in LDS at a time
    // igemm, reductions of at most 32: the spare half of the only k-step holds -(zw - 128) against a second copy
    // of the activations, which makes the weight zero point's share of the product part of the multiplication
    int fold = 0;
    // igemm: packed for the wide-tile kernels (qconv_wide.hpp): 1 = long reductions over many pixels and channels
    // (blocks of 256 or 128 pixels, waves of 64), 2 = reductions of five k-steps and more over fewer pixels (blocks of
    // 128 pixels x 64 channels or 64 x 32, waves of 32 pixels)
    int wide = 0;
    long long dw_const_bound = 0; // depthwise: max over channels of |bias| + 255 |sum(w - zw)|
    long long bias_absmax = 0;    // largest |bias|
    int64_t pixels_hint = 0; // output pixels per call the tiling was planned for (0 = unknown)
    int32_t zw = 0;
    float sw = 1.f;
    // igemm: [groups][nchunks][ksteps][tiles] fragments of 1024 bytes (s8, MFMA operand order)
    // depthwise: [kernel_h * kernel_w][channels] int16 (w - zw)
    void *d_packed = nullptr;
    uint32_t *d_post_lut = nullptr; // optional fused unary operator: 256-entry byte table (dense kernels)
    nncase_hip_quant_param_t post_lut_qp{0, 1.f};
    int32_t *d_wsum = nullptr; // igemm: sum_k (w ^ 0x80 as s8) per out channel; depthwise: sum_t (w - zw)
    int32_t *d_bias = nullptr; // [out_channels]
    size_t packed_bytes = 0;
    // few-input-channel 3x3 convolutions also carry a [oc][k] s8 layout for the per-pixel dot-product kernel
    void *d_smallc = nullptr;
    size_t smallc_bytes = 0;
    // dense 1x1 convolutions planned for a handful of pixels (a classifier head, a batch-1 matmul) also carry the
    // weights in the order of the kernel that keeps them in registers (qpair.hip: second convolution only)
    struct nncase_hip_qpair *rows_pack = nullptr;
};

namespace nnhip {

// Output forms of the conv / matmul epilogue.
enum OutMode { kOutU8 = 0, kOutI32 = 1, kOutF32 = 2 };

// Parameters of the fused epilogue  acc -> fp32 -> clamp -> requantise.
//   f = (float)acc * mult
//   F32 output: clamp(f, lo, hi)
//   U8  output: sat_u8(rne(clamp(f, lo, hi) / sy + zy))
// g(v) = RN(RN(v / sy) + zy) is monotone non-decreasing, so it commutes with the
// clamp and the two clamps fold into one on g(f):
//   clamp(g(clamp(f, lo, hi)), 0, 255) = clamp(g(f), qlo, qhi),
//   qlo = clamp(g(lo), 0, 255), qhi = clamp(g(hi), 0, 255)      (computed on the host)
struct Epilogue {
    float mult;     // sx * sw
    float lo, hi;   // fused clamp on the fp32 value (F32 output)
    float sy, rsy;  // output scale and its correctly rounded reciprocal
    float zy;
    float qlo, qhi; // clamp on the requantised value before rounding to an integer
    int out_mode;
    // One-instruction form of the same map (U8 output): the requantised code is a monotone step function of
    // the int32 accumulator, and the host looks for constants with which
    //   RN(fma((float)acc, c1, c2))
    // steps at exactly the same accumulators as the three-rounding sequence above (make_epilogue checks
    // every step of the staircase, so the bytes are identical); fast == 0 when no such pair was found.
    float c1, c2;
    int fast;
    int full; // rne(qlo) == 0 and rne(qhi) == 255: the saturating conversion to u8 is the whole clamp
    // The same form on an accumulator that was started from kMagicBias: while |acc| < 2^22 the bits of
    // kMagicBias + acc, read as a float, ARE the float 12582912 + acc, so the int -> float conversion disappears:
    //   RN(fma(as_float(kMagicBias + acc), m1, m2)),  m2 = zy - 12582912 * m1 exactly (m1 has two spare mantissa bits).
    // Beyond 2^22 the float keeps growing with the accumulator (positive floats order like their bit patterns), which
    // is all the proof needs: both maps are monotone, and make_epilogue checks them equal at every step of the
    // staircase and at both ends of the accumulator range [-magic_limit, magic_limit] it vouches for.
    float m1, m2;
    int magic;            // 0: no such pair was found
    int32_t magic_limit;  // largest |acc| the equality was established for
};
constexpr int32_t kMagicBias = 0x4B400000; // the bits of 12582912.0f = 1.5 * 2^23

// Second requantisation stage of a fused residual add:
//   s = ((float)q - zy) * sy + ((float)r - zr) * sr;   out = sat_u8(rne(clamp(s) / sum.sy + sum.zy))
struct ResidualEpilogue {
    const uint8_t *res; // nullptr: no residual
    float zy, sy;       // dequantisation of the convolution's own u8 result
    float zr, sr;       // dequantisation of the residual
    Epilogue sum;       // requantisation of the sum (mult unused)
};

// Fills an Epilogue; returns 0 or a negative error for scales outside the range in
// which the division-free requantisation is exact.
int make_residual_epilogue(nncase_hip_ctx *ctx, ResidualEpilogue *rep, const nncase_hip_conv2d_args_t *c,
                           const nncase_hip_weights *w);
int make_epilogue(nncase_hip_ctx *ctx, Epilogue *ep, float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min,
                  float clamp_max, int out_dtype, const char *who);

// RN(1 / b) for a finite positive b, exactly (the double quotient is corrected by
// comparing exact residuals of the neighbouring floats).
float reciprocal_rn(float b);

int launch_qconv_igemm(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                       const nncase_hip_conv2d_args_t *a, int out_h, int out_w);
int launch_qconv_smallc(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                        const nncase_hip_conv2d_args_t *a, int out_h, int out_w);
bool smallc_supported(const nncase_hip_weights *w);
int prepack_smallc(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw);
int launch_qconv_depthwise(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                           const nncase_hip_conv2d_args_t *a, int out_h, int out_w);

// The few-pixel path of a dense 1x1 convolution (qpair.hip): packing at pre-pack time, whether a call takes it, the launch
// (pool != nullptr: x is [batch, pool_hw, channels] and the convolution reads its global average, requantised to c->x_qp).
struct PoolFront {
    int hw;
    nncase_hip_quant_param_t x_qp;
};
bool rows_shapes_ok(int in_channels, int out_channels, int64_t pixels);   // what rows_prepack packs and rows_path_taken takes
bool pool_front_pays(int rows, int hw, int channels);
int rows_prepack(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw);
void rows_free(nncase_hip_weights *w);
bool rows_path_taken(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c, int out_h, int out_w);
int launch_qconv_rows(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y, const nncase_hip_conv2d_args_t *c,
                      const PoolFront *pool);

// Writes the name of the kernel a conv with these weights / arguments launches.
void describe_conv_kernel(const nncase_hip_ctx *ctx, const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *a, char *buf,
                          size_t cap);
int igemm_pixel_groups(const nncase_hip_ctx *ctx, const nncase_hip_weights *w, int m);
int igemm_load_mode(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c, int out_h, int out_w);
} // namespace nnhip
// Writes the name of the kernel a fused block launches.
void nncase_hip_qblock_describe(const nncase_hip_qblock_t *b, const nncase_hip_qblock_args_t *a, char *buf, size_t cap);
namespace nnhip {
bool depthwise_uses_3x3(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c);

// Correctly rounded a / b from b and rb = RN(1 / b): one multiply and two fused
// multiply-adds (Markstein's correction step: the residual a - b*q0 is exact in an
// FMA and q0 + residual * rb rounds to the correctly rounded quotient).  Valid while
// neither the quotient nor the residual leaves the normal range; make_epilogue
// guarantees that for every value whose rounding can matter.
__device__ __forceinline__ float div_rn(float a, float b, float rb) {
    const float q0 = a * rb;
    const float e = __builtin_fmaf(-b, q0, a);
    return __builtin_fmaf(e, rb, q0);
}

// sat_u8(rne(f / sy + zy)) of an fp32 value, returned in the LOW BYTE of the result
// (the other bytes are not zero).  Adding 1.5 * 2^23 makes the fp32 adder perform the
// round-half-even to an integer and leaves that integer in the low mantissa bits.
__device__ __forceinline__ uint32_t requant_u8_lowbyte(float f, const Epilogue &ep) {
    float u = div_rn(f, ep.sy, ep.rsy) + ep.zy;
    u = __builtin_amdgcn_fmed3f(u, ep.qlo, ep.qhi);
    return __float_as_uint(u + 12582912.0f);
}

// The requantised codes of four int32 accumulators, packed as bytes 0..3 of a dword: the one-instruction form
// when the host has proved it equal to the three-rounding sequence for this layer.  v_cvt_pk_u8_f32 rounds to
// the nearest integer (ties to even), saturates to [0, 255] and inserts the byte, so conversion, clamp and
// packing are one instruction per code; rounding is monotone, so a clamp to [qlo, qhi] before it is needed
// only when it is tighter than the saturation.
__device__ __forceinline__ uint32_t requant4_u8_packed(const int32_t (&v)[4], const Epilogue &ep) {
    uint32_t d = 0;
    if (ep.fast) {
        if (ep.full) {
#pragma unroll
            for (int r = 0; r < 4; r++) d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf((float)v[r], ep.c1, ep.c2), r, d);
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int32_t vr = v[r]; // hidden from the optimiser for the reason given below
                asm volatile("" : "+v"(vr));
                const float u = __builtin_fmaf((float)vr, ep.c1, ep.c2);
                d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(u, ep.qlo, ep.qhi), r, d);
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            // (the value is hidden from the optimiser here: sharing its conversion with the branches above, it
            // converts every accumulator of a tile ahead of the branch and keeps them all in registers)
            int32_t vr = v[r];
            asm volatile("" : "+v"(vr));
            const float u = div_rn((float)vr * ep.mult, ep.sy, ep.rsy) + ep.zy;
            d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(u, ep.qlo, ep.qhi), r, d);
        }
    }
    return d;
}

// The same for accumulators already held in fp32 (exact integers).
__device__ __forceinline__ uint32_t requant4_u8_packed(const float (&v)[4], const Epilogue &ep) {
    uint32_t d = 0;
    if (ep.fast) {
        if (ep.full) {
#pragma unroll
            for (int r = 0; r < 4; r++) d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(v[r], ep.c1, ep.c2), r, d);
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++)
                d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(__builtin_fmaf(v[r], ep.c1, ep.c2), ep.qlo, ep.qhi), r, d);
        }
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float u = div_rn(v[r] * ep.mult, ep.sy, ep.rsy) + ep.zy;
            d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(u, ep.qlo, ep.qhi), r, d);
        }
    }
    return d;
}

// The one-instruction-per-code form alone, for kernels that are instantiated separately for layers whose
// epilogue has fast != 0 and full != 0: no branch on the epilogue's flags is left in the instruction stream,
// so the conversions of a row can be scheduled among its stores and the loads of the rows that follow.
template <typename T> __device__ __forceinline__ uint32_t requant4_u8_packed_direct(const T (&v)[4], const Epilogue &ep) {
    uint32_t d = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf((float)v[r], ep.c1, ep.c2), r, d);
    return d;
}

// The magic-bias form: v are accumulators that were started from kMagicBias (see Epilogue::magic).
__device__ __forceinline__ uint32_t requant4_u8_packed_magic(const int32_t (&v)[4], const Epilogue &ep) {
    uint32_t d = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_fmaf(__int_as_float(v[r]), ep.m1, ep.m2), r, d);
    return d;
}

// Packs the low bytes of four dwords into one dword (3 byte-permutes).
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t b0, uint32_t b1, uint32_t b2, uint32_t b3) {
    const uint32_t lo = __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u); // [b0.0, b1.0, 0, 0]
    const uint32_t hi = __builtin_amdgcn_perm(b3, b2, 0x04000c0cu); // [0, 0, b2.0, b3.0]
    return lo | hi;
}

// The four u8 codes of `q` plus the four of `res`, each pair dequantised, added and requantised; packed.
__device__ __forceinline__ uint32_t residual4_packed(uint32_t q, uint32_t res, const ResidualEpilogue &r) {
    uint32_t d = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const float fa = ((float)((q >> (8 * e)) & 0xffu) - r.zy) * r.sy;
        const float fb = ((float)((res >> (8 * e)) & 0xffu) - r.zr) * r.sr;
        const float u = div_rn(fa + fb, r.sum.sy, r.sum.rsy) + r.sum.zy;
        d = __builtin_amdgcn_cvt_pk_u8_f32(__builtin_amdgcn_fmed3f(u, r.sum.qlo, r.sum.qhi), e, d);
    }
    return d;
}

// Global average pool of four adjacent channels of one image (NHWC u8, p at the image's first pixel): the dequantised
// values are added in pixel order with a float accumulator, exactly the order of the reference's reduction loop
// (src/Native/src/kernels/stackvm/reference/reduce.cpp), then mean, requantisation and rounding; the four codes packed.
// The loads of 64 pixels (a whole 7x7 map) are issued before their values are added: one memory round trip per 64.
__device__ __forceinline__ uint32_t global_avgpool4(const uint8_t *p, int hw, int channels, float zx, float sx, float zy, float sy) {
    float value[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i0 = 0; i0 < hw; i0 += 64) {
        uint32_t d[64];
#pragma unroll
        for (int k = 0; k < 64; k++) d[k] = *reinterpret_cast<const uint32_t *>(p + (size_t)min(i0 + k, hw - 1) * channels);
#pragma unroll
        for (int k = 0; k < 64; k++)
            if (i0 + k < hw) {
#pragma unroll
                for (int e = 0; e < 4; e++) value[e] = value[e] + ((float)((d[k] >> (8 * e)) & 0xffu) - zx) * sx;
            }
    }
    uint32_t q = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const float mean = value[e] / (float)hw;
        float t = mean / sy + zy;
        t = fminf(fmaxf(t, 0.f), 255.f);
        q |= (uint32_t)(int32_t)rintf(t) << (8 * e);
    }
    return q;
}

// a + b + c in one instruction (the compiler otherwise re-associates the zero-point
// correction into a subtract and an add).
__device__ __forceinline__ int32_t add3(int32_t a, int32_t b, int32_t c) {
    int32_t d;
    asm("v_add3_u32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// acc + x.i16[H] * w.i16[H] (v_mad_i32_i16 with op_sel picking the 16-bit halves): the
// multiply-add reads both 16-bit halves of a register directly, so activations are kept
// as two zero-extended bytes per register and weights as the int16 pairs they are stored as.
__device__ __forceinline__ int32_t mad16_lo(uint32_t x, uint32_t w, int32_t acc) {
    int32_t d;
    asm("v_mad_i32_i16 %0, %1, %2, %3" : "=v"(d) : "v"(x), "v"(w), "v"(acc));
    return d;
}
__device__ __forceinline__ int32_t mad16_hi(uint32_t x, uint32_t w, int32_t acc) {
    int32_t d;
    asm("v_mad_i32_i16 %0, %1, %2, %3 op_sel:[1,1,0,0]" : "=v"(d) : "v"(x), "v"(w), "v"(acc));
    return d;
}

__device__ __forceinline__ float clamp_ref(float v, float lo, float hi) {
    return __builtin_fmaxf(__builtin_fminf(v, hi), lo);
}

} // namespace nnhip
