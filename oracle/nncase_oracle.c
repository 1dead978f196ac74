/*
 * CPU oracle for the nncase `hip` hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic that nncase's CPU target
 * runs for the operators the HIP library replaces.  It is the checker that
 * the parity tests, the smoke check and the benchmark's CPU-baseline leg
 * call; nothing in the product (the HIP library or its Python host side)
 * may link, import or execute it.
 *
 * Two families of functions live here.
 *
 *  (1) "ref_*": loop-for-loop restatements of the reference's float kernels,
 *      same loop order, same accumulator type, same expression order:
 *        ref_quantize_*      src/Native/src/kernels/stackvm/reference/quantize.cpp:29-43
 *                            (== optimized/quantize.cpp:64-68 on contiguous data)
 *        ref_dequantize_*    .../reference/dequantize.cpp:29-39
 *        ref_conv2d_f32      .../reference/convolution.cpp:26-105,
 *                            output size kernel_utils.h:86-93, clamp :123-130
 *        ref_matmul_f32      .../reference/matmul.cpp:28-48 (unit) and :50-91 (batching)
 *        ref_reduce_window2d_mean_f32
 *                            .../reference/reduce_window.cpp:36-109,133-135
 *        ref_get_quant_param / ref_fixup_range
 *                            src/Nncase.Core/Utilities/QuantUtility.cs:41-97
 *        ref_calib_fixup_range
 *                            src/Nncase.Quantization/Quantization/Quantizer.cs:358-386
 *        ref_f32_to_f16 / ref_f16_to_f32
 *                            src/Native/include/nncase/runtime/half.h:66-140
 *      Pins: quantize/dequantize against the literal vectors of
 *      src/Nncase.Tests/Evaluator/UnitTestEvaluatorMath.cs:455-510 and the tie
 *      and saturation vectors of tests/test_oracle.py; get_quant_param /
 *      fixup_range against the literals of
 *      src/Nncase.Tests/Core/UnitTestQuantUtility.cs:17-37; conv2d / matmul
 *      against float64 numpy/scipy brute force on the reference's own shape
 *      grids; half conversion exhaustively against IEEE binary16.
 *
 *  (2) "q*": the integer-exact definition of the u8/u8 operators, which the
 *      reference only expresses as Dequantize -> float op -> Quantize
 *      (src/Nncase.Importer/Onnx/QLinearConv.cs:61-75, QLinearMatmul.cs:25-28,
 *      src/Nncase.Importer/TFLite/Conv2D.cs:39-98):
 *        acc = sum (x - zx) * (w - zw) + bias          (exact integers)
 *        y   = clamp((float)acc * (sx * sw), lo, hi)   (one fp32 multiply)
 *        q   = sat_u8(rne(y / sy + (float)zy))          (quantize.cpp:37-43)
 *      The reference has no integer accumulator, so the int32 accumulators are
 *      pinned by mathematics only (int64 brute force, zero-point identity,
 *      linearity, extremes); the requantised bytes are additionally
 *      cross-checked to be within 1 LSB of the reference float chain.
 *
 *  (3) paged-attention decode and pack/unpack have no counterpart in the
 *      reference (parity unpinned by the reference): the functions here are
 *      float64 brute-force definitions pinned by closed forms in the tests.
 *
 * Build:  gcc -O2 -fno-fast-math -ffp-contract=off -fPIC -shared \
 *             -o oracle/libnncase_oracle.so oracle/nncase_oracle.c -lm
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

enum { ORACLE_U8 = 0, ORACLE_I8 = 1, ORACLE_I16 = 2 };
enum { ORACLE_OUT_U8 = 0, ORACLE_OUT_I32 = 1, ORACLE_OUT_F32 = 2 };

/* ------------------------------------------------------------------------ */
/* small helpers                                                            */
/* ------------------------------------------------------------------------ */

/* kernel_utils.h:123-125 : clamp(v, lo, hi) = max(min(v, hi), lo), written
 * with the comparison direction std::min / std::max use.                   */
static inline float clampf_ref(float v, float lo, float hi) {
    float t = (hi < v) ? hi : v;
    return (t < lo) ? lo : t;
}

static inline int32_t clampi_ref(int32_t v, int32_t lo, int32_t hi) {
    int32_t t = (hi < v) ? hi : v;
    return (t < lo) ? lo : t;
}

/* kernel_utils.h:86-93 */
static inline int32_t windowed_out(int32_t size, int32_t filter, int32_t stride,
                                   int32_t dilation, int32_t pad_before,
                                   int32_t pad_after) {
    int32_t eff = (filter - 1) * dilation + 1;
    return (size + pad_before + pad_after - eff + stride) / stride;
}

ORACLE_API int32_t oracle_windowed_output_size(int32_t size, int32_t filter,
                                               int32_t stride, int32_t dilation,
                                               int32_t pad_before,
                                               int32_t pad_after) {
    return windowed_out(size, filter, stride, dilation, pad_before, pad_after);
}

/* Round-half-even to an int32 with saturation.  quantize.cpp:38-39 does
 * (int32_t)lrintf(v); that is identical for |v| < 2^31, which is the domain
 * parity is claimed on (beyond it the reference's cast wraps modulo 2^32 on
 * LP64 and is undefined past 2^63; this oracle saturates instead).          */
static inline int32_t rne_sat_i32(float v) {
    if (!(v > -2147483648.0f)) return INT32_MIN; /* also NaN -> INT32_MIN */
    if (v >= 2147483648.0f) return INT32_MAX;
    return (int32_t)lrintf(v);
}

static inline void qrange(int dtype, int32_t *lo, int32_t *hi) {
    switch (dtype) {
    case ORACLE_U8: *lo = 0; *hi = 255; break;
    case ORACLE_I8: *lo = -128; *hi = 127; break;
    default: *lo = -32768; *hi = 32767; break;
    }
}

/* ------------------------------------------------------------------------ */
/* (1) reference float kernels                                              */
/* ------------------------------------------------------------------------ */

/* quantize.cpp:36-43 : value = x / scale + bias; q = clamp(lrintf(value)). */
ORACLE_API int ref_quantize_f32(const float *x, void *out, size_t n, float scale,
                                float bias, int dtype) {
    int32_t lo, hi;
    if (dtype < ORACLE_U8 || dtype > ORACLE_I16) return -1;
    qrange(dtype, &lo, &hi);
    for (size_t i = 0; i < n; i++) {
        float v = x[i];
        v = v / scale + bias;
        int32_t q = clampi_ref(rne_sat_i32(v), lo, hi);
        if (dtype == ORACLE_U8) ((uint8_t *)out)[i] = (uint8_t)q;
        else if (dtype == ORACLE_I8) ((int8_t *)out)[i] = (int8_t)q;
        else ((int16_t *)out)[i] = (int16_t)q;
    }
    return 0;
}

/* The C# Evaluator's order of operations (OrtKI QuantizeLinear, third party,
 * ONNX Runtime semantics): rne(x / scale) + zp, then saturate.  Kept only to
 * document where the reference's two implementations differ (exact .5 ties). */
ORACLE_API int ref_quantize_f32_ort_order(const float *x, void *out, size_t n,
                                          float scale, int32_t zp, int dtype) {
    int32_t lo, hi;
    if (dtype < ORACLE_U8 || dtype > ORACLE_I16) return -1;
    qrange(dtype, &lo, &hi);
    for (size_t i = 0; i < n; i++) {
        float v = x[i] / scale;
        int64_t q = (int64_t)rne_sat_i32(v) + zp;
        if (q < lo) q = lo;
        if (q > hi) q = hi;
        if (dtype == ORACLE_U8) ((uint8_t *)out)[i] = (uint8_t)q;
        else if (dtype == ORACLE_I8) ((int8_t *)out)[i] = (int8_t)q;
        else ((int16_t *)out)[i] = (int16_t)q;
    }
    return 0;
}

/* dequantize.cpp:36-39 : value = ((float)q - bias) * scale. */
ORACLE_API int ref_dequantize_f32(const void *in, float *y, size_t n, float scale,
                                  float bias, int dtype) {
    if (dtype < ORACLE_U8 || dtype > ORACLE_I16) return -1;
    for (size_t i = 0; i < n; i++) {
        float v;
        if (dtype == ORACLE_U8) v = (float)((const uint8_t *)in)[i];
        else if (dtype == ORACLE_I8) v = (float)((const int8_t *)in)[i];
        else v = (float)((const int16_t *)in)[i];
        y[i] = (v - bias) * scale;
    }
    return 0;
}

/* The stride arithmetic the reference performs per element
 * (kernel_utils.h `offset(strides, index)`): a dot product of a 4-entry index
 * with a 4-entry stride vector.  Kept so that the timed CPU baseline does the
 * same work per multiply-accumulate as the reference kernel.               */
static inline size_t dot4(const size_t *s, const size_t *i) {
    return s[0] * i[0] + s[1] * i[1] + s[2] * i[2] + s[3] * i[3];
}

/* convolution.cpp:26-105.  NCHW input, OIHW weights, contiguous tensors.
 * Loop order batch, group, oc, oy, ox | ic, ky, kx; accumulator is a float
 * that starts from the bias; the window is clipped to the image so padding
 * contributes nothing; the fused clamp is applied to the float sum.         */
ORACLE_API int ref_conv2d_f32(const float *input, const float *weights,
                              const float *bias, float *output, int32_t n,
                              int32_t c, int32_t h, int32_t w, int32_t oc_total,
                              int32_t kh, int32_t kw, int32_t stride_h,
                              int32_t stride_w, int32_t pad_h0, int32_t pad_h1,
                              int32_t pad_w0, int32_t pad_w1, int32_t dil_h,
                              int32_t dil_w, int32_t groups, float act_lo,
                              float act_hi) {
    if (groups <= 0 || c % groups || oc_total % groups) return -1;
    const int32_t out_h = windowed_out(h, kh, stride_h, dil_h, pad_h0, pad_h1);
    const int32_t out_w = windowed_out(w, kw, stride_w, dil_w, pad_w0, pad_w1);
    const size_t g_ic = (size_t)(c / groups), g_oc = (size_t)(oc_total / groups);
    const size_t in_st[4] = {(size_t)c * h * w, (size_t)h * w, (size_t)w, 1};
    const size_t w_st[4] = {g_ic * kh * kw, (size_t)kh * kw, (size_t)kw, 1};
    const size_t out_st[4] = {(size_t)oc_total * out_h * out_w,
                              (size_t)out_h * out_w, (size_t)out_w, 1};
    size_t in_ix[4], w_ix[4], out_ix[4];
    for (size_t b = 0; b < (size_t)n; b++) {
        in_ix[0] = out_ix[0] = b;
        for (size_t og = 0; og < (size_t)groups; og++) {
            for (size_t o = 0; o < g_oc; o++) {
                const size_t ochan = og * g_oc + o;
                out_ix[1] = w_ix[0] = ochan;
                for (size_t oy = 0; oy < (size_t)out_h; oy++) {
                    out_ix[2] = oy;
                    for (size_t ox = 0; ox < (size_t)out_w; ox++) {
                        out_ix[3] = ox;
                        const int32_t y0 = (int32_t)oy * stride_h - pad_h0;
                        const int32_t x0 = (int32_t)ox * stride_w - pad_w0;
                        int32_t ky0 = (-y0 + dil_h - 1) / dil_h;
                        if (ky0 < 0) ky0 = 0;
                        int32_t ky1 = (h - y0 + dil_h - 1) / dil_h;
                        if (ky1 > kh) ky1 = kh;
                        int32_t kx0 = (-x0 + dil_w - 1) / dil_w;
                        if (kx0 < 0) kx0 = 0;
                        int32_t kx1 = (w - x0 + dil_w - 1) / dil_w;
                        if (kx1 > kw) kx1 = kw;
                        float value = bias[ochan];
                        for (size_t ic = 0; ic < g_ic; ic++) {
                            in_ix[1] = og * g_ic + ic;
                            w_ix[1] = ic;
                            for (int32_t ky = ky0; ky < ky1; ky++) {
                                w_ix[2] = (size_t)ky;
                                for (int32_t kx = kx0; kx < kx1; kx++) {
                                    w_ix[3] = (size_t)kx;
                                    in_ix[2] = (size_t)(y0 + dil_h * ky);
                                    in_ix[3] = (size_t)(x0 + dil_w * kx);
                                    const float a = input[dot4(in_st, in_ix)];
                                    const float k = weights[dot4(w_st, w_ix)];
                                    value += a * k;
                                }
                            }
                        }
                        output[dot4(out_st, out_ix)] =
                            clampf_ref(value, act_lo, act_hi);
                    }
                }
            }
        }
    }
    return 0;
}

/* matmul.cpp:28-48 */
static void matmul_unit_f32(const float *a, const float *b, float *o,
                            int32_t rows, int32_t inner, int32_t cols) {
    for (int32_t oy = 0; oy < rows; oy++) {
        for (int32_t ox = 0; ox < cols; ox++) {
            float value = 0.0f;
            for (int32_t i = 0; i < inner; i++)
                value += a[oy * inner + i] * b[i * cols + ox];
            o[oy * cols + ox] = value;
        }
    }
}

/* matmul.cpp:50-91.  Shapes are already widened to rank 4 by the caller
 * (rank-1 A gains a leading 1, rank-1 B a trailing 1, then left-pad with 1s);
 * batch and channel dims broadcast when one side is 1.                      */
ORACLE_API int ref_matmul_f32(const float *a, const float *b, float *out,
                              const int32_t a_shape[4], const int32_t b_shape[4]) {
    if (a_shape[3] != b_shape[2]) return -1;
    const size_t a_unit = (size_t)a_shape[2] * a_shape[3];
    const size_t b_unit = (size_t)b_shape[2] * b_shape[3];
    const size_t o_unit = (size_t)a_shape[2] * b_shape[3];
    const int32_t batches = a_shape[0] > b_shape[0] ? a_shape[0] : b_shape[0];
    const int32_t chans = a_shape[1] > b_shape[1] ? a_shape[1] : b_shape[1];
    const size_t ab = a_unit * a_shape[1], bb = b_unit * b_shape[1];
    const size_t ob = o_unit * chans;
    for (int32_t nn = 0; nn < batches; nn++) {
        const size_t an = a_shape[0] == 1 ? 0 : nn, bn = b_shape[0] == 1 ? 0 : nn;
        for (int32_t cc = 0; cc < chans; cc++) {
            const size_t ac = a_shape[1] == 1 ? 0 : cc;
            const size_t bc = b_shape[1] == 1 ? 0 : cc;
            matmul_unit_f32(a + an * ab + ac * a_unit, b + bn * bb + bc * b_unit,
                            out + nn * ob + cc * o_unit, a_shape[2], a_shape[3],
                            b_shape[3]);
        }
    }
    return 0;
}

/* reduce_window.cpp:36-109 with the mean window op (:133-135): sequential
 * float sum over the clipped window in (ky, kx) order, then `pad_count`
 * additions of 0, then division by the element count.                       */
ORACLE_API int ref_reduce_window2d_mean_f32(
    const float *input, float *output, int32_t n, int32_t c, int32_t h, int32_t w,
    int32_t fh, int32_t fw, int32_t stride_h, int32_t stride_w, int32_t pad_h0,
    int32_t pad_h1, int32_t pad_w0, int32_t pad_w1, int32_t count_include_pad,
    float act_lo, float act_hi) {
    const int32_t out_h = windowed_out(h, fh, stride_h, 1, pad_h0, pad_h1);
    const int32_t out_w = windowed_out(w, fw, stride_w, 1, pad_w0, pad_w1);
    for (int32_t b = 0; b < n; b++)
        for (int32_t ch = 0; ch < c; ch++)
            for (int32_t oy = 0; oy < out_h; oy++)
                for (int32_t ox = 0; ox < out_w; ox++) {
                    const int32_t y0 = oy * stride_h - pad_h0;
                    const int32_t x0 = ox * stride_w - pad_w0;
                    int32_t ky0 = -y0 > 0 ? -y0 : 0, ky1 = h - y0 < fh ? h - y0 : fh;
                    int32_t kx0 = -x0 > 0 ? -x0 : 0, kx1 = w - x0 < fw ? w - x0 : fw;
                    float value = 0.0f;
                    int32_t count = 0;
                    for (int32_t ky = ky0; ky < ky1; ky++)
                        for (int32_t kx = kx0; kx < kx1; kx++) {
                            value = value +
                                    input[(((size_t)b * c + ch) * h + (y0 + ky)) * w +
                                          (x0 + kx)];
                            count++;
                        }
                    for (int32_t i = fh * fw - count; i > 0; i--) value = value + 0.0f;
                    if (count_include_pad) count = fh * fw;
                    output[(((size_t)b * c + ch) * out_h + oy) * out_w + ox] =
                        clampf_ref(value / (float)count, act_lo, act_hi);
                }
    return 0;
}

/* QuantUtility.cs:72-97.  All arithmetic is on C# floats. */
ORACLE_API void ref_fixup_range(float lo, float hi, int symmetric, float out[2]) {
    if (symmetric) {
        float r = fmaxf(fmaxf(fabsf(lo), fabsf(hi)), 0.01f);
        out[0] = -r;
        out[1] = r;
        return;
    }
    hi = fmaxf(0.0f, hi);
    lo = fminf(0.0f, lo);
    float r = hi - lo;
    if (r == 0.0f) r = 0.1f;
    else if (r < 0.01f) r = 0.01f;
    out[0] = lo;
    out[1] = lo + r;
}

/* Quantizer.cs:358-386 (the calibrator's own variant). */
ORACLE_API void ref_calib_fixup_range(float lo, float hi, int symmetric,
                                      float out[2]) {
    if (symmetric) {
        float r = fmaxf(0.01f, fmaxf(fabsf(lo), fabsf(hi)));
        out[0] = -r;
        out[1] = r;
        return;
    }
    if (hi < 0.0f) hi = 0.0f;
    if (lo > 0.0f) lo = 0.0f;
    float r = hi - lo;
    if (r < 1e-6f) r = 0.1f;
    out[0] = lo;
    out[1] = lo + r;
}

/* QuantUtility.cs:41-67.  mode: 0 unsigned, 1 signed symmetric, 2 signed
 * asymmetric.  `max - min` is a float subtraction (both operands are C#
 * floats); everything around it is double; Math.Round is half-to-even.      */
ORACLE_API int ref_get_quant_param(float lo, float hi, int bits, int mode,
                                   int32_t *zero_point, float *scale) {
    float r[2];
    double qmin, qmax;
    ref_fixup_range(lo, hi, mode == 1, r);
    switch (mode) {
    case 0: qmin = 0; qmax = (double)((1 << bits) - 1); break;
    case 1: qmin = (double)(-(1 << (bits - 1)) + 1); qmax = (double)((1 << (bits - 1)) - 1); break;
    case 2: qmin = (double)(-(1 << (bits - 1))); qmax = (double)((1 << (bits - 1)) - 1); break;
    default: return -1;
    }
    const float span = r[1] - r[0];
    const double s = (double)span / (qmax - qmin);
    const double b = nearbyint((double)r[0] * (qmin - qmax) / (double)span) + qmin;
    *zero_point = (int32_t)b;
    *scale = (float)s;
    return 0;
}

/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept,
 * NaN -> 0x7e00 with the sign preserved (half.h:95-140).                    */
ORACLE_API uint16_t ref_f32_to_f16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t mag = u & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 or inf */
    const int32_t e = (int32_t)(mag >> 23) - 127;
    if (e < -25) return sign; /* below half the smallest subnormal */
    uint32_t mant = (mag & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift;       /* bits to drop */
    uint32_t base;   /* exponent field contribution */
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }
    else { shift = 13; base = (uint32_t)(e + 15) << 10; mant &= 0x7fffffu; }
    uint32_t kept = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) kept++;
    uint32_t h = base + kept; /* a carry out of the mantissa bumps the exponent */
    if (h >= 0x7c00u) h = 0x7c00u;
    return (uint16_t)(sign | h);
}

ORACLE_API float ref_f16_to_f32(uint16_t hbits) {
    const uint32_t sign = ((uint32_t)hbits & 0x8000u) << 16;
    const uint32_t e = (hbits >> 10) & 0x1fu, m = hbits & 0x3ffu;
    uint32_t u;
    if (e == 0x1fu) u = sign | 0x7f800000u | (m << 13);
    else if (e != 0) u = sign | ((e + 112u) << 23) | (m << 13);
    else if (m == 0) u = sign;
    else {
        float v = (float)m * 5.9604644775390625e-8f; /* m * 2^-24, exact */
        memcpy(&u, &v, 4);
        u |= sign;
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

ORACLE_API void ref_f32_to_f16_array(const float *x, uint16_t *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = ref_f32_to_f16(x[i]);
}
ORACLE_API void ref_f16_to_f32_array(const uint16_t *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = ref_f16_to_f32(x[i]);
}

/* ------------------------------------------------------------------------ */
/* (2) integer-exact u8/u8 operators                                        */
/* ------------------------------------------------------------------------ */

/* acc -> float -> clamp -> quantize, each step a single fp32 operation.    */
static inline uint8_t requant_one(int32_t acc, float m, float lo, float hi,
                                  float sy, float zy) {
    float y = (float)acc * m;
    y = clampf_ref(y, lo, hi);
    float t = y / sy + zy;
    return (uint8_t)clampi_ref(rne_sat_i32(t), 0, 255);
}

ORACLE_API void q_requant_u8(const int32_t *acc, uint8_t *out, size_t n, float sx,
                             float sw, float lo, float hi, float sy, int32_t zy) {
    const float m = sx * sw;
    for (size_t i = 0; i < n; i++)
        out[i] = requant_one(acc[i], m, lo, hi, sy, (float)zy);
}

static inline int store_out(void *out, size_t idx, int64_t acc, int out_mode,
                            float m, float lo, float hi, float sy, float zy) {
    if (acc > INT32_MAX || acc < INT32_MIN) return -2; /* int32 accumulator overflow */
    if (out_mode == ORACLE_OUT_I32) ((int32_t *)out)[idx] = (int32_t)acc;
    else if (out_mode == ORACLE_OUT_F32)
        ((float *)out)[idx] = clampf_ref((float)(int32_t)acc * m, lo, hi);
    else ((uint8_t *)out)[idx] = requant_one((int32_t)acc, m, lo, hi, sy, zy);
    return 0;
}

/* u8/u8 convolution, NCHW / OIHW, any groups (groups == C is depthwise).
 * Padding contributes nothing, i.e. a padded tap has the real value 0, which
 * is the quantised value zx.  out_mode picks int32 accumulators, the clamped
 * fp32 value acc * (sx*sw), or requantised u8.                              */
ORACLE_API int q_conv2d_u8(const uint8_t *x, const uint8_t *wq, const int32_t *bias,
                           void *out, int32_t n, int32_t c, int32_t h, int32_t w,
                           int32_t oc_total, int32_t kh, int32_t kw,
                           int32_t stride_h, int32_t stride_w, int32_t pad_h0,
                           int32_t pad_h1, int32_t pad_w0, int32_t pad_w1,
                           int32_t dil_h, int32_t dil_w, int32_t groups, int32_t zx,
                           float sx, int32_t zw, float sw, int32_t zy, float sy,
                           float act_lo, float act_hi, int out_mode) {
    if (groups <= 0 || c % groups || oc_total % groups) return -1;
    const int32_t out_h = windowed_out(h, kh, stride_h, dil_h, pad_h0, pad_h1);
    const int32_t out_w = windowed_out(w, kw, stride_w, dil_w, pad_w0, pad_w1);
    const int32_t g_ic = c / groups, g_oc = oc_total / groups;
    const float m = sx * sw;
    int err = 0;
    /* Every output element is an exact integer sum of its own: the (image, channel) planes are computed by as
     * many threads as the host offers, which changes no value. */
#pragma omp parallel for collapse(2) schedule(dynamic)
    for (int32_t b = 0; b < n; b++)
        for (int32_t o = 0; o < oc_total; o++) {
            const int32_t g = o / g_oc;
            for (int32_t oy = 0; oy < out_h; oy++)
                for (int32_t ox = 0; ox < out_w; ox++) {
                    int64_t acc = bias ? bias[o] : 0;
                    for (int32_t ic = 0; ic < g_ic; ic++)
                        for (int32_t ky = 0; ky < kh; ky++) {
                            const int32_t iy = oy * stride_h - pad_h0 + ky * dil_h;
                            if (iy < 0 || iy >= h) continue;
                            for (int32_t kx = 0; kx < kw; kx++) {
                                const int32_t ix = ox * stride_w - pad_w0 + kx * dil_w;
                                if (ix < 0 || ix >= w) continue;
                                const int32_t xv =
                                    x[(((size_t)b * c + g * g_ic + ic) * h + iy) * w + ix];
                                const int32_t wv =
                                    wq[(((size_t)o * g_ic + ic) * kh + ky) * kw + kx];
                                acc += (int64_t)(xv - zx) * (wv - zw);
                            }
                        }
                    const size_t idx = (((size_t)b * oc_total + o) * out_h + oy) * out_w + ox;
                    const int rc = store_out(out, idx, acc, out_mode, m, act_lo, act_hi, sy,
                                             (float)zy);
                    if (rc) {
#pragma omp atomic write
                        err = rc;
                    }
                }
        }
    return err;
}

/* u8/u8 matmul: A [M,K] row-major, B [K,N] row-major, optional int32 bias[N]. */
ORACLE_API int q_matmul_u8(const uint8_t *a, const uint8_t *b, const int32_t *bias,
                           void *out, int32_t mm, int32_t kk, int32_t nn, int32_t za,
                           float sa, int32_t zb, float sb, int32_t zy, float sy,
                           float act_lo, float act_hi, int out_mode) {
    const float m = sa * sb;
    for (int32_t i = 0; i < mm; i++)
        for (int32_t j = 0; j < nn; j++) {
            int64_t acc = bias ? bias[j] : 0;
            for (int32_t k = 0; k < kk; k++)
                acc += (int64_t)((int32_t)a[(size_t)i * kk + k] - za) *
                       ((int32_t)b[(size_t)k * nn + j] - zb);
            int rc = store_out(out, (size_t)i * nn + j, acc, out_mode, m, act_lo,
                               act_hi, sy, (float)zy);
            if (rc) return rc;
        }
    return 0;
}

/* u8 + u8 -> u8 through the float domain: Q(DQ(a) + DQ(b)) with the
 * dequantize / quantize formulas above and one float addition
 * (binary add, src/Native/src/kernels/stackvm/reference/binary.cpp).        */
ORACLE_API void q_add_u8(const uint8_t *a, const uint8_t *b, uint8_t *out, size_t n,
                         int32_t za, float sa, int32_t zb, float sb, int32_t zy,
                         float sy, float act_lo, float act_hi) {
    for (size_t i = 0; i < n; i++) {
        float fa = ((float)a[i] - (float)za) * sa;
        float fb = ((float)b[i] - (float)zb) * sb;
        float s = clampf_ref(fa + fb, act_lo, act_hi);
        float t = s / sy + (float)zy;
        out[i] = (uint8_t)clampi_ref(rne_sat_i32(t), 0, 255);
    }
}

/* Global average pool on u8 NCHW: Q(mean(DQ(x))) where mean is the
 * reference's sequential float window sum over (y, x) divided by the count. */
ORACLE_API void q_global_avgpool_u8(const uint8_t *x, uint8_t *out, int32_t n,
                                    int32_t c, int32_t h, int32_t w, int32_t zx,
                                    float sx, int32_t zy, float sy) {
    for (int32_t b = 0; b < n; b++)
        for (int32_t ch = 0; ch < c; ch++) {
            float value = 0.0f;
            const uint8_t *p = x + ((size_t)b * c + ch) * h * w;
            for (int32_t i = 0; i < h * w; i++)
                value = value + ((float)p[i] - (float)zx) * sx;
            float mean = value / (float)(h * w);
            float t = mean / sy + (float)zy;
            out[(size_t)b * c + ch] = (uint8_t)clampi_ref(rne_sat_i32(t), 0, 255);
        }
}

/* Byte tables for u8 -> u8 operators that sit between Dequantize and Quantize
 * (the form a unary op takes in a u8/u8 graph): lut[v] = Q(f(DQ(v))).
 * kind 0: identity (a pure requantisation, what Concat inserts when its
 *         inputs carry different quant params);
 * kind 1: swish / SiLU, x / (1 + exp(-x))
 *         (src/Native/src/kernels/stackvm/reference/activation.cpp:36).       */
ORACLE_API void q_unary_lut_u8(int32_t kind, int32_t zx, float sx, int32_t zy, float sy,
                               uint8_t *lut) {
    for (int v = 0; v < 256; v++) {
        float x = ((float)v - (float)zx) * sx;
        float f = x;
        if (kind == 1) f = x / (1 + expf(-x));
        float t = f / sy + (float)zy;
        lut[v] = (uint8_t)clampi_ref(rne_sat_i32(t), 0, 255);
    }
}

/* Nearest-neighbour resize of an NCHW tensor of `es`-byte elements
 * (src/Native/src/kernels/stackvm/reference/resize_image.cpp:91-139; the
 * coordinate and rounding functions of
 * src/Native/include/nncase/kernels/stackvm/resize_image.h:30-92, scales from
 * src/Native/include/nncase/kernels/kernel_utils.h:224-233).
 * transformation_mode: 0 half_pixel, 1 pytorch_half_pixel, 2 align_corners,
 * 3 asymmetric, 4 tfcrop_and_resize (the kernel passes roi 0, 0);
 * nearest_mode: 0 round_prefer_floor, 1 round_prefer_ceil, 2 floor, 3 ceil.   */
static float resize_coordinate(int32_t mode, float x_resized, float x_scale,
                               float length_resized, float length_original) {
    switch (mode) {
    case 3: return x_resized * x_scale;
    case 1: return length_resized > 1 ? (x_resized + 0.5f) * x_scale - 0.5f : 0.0f;
    case 2:
        return length_resized == 1 ? 0 : x_resized * (length_original - 1) / (length_resized - 1);
    case 4: {
        const float roi_start = 0, roi_end = 0;
        double orig = length_resized > 1
                          ? roi_start * (length_original - 1) +
                                (x_resized * (roi_end - roi_start) * (length_original - 1)) /
                                    (length_resized - 1)
                          : 0.5 * (roi_start + roi_end) * (length_original - 1);
        return (float)orig;
    }
    default: return ((x_resized + 0.5f) * x_scale) - 0.5f;
    }
}

static int64_t resize_nearest_pixel(int32_t mode, float x_original) {
    switch (mode) {
    case 1: return (int64_t)roundf(x_original);
    case 2: return (int64_t)floorf(x_original);
    case 3: return (int64_t)ceilf(x_original);
    default:
        if (x_original == (int64_t)x_original + 0.5f) return (int64_t)floorf(x_original);
        return (int64_t)roundf(x_original);
    }
}

ORACLE_API void ref_resize_nearest(const uint8_t *in, uint8_t *out, int32_t es, int32_t n,
                                   int32_t c, int32_t h, int32_t w, int32_t out_h,
                                   int32_t out_w, int32_t transformation_mode,
                                   int32_t nearest_mode) {
    const int align_corners = transformation_mode == 2;
    float height_scale = (float)h / out_h;
    float width_scale = (float)w / out_w;
    if (align_corners && out_h > 1) height_scale = (float)(h - 1) / (out_h - 1);
    if (align_corners && out_w > 1) width_scale = (float)(w - 1) / (out_w - 1);
    for (int32_t b = 0; b < n; b++)
        for (int32_t oc = 0; oc < c; oc++)
            for (int32_t oy = 0; oy < out_h; oy++) {
                float iy = resize_coordinate(transformation_mode, (float)oy, height_scale,
                                             (float)out_h, (float)h);
                int64_t in_y = resize_nearest_pixel(nearest_mode, iy);
                if (in_y < 0) in_y = 0;
                if (in_y >= h) in_y = h - 1;
                for (int32_t ox = 0; ox < out_w; ox++) {
                    float ix = resize_coordinate(transformation_mode, (float)ox, width_scale,
                                                 (float)out_w, (float)w);
                    int64_t in_x = resize_nearest_pixel(nearest_mode, ix);
                    if (in_x < 0) in_x = 0;
                    if (in_x >= w) in_x = w - 1;
                    const uint8_t *src = in + ((((size_t)b * c + oc) * h + in_y) * w + in_x) * es;
                    uint8_t *dst = out + ((((size_t)b * c + oc) * out_h + oy) * out_w + ox) * es;
                    for (int32_t k = 0; k < es; k++) dst[k] = src[k];
                }
            }
}

/* Max pooling of a u8 NCHW tensor between Dequantize and Quantize:
 * the window loop of reduce_window2d with binary_op = max, init = lowest,
 * window_op = identity (src/Native/src/kernels/stackvm/reference/reduce_window.cpp:35-109):
 * only in-bounds positions are read, then the value 0 is folded in once per
 * position that lies in the padding (:88-91).                                 */
ORACLE_API void q_maxpool_u8(const uint8_t *x, uint8_t *out, int32_t n, int32_t c, int32_t h,
                             int32_t w, int32_t kh, int32_t kw, int32_t sh, int32_t sw,
                             int32_t ph0, int32_t ph1, int32_t pw0, int32_t pw1, int32_t zx,
                             float sx, int32_t zy, float sy) {
    const int32_t out_h = oracle_windowed_output_size(h, kh, sh, 1, ph0, ph1);
    const int32_t out_w = oracle_windowed_output_size(w, kw, sw, 1, pw0, pw1);
    for (int32_t b = 0; b < n; b++)
        for (int32_t ch = 0; ch < c; ch++)
            for (int32_t oy = 0; oy < out_h; oy++)
                for (int32_t ox = 0; ox < out_w; ox++) {
                    const int32_t y0 = oy * sh - ph0, x0 = ox * sw - pw0;
                    const int32_t fy0 = y0 < 0 ? -y0 : 0, fy1 = (h - y0) < kh ? (h - y0) : kh;
                    const int32_t fx0 = x0 < 0 ? -x0 : 0, fx1 = (w - x0) < kw ? (w - x0) : kw;
                    float value = -FLT_MAX;
                    int32_t count = 0;
                    for (int32_t ky = fy0; ky < fy1; ky++)
                        for (int32_t kx = fx0; kx < fx1; kx++) {
                            const uint8_t q = x[(((size_t)b * c + ch) * h + (y0 + ky)) * w + (x0 + kx)];
                            const float v = ((float)q - (float)zx) * sx;
                            value = value > v ? value : v;
                            count++;
                        }
                    for (int32_t i = 0; i < kh * kw - count; i++) value = value > 0.0f ? value : 0.0f;
                    float t = value / sy + (float)zy;
                    out[(((size_t)b * c + ch) * out_h + oy) * out_w + ox] =
                        (uint8_t)clampi_ref(rne_sat_i32(t), 0, 255);
                }
}

/* ------------------------------------------------------------------------ */
/* (3) definitions with no reference counterpart                            */
/* ------------------------------------------------------------------------ */

/* Paged-attention decode, float64 brute force.
 *   q        [B, Hq, D]                      fp16 bits
 *   k_cache  [num_blocks, Hkv, block, D]     fp16 bits
 *   v_cache  [num_blocks, Hkv, block, D]     fp16 bits
 *   block_table [B, max_blocks] int32, ctx_lens [B] int32
 *   out      [B, Hq, D] float64
 * kv head of query head h is h / (Hq / Hkv); logits scaled by `scale`.      */
ORACLE_API int attn_paged_decode_f64(const uint16_t *q, const uint16_t *k_cache,
                                     const uint16_t *v_cache,
                                     const int32_t *block_table,
                                     const int32_t *ctx_lens, double *out, int32_t bsz,
                                     int32_t hq, int32_t hkv, int32_t d,
                                     int32_t block, int32_t max_blocks,
                                     int32_t num_blocks, double scale) {
    if (hkv <= 0 || hq % hkv) return -1;
    const int32_t rep = hq / hkv;
    for (int32_t b = 0; b < bsz; b++) {
        const int32_t len = ctx_lens[b];
        if (len < 0 || len > max_blocks * block) return -1;
        double *logit = (double *)malloc(sizeof(double) * (size_t)(len > 0 ? len : 1));
        if (!logit) return -3;
        for (int32_t hh = 0; hh < hq; hh++) {
            const int32_t kvh = hh / rep;
            double *o = out + ((size_t)b * hq + hh) * d;
            for (int32_t e = 0; e < d; e++) o[e] = 0.0;
            if (len == 0) continue;
            double mx = -INFINITY;
            for (int32_t t = 0; t < len; t++) {
                const int32_t pb = block_table[(size_t)b * max_blocks + t / block];
                if (pb < 0 || pb >= num_blocks) { free(logit); return -1; }
                const uint16_t *kr =
                    k_cache + (((size_t)pb * hkv + kvh) * block + t % block) * d;
                double s = 0.0;
                for (int32_t e = 0; e < d; e++)
                    s += (double)ref_f16_to_f32(q[((size_t)b * hq + hh) * d + e]) *
                         (double)ref_f16_to_f32(kr[e]);
                logit[t] = s * scale;
                if (logit[t] > mx) mx = logit[t];
            }
            double den = 0.0;
            for (int32_t t = 0; t < len; t++) {
                logit[t] = exp(logit[t] - mx);
                den += logit[t];
            }
            for (int32_t t = 0; t < len; t++) {
                const int32_t pb = block_table[(size_t)b * max_blocks + t / block];
                /* V is cached d-major: [block][kv head][d][token in block] */
                const uint16_t *vr = v_cache + ((size_t)pb * hkv + kvh) * d * block + t % block;
                const double p = logit[t] / den;
                for (int32_t e = 0; e < d; e++)
                    o[e] += p * (double)ref_f16_to_f32(vr[(size_t)e * block]);
            }
        }
        free(logit);
    }
    return 0;
}
