// Entry points of the u8/u8 convolution and matmul: argument checks, shape
// inference and dispatch to the MFMA implicit-GEMM kernel or the depthwise
// streaming kernel.
#include "qconv.hpp"

#include <algorithm>
#include <cmath>
#include <mutex>
#include <new>
#include <utility>
#include <vector>

namespace nnhip {
int prepack_igemm(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw, const int32_t *bias);
int prepack_depthwise(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw, const int32_t *bias);
} // namespace nnhip

using namespace nnhip;

void nnhip::describe_conv_kernel(const nncase_hip_ctx *ctx, const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *a,
                                 char *buf, size_t cap) {
    if (w->kind == nncase_hip_weights::kDepthwise) {
        if (depthwise_uses_3x3(w, a)) snprintf(buf, cap, "dw3x3<S=%d>", a->stride_h);
        else snprintf(buf, cap, "dw_generic<VEC=%d>", w->out_channels % 4 == 0 ? 4 : 1);
        return;
    }
    if (w->d_smallc && a->dilation_h == 1 && a->dilation_w == 1 && !a->residual_dev && !w->d_post_lut && !a->dequantize_output &&
        !a->out_channel_stride) {
        snprintf(buf, cap, "qconv_smallc<C=%d>", w->in_channels);
        return;
    }
    static const char *modes[] = {"rows16", "vec16", "vec8", "vec4", "bytes", "rows8"};
    const int out_h = windowed_output_size(a->in_h, w->kernel_h, a->stride_h, a->dilation_h, a->pad_h_before, a->pad_h_after);
    const int out_w = windowed_output_size(a->in_w, w->kernel_w, a->stride_w, a->dilation_w, a->pad_w_before, a->pad_w_after);
    if (rows_path_taken(w, a, out_h, out_w)) {
        snprintf(buf, cap, "qpointwise_rows%s%s", w->d_post_lut ? "+lut" : "", a->dequantize_output ? "+dequantize" : "");
        return;
    }
    const long long m = (long long)a->batch * out_h * out_w;
    const int mode = igemm_load_mode(w, a, out_h, out_w);
    const int mi = (int)std::min<long long>(m, 1 << 30);
    if (w->wide) {
        snprintf(buf, cap, "qconv_wide%s%s%s<T=%d,%s%s>", w->d_post_lut ? "+lut" : "", a->residual_dev ? "+add" : "",
                 a->dequantize_output ? "+dequantize" : "", w->tiles,
                 w->wide == 2 ? "RG=2," : "", modes[mode]);
        return;
    }
    snprintf(buf, cap, "qconv_igemm%s%s%s<T=%d,RG=%d,%s>", w->d_post_lut ? "+lut" : "", a->residual_dev ? "+add" : "",
             a->dequantize_output ? "+dequantize" : "", w->tiles,
             igemm_pixel_groups(ctx, w, mi), modes[mode]);
}

float nnhip::reciprocal_rn(float b) {
    float best = (float)(1.0 / (double)b);
    // the product of two floats is exact in double, so |1 - b * r| ranks the candidates exactly
    double err = std::fabs(1.0 - (double)b * (double)best);
    const float cand[2] = {std::nextafterf(best, INFINITY), std::nextafterf(best, -INFINITY)};
    for (float c : cand) {
        const double e = std::fabs(1.0 - (double)b * (double)c);
        if (e < err) {
            err = e;
            best = c;
        }
    }
    return best;
}

namespace {

// Host emulation of the device's two requantisation forms (same single IEEE operations).
inline int requant_ref(int32_t v, const nnhip::Epilogue &ep) {
    volatile float f = (float)v * ep.mult;
    volatile float t = f / ep.sy; // what div_rn returns: the correctly rounded quotient
    volatile float u = t + ep.zy;
    float c = std::fmin(std::fmax((float)u, ep.qlo), ep.qhi);
    return (int)std::nearbyintf(c);
}
inline int requant_fma(int32_t v, float c1, float c2, const nnhip::Epilogue &ep) {
    const float u = std::fmaf((float)v, c1, c2);
    float c = std::fmin(std::fmax(u, ep.qlo), ep.qhi);
    return (int)std::nearbyintf(c);
}

// The magic-bias form (Epilogue::magic) on accumulator v; -1 where kMagicBias + v is no positive finite float.
inline int requant_magic(int64_t v, float m1, float m2, const nnhip::Epilogue &ep) {
    const int64_t bits = (int64_t)nnhip::kMagicBias + v;
    if (bits <= 0 || bits >= 0x7f800000) return -1;
    const uint32_t b = (uint32_t)bits;
    float x;
    memcpy(&x, &b, sizeof(x));
    const float u = std::fmaf(x, m1, m2);
    float c = std::fmin(std::fmax(u, ep.qlo), ep.qhi);
    return (int)std::nearbyintf(c);
}
// Accumulators the magic-bias form is vouched for: every |acc| up to this bound (far more than a reduction of
// 16 384 products of bytes plus a bias can reach; kMagicBias + acc stays a positive finite float up to 8.7e8).
constexpr int32_t kMagicLimit = 800000000;

// Both forms are monotone non-decreasing step functions of the accumulator, so they are equal everywhere iff
// they agree at both ends of the int32 range and on both sides of every step of the reference form.
void find_fast_requant(nnhip::Epilogue *ep) {
    ep->fast = 0;
    ep->c1 = ep->c2 = 0.f;
    ep->magic = 0;
    ep->m1 = ep->m2 = 0.f;
    ep->magic_limit = 0;
    if (!(ep->mult > 0.f) || !(ep->sy > 0.f)) return;
    const int32_t vmin = INT32_MIN + 1, vmax = INT32_MAX;
    const int rmin = requant_ref(vmin, *ep), rmax = requant_ref(vmax, *ep);
    // steps[k - rmin - 1] = smallest accumulator whose code is >= k
    std::vector<int32_t> steps;
    steps.reserve(256);
    int32_t lo = vmin;
    for (int k = rmin + 1; k <= rmax; k++) {
        int64_t a = lo, b = vmax; // requant_ref(a) < k <= requant_ref(b)
        while (b - a > 1) {
            const int64_t m = a + (b - a) / 2;
            if (requant_ref((int32_t)m, *ep) >= k) b = m;
            else a = m;
        }
        steps.push_back((int32_t)b);
        lo = (int32_t)a;
    }
    auto matches = [&](float c1, float c2) {
        if (requant_fma(vmin, c1, c2, *ep) != rmin || requant_fma(vmax, c1, c2, *ep) != rmax) return false;
        for (size_t i = 0; i < steps.size(); i++) {
            const int k = rmin + 1 + (int)i;
            // several codes can share one step when the accumulator scale is coarse
            if (requant_fma(steps[i], c1, c2, *ep) != requant_ref(steps[i], *ep)) return false;
            if (requant_fma(steps[i] - 1, c1, c2, *ep) != requant_ref(steps[i] - 1, *ep)) return false;
            (void)k;
        }
        return true;
    };
    const float c1_0 = (float)((double)ep->mult / (double)ep->sy);
    if (!std::isfinite(c1_0) || c1_0 <= 0.f) return;
    // The magic-bias pair: m1 near the nominal slope with its two lowest mantissa bits clear, so that 12582912 * m1
    // (a product with 3 * 2^22) is exact in fp32 and m2 = zy - 12582912 * m1 can be too; the map is then
    // RN(acc * m1 + zy) in one rounding.  Checked like the pair below, over the accumulator range it is used for.
    {
        auto magic_matches = [&](float m1, float m2) {
            if (requant_magic(-(int64_t)kMagicLimit, m1, m2, *ep) != requant_ref(-kMagicLimit, *ep)) return false;
            if (requant_magic(kMagicLimit, m1, m2, *ep) != requant_ref(kMagicLimit, *ep)) return false;
            for (size_t i = 0; i < steps.size(); i++) {
                if (requant_magic(steps[i], m1, m2, *ep) != requant_ref(steps[i], *ep)) return false;
                if (requant_magic((int64_t)steps[i] - 1, m1, m2, *ep) != requant_ref(steps[i] - 1, *ep)) return false;
            }
            return true;
        };
        uint32_t bits;
        memcpy(&bits, &c1_0, sizeof(bits));
        for (int k = 0; k <= 12 && !ep->magic; k++)
            for (int sgn = 1; sgn >= -1 && !ep->magic; sgn -= 2) {
                if (k == 0 && sgn < 0) continue;
                const uint32_t cb = (bits & ~3u) + (uint32_t)(sgn * 4 * k);
                float m1;
                memcpy(&m1, &cb, sizeof(m1));
                if (!(m1 > 0.f) || !std::isfinite(m1)) continue;
                const double m2d = (double)ep->zy - 12582912.0 * (double)m1;
                const float m2 = (float)m2d;
                if ((double)m2 != m2d) continue; // not representable: the sum would be rounded twice
                if (magic_matches(m1, m2)) {
                    ep->m1 = m1, ep->m2 = m2, ep->magic = 1, ep->magic_limit = kMagicLimit;
                }
            }
    }
    // nominal constants first, then small perturbations of both (the reference's own rounding noise decides a
    // few steps that sit almost exactly on an integer accumulator)
    for (int ring = 0; ring <= 24; ring++)
        for (int i = -ring; i <= ring; i++)
            for (int j = -ring; j <= ring; j++) {
                if (std::max(std::abs(i), std::abs(j)) != ring) continue;
                float c1 = c1_0;
                for (int s = 0; s < std::abs(i); s++) c1 = std::nextafterf(c1, i > 0 ? INFINITY : 0.f);
                const float c2 = ep->zy + (float)j * 0x1p-18f;
                if (matches(c1, c2)) {
                    ep->c1 = c1;
                    ep->c2 = c2;
                    ep->fast = 1;
                    return;
                }
            }
}

struct EpilogueKey {
    float mult, sy, zy, lo, hi;
    bool operator==(const EpilogueKey &o) const { return memcmp(this, &o, sizeof(*this)) == 0; }
};
// The search costs a few hundred thousand float operations; the same layer is set up again on every eager call.
struct EpilogueCache {
    std::mutex mu;
    std::vector<std::pair<EpilogueKey, nnhip::Epilogue>> entries;
};
EpilogueCache g_epilogues;

} // namespace

int nnhip::make_epilogue(nncase_hip_ctx *ctx, Epilogue *ep, float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min,
                         float clamp_max, int out_dtype, const char *who) {
    ep->mult = sx * sw;
    ep->lo = clamp_min;
    ep->hi = clamp_max;
    ep->sy = y_qp.scale;
    ep->zy = (float)y_qp.zero_point;
    ep->rsy = 1.f;
    ep->qlo = 0.f;
    ep->qhi = 255.f;
    ep->c1 = ep->c2 = 0.f;
    ep->fast = 0;
    ep->full = 1;
    ep->m1 = ep->m2 = 0.f;
    ep->magic = 0;
    ep->magic_limit = 0;
    ep->out_mode = out_dtype == NNCASE_HIP_DT_U8 ? kOutU8 : (out_dtype == NNCASE_HIP_DT_I32 ? kOutI32 : kOutF32);
    NNHIP_REQUIRE(ctx, !(clamp_min > clamp_max), -EINVAL, "%s: fused clamp minimum above maximum", who);
    if (ep->out_mode != kOutU8) return 0;
    NNHIP_REQUIRE(ctx, y_qp.zero_point >= 0 && y_qp.zero_point <= 255, -EINVAL, "%s: output zero point %d outside u8", who,
                  y_qp.zero_point);
    // Range in which q0 = f * rsy and the residual f - sy * q0 stay normal for every f whose
    // requantised value is not already pinned to an end of [0, 255].
    NNHIP_REQUIRE(ctx, ep->sy >= 0x1p-64f && ep->sy <= 0x1p64f, -ERANGE, "%s: output scale %g outside [2^-64, 2^64]", who,
                  (double)ep->sy);
    NNHIP_REQUIRE(ctx, std::isfinite(ep->mult) && std::fabs(ep->mult) <= 0x1p64f &&
                           std::fabs((double)ep->mult) / (double)ep->sy <= 0x1p64,
                  -ERANGE, "%s: input scale * weight scale = %g outside the supported range", who, (double)ep->mult);
    ep->rsy = reciprocal_rn(ep->sy);
    // g(v) = RN(RN(v / sy) + zy), evaluated with the same single fp32 operations as the device
    volatile float glo = clamp_min / ep->sy;
    glo = glo + ep->zy;
    volatile float ghi = clamp_max / ep->sy;
    ghi = ghi + ep->zy;
    ep->qlo = std::fmin(std::fmax((float)glo, 0.f), 255.f);
    ep->qhi = std::fmin(std::fmax((float)ghi, 0.f), 255.f);
    ep->full = std::nearbyintf(ep->qlo) == 0.f && std::nearbyintf(ep->qhi) == 255.f;
    {
        const EpilogueKey key{ep->mult, ep->sy, ep->zy, ep->lo, ep->hi};
        std::lock_guard<std::mutex> lock(g_epilogues.mu);
        for (const auto &e : g_epilogues.entries)
            if (e.first == key) {
                ep->c1 = e.second.c1, ep->c2 = e.second.c2, ep->fast = e.second.fast;
                ep->m1 = e.second.m1, ep->m2 = e.second.m2, ep->magic = e.second.magic, ep->magic_limit = e.second.magic_limit;
                return 0;
            }
        find_fast_requant(ep);
        if (g_epilogues.entries.size() >= 4096) g_epilogues.entries.clear();
        g_epilogues.entries.emplace_back(key, *ep);
    }
    return 0;
}

int nnhip::make_residual_epilogue(nncase_hip_ctx *ctx, ResidualEpilogue *rep, const nncase_hip_conv2d_args_t *c,
                                  const nncase_hip_weights *w) {
    memset(rep, 0, sizeof(*rep));
    rep->res = c->residual_dev;
    if (!c->residual_dev) return 0;
    NNHIP_REQUIRE(ctx, c->out_dtype == NNCASE_HIP_DT_U8, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                  "qconv2d: a fused residual needs u8 output");
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(c->residual_dev) & 15u) == 0, -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION,
                  "qconv2d: residual buffer must be 16-byte aligned");
    NNHIP_REQUIRE(ctx, std::isfinite(c->y_qp.scale) && std::isfinite(c->residual_qp.scale) &&
                           std::fabs(c->y_qp.scale) <= 0x1p20f && std::fabs(c->residual_qp.scale) <= 0x1p20f,
                  -ERANGE, "qconv2d: residual input scale outside the supported range");
    // the residual stage dequantises what the first stage produced: the table's output if there is one
    const nncase_hip_quant_param_t own = (w && w->d_post_lut) ? w->post_lut_qp : c->y_qp;
    rep->zy = (float)own.zero_point;
    rep->sy = own.scale;
    rep->zr = (float)c->residual_qp.zero_point;
    rep->sr = c->residual_qp.scale;
    return make_epilogue(ctx, &rep->sum, 1.f, 1.f, c->sum_qp, c->sum_clamp_min, c->sum_clamp_max, NNCASE_HIP_DT_U8,
                         "qconv2d(residual)");
}

static void free_weights(nncase_hip_weights *w) {
    if (!w) return;
    if (w->d_packed) (void)hipFree(w->d_packed);
    if (w->d_wsum) (void)hipFree(w->d_wsum);
    if (w->d_bias) (void)hipFree(w->d_bias);
    if (w->d_smallc) (void)hipFree(w->d_smallc);
    if (w->d_post_lut) (void)hipFree(w->d_post_lut);
    rows_free(w);
    delete w;
}

extern "C" int nncase_hip_requant_plan(float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max, float *c1,
                                       float *c2) {
    Epilogue ep;
    const int rc = make_epilogue(nullptr, &ep, sx, sw, y_qp, clamp_min, clamp_max, NNCASE_HIP_DT_U8, "requant_plan");
    if (rc) return rc;
    if (c1) *c1 = ep.c1;
    if (c2) *c2 = ep.c2;
    return ep.fast;
}

extern "C" int nncase_hip_requant_host(float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max,
                                       const int32_t *acc_host, size_t count, uint8_t *out_host, int32_t *form_used) {
    if (!acc_host || !out_host) return -EINVAL;
    Epilogue ep;
    const int rc = make_epilogue(nullptr, &ep, sx, sw, y_qp, clamp_min, clamp_max, NNCASE_HIP_DT_U8, "requant_host");
    if (rc) return rc;
    if (form_used) *form_used = ep.fast;
    for (size_t i = 0; i < count; i++)
        out_host[i] = (uint8_t)(ep.fast ? requant_fma(acc_host[i], ep.c1, ep.c2, ep) : requant_ref(acc_host[i], ep));
    return 0;
}

extern "C" int nncase_hip_requant_host_magic(float sx, float sw, nncase_hip_quant_param_t y_qp, float clamp_min, float clamp_max,
                                             const int32_t *acc_host, size_t count, uint8_t *out_host, float *m1, float *m2,
                                             int32_t *limit) {
    if (count && (!acc_host || !out_host)) return -EINVAL;
    Epilogue ep;
    const int rc = make_epilogue(nullptr, &ep, sx, sw, y_qp, clamp_min, clamp_max, NNCASE_HIP_DT_U8, "requant_host_magic");
    if (rc) return rc;
    if (!ep.magic) return 0;
    if (m1) *m1 = ep.m1;
    if (m2) *m2 = ep.m2;
    if (limit) *limit = ep.magic_limit;
    for (size_t i = 0; i < count; i++) {
        const int64_t v = acc_host[i];
        out_host[i] = (v < -(int64_t)ep.magic_limit || v > ep.magic_limit) ? 0 : (uint8_t)requant_magic(v, ep.m1, ep.m2, ep);
    }
    return 1;
}

extern "C" int nncase_hip_qconv2d_prepack(nncase_hip_ctx_t *ctx, const nncase_hip_conv2d_desc_t *desc,
                                          const uint8_t *weights_oihw_host, const int32_t *bias_host,
                                          nncase_hip_weights_t **weights) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, desc && weights_oihw_host && weights, -EINVAL, "qconv2d_prepack: null argument");
    *weights = nullptr;
    NNHIP_REQUIRE(ctx, desc->in_channels > 0 && desc->out_channels > 0 && desc->kernel_h > 0 && desc->kernel_w > 0,
                  -EINVAL, "qconv2d_prepack: non-positive dimension");
    NNHIP_REQUIRE(ctx, desc->groups > 0 && desc->in_channels % desc->groups == 0 &&
                           desc->out_channels % desc->groups == 0,
                  -NNCASE_HIP_ERR_SHAPE_MISMATCH, "qconv2d_prepack: groups=%d does not divide channels %d/%d",
                  desc->groups, desc->in_channels, desc->out_channels);
    NNHIP_REQUIRE(ctx, desc->w_qp.zero_point >= 0 && desc->w_qp.zero_point <= 255, -EINVAL,
                  "qconv2d_prepack: weight zero point %d outside u8", desc->w_qp.zero_point);
    nncase_hip_weights *w = new (std::nothrow) nncase_hip_weights();
    NNHIP_REQUIRE(ctx, w, -ENOMEM, "qconv2d_prepack: out of host memory");
    w->in_channels = desc->in_channels;
    w->out_channels = desc->out_channels;
    w->kernel_h = desc->kernel_h;
    w->kernel_w = desc->kernel_w;
    w->groups = desc->groups;
    w->g_ic = desc->in_channels / desc->groups;
    w->g_oc = desc->out_channels / desc->groups;
    w->zw = desc->w_qp.zero_point;
    w->sw = desc->w_qp.scale;
    w->pixels_hint = desc->expected_pixels > 0 ? desc->expected_pixels : 0;
    const bool depthwise = desc->groups > 1 && w->g_ic == 1 && w->g_oc == 1;
    w->kind = depthwise ? nncase_hip_weights::kDepthwise : nncase_hip_weights::kIgemm;
    NNHIP_HIP(ctx, hipSetDevice(ctx->device));
    int rc = depthwise ? prepack_depthwise(ctx, w, weights_oihw_host, bias_host)
                       : prepack_igemm(ctx, w, weights_oihw_host, bias_host);
    if (rc == 0 && !depthwise && smallc_supported(w)) rc = prepack_smallc(ctx, w, weights_oihw_host);
    if (rc == 0 && !depthwise) rc = rows_prepack(ctx, w, weights_oihw_host);
    if (rc) {
        free_weights(w);
        return rc;
    }
    *weights = w;
    return 0;
}

extern "C" int nncase_hip_weights_destroy(nncase_hip_ctx_t *ctx, nncase_hip_weights_t *weights) {
    NNHIP_CHECK_CTX(ctx);
    if (!weights) return 0;
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    free_weights(weights);
    return 0;
}

extern "C" int nncase_hip_weights_set_post_lut(nncase_hip_ctx_t *ctx, nncase_hip_weights_t *w, const uint8_t *lut256_host,
                                               nncase_hip_quant_param_t table_qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, w, -EINVAL, "weights_set_post_lut: null weights");
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream)); // earlier launches may still read the old table
    if (!lut256_host) {
        if (w->d_post_lut) (void)hipFree(w->d_post_lut);
        w->d_post_lut = nullptr;
        return 0;
    }
    NNHIP_REQUIRE(ctx, w->kind == nncase_hip_weights::kIgemm, -EINVAL,
                  "weights_set_post_lut: a fused table is only supported by the dense (MFMA) kernels");
    if (!w->d_post_lut) NNHIP_HIP(ctx, hipMalloc((void **)&w->d_post_lut, 256));
    NNHIP_HIP(ctx, hipMemcpy(w->d_post_lut, lut256_host, 256, hipMemcpyHostToDevice));
    w->post_lut_qp = table_qp;
    return 0;
}

static int check_out_dtype(nncase_hip_ctx *ctx, int dt, nncase_hip_quant_param_t y_qp, const char *who) {
    NNHIP_REQUIRE(ctx, dt == NNCASE_HIP_DT_U8 || dt == NNCASE_HIP_DT_I32 || dt == NNCASE_HIP_DT_F32,
                  -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "%s: unsupported output type 0x%x", who, dt);
    if (dt == NNCASE_HIP_DT_U8) {
        NNHIP_REQUIRE(ctx, y_qp.scale > 0.f && std::isfinite(y_qp.scale), -EINVAL, "%s: output scale must be positive", who);
        NNHIP_REQUIRE(ctx, y_qp.zero_point >= 0 && y_qp.zero_point <= 255, -EINVAL, "%s: output zero point %d outside u8",
                      who, y_qp.zero_point);
    }
    return 0;
}

extern "C" int nncase_hip_qconv2d(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_weights_t *w, void *y_dev,
                                  const nncase_hip_conv2d_args_t *a) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && w && y_dev && a, -EINVAL, "qconv2d: null argument");
    NNHIP_REQUIRE(ctx, a->batch > 0 && a->in_h > 0 && a->in_w > 0, -EINVAL, "qconv2d: non-positive input shape");
    NNHIP_REQUIRE(ctx, a->stride_h > 0 && a->stride_w > 0 && a->dilation_h > 0 && a->dilation_w > 0, -EINVAL,
                  "qconv2d: stride and dilation must be positive");
    NNHIP_REQUIRE(ctx, a->pad_h_before >= 0 && a->pad_h_after >= 0 && a->pad_w_before >= 0 && a->pad_w_after >= 0, -EINVAL,
                  "qconv2d: negative padding");
    NNHIP_REQUIRE(ctx, a->x_qp.zero_point >= 0 && a->x_qp.zero_point <= 255, -EINVAL,
                  "qconv2d: input zero point %d outside u8", a->x_qp.zero_point);
    nncase_hip_conv2d_args_t through_u8;
    if (a->dequantize_output != 0) {
        // the u8 result, stored as its float32 value: the kernels see a u8 call with the flag set
        NNHIP_REQUIRE(ctx, a->out_dtype == NNCASE_HIP_DT_F32, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                      "qconv2d: dequantize_output needs out_dtype float32");
        NNHIP_REQUIRE(ctx, w->kind == nncase_hip_weights::kIgemm && a->out_channel_stride == 0 && a->out_channel_offset == 0, -EINVAL,
                      "qconv2d: dequantize_output is only supported by the dense (MFMA) kernels, with a dense output");
        through_u8 = *a;
        through_u8.out_dtype = NNCASE_HIP_DT_U8;
        a = &through_u8;
    }
    int rc = check_out_dtype(ctx, a->out_dtype, a->y_qp, "qconv2d");
    if (rc) return rc;
    const int out_h = windowed_output_size(a->in_h, w->kernel_h, a->stride_h, a->dilation_h, a->pad_h_before, a->pad_h_after);
    const int out_w = windowed_output_size(a->in_w, w->kernel_w, a->stride_w, a->dilation_w, a->pad_w_before, a->pad_w_after);
    NNHIP_REQUIRE(ctx, out_h > 0 && out_w > 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH, "qconv2d: window larger than padded input");
    if (rows_path_taken(w, a, out_h, out_w)) return launch_qconv_rows(ctx, x_dev, w, y_dev, a, nullptr);
    if (a->out_channel_stride != 0 || a->out_channel_offset != 0) {
        NNHIP_REQUIRE(ctx, w->kind == nncase_hip_weights::kIgemm, -EINVAL,
                      "qconv2d: an output inside a wider tensor is only supported by the dense (MFMA) kernels");
        if (!a->residual_dev && !w->d_post_lut) return launch_qconv_igemm(ctx, x_dev, w, y_dev, a, out_h, out_w);
    }
    if (a->dequantize_output != 0 && !a->residual_dev && !w->d_post_lut) return launch_qconv_igemm(ctx, x_dev, w, y_dev, a, out_h, out_w);
    if (a->residual_dev || w->d_post_lut) {
        if (a->residual_dev) {
            rc = check_out_dtype(ctx, NNCASE_HIP_DT_U8, a->sum_qp, "qconv2d(residual)");
            if (rc) return rc;
            NNHIP_REQUIRE(ctx, a->out_dtype == NNCASE_HIP_DT_U8, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                          "qconv2d: a fused residual needs u8 output");
        }
        NNHIP_REQUIRE(ctx, w->kind == nncase_hip_weights::kIgemm, -EINVAL,
                      "qconv2d: a fused table or residual is only supported by the dense (MFMA) kernels");
        return launch_qconv_igemm(ctx, x_dev, w, y_dev, a, out_h, out_w);
    }
    if (w->kind == nncase_hip_weights::kDepthwise) return launch_qconv_depthwise(ctx, x_dev, w, y_dev, a, out_h, out_w);
    if (w->d_smallc && a->dilation_h == 1 && a->dilation_w == 1) return launch_qconv_smallc(ctx, x_dev, w, y_dev, a, out_h, out_w);
    return launch_qconv_igemm(ctx, x_dev, w, y_dev, a, out_h, out_w);
}

extern "C" int nncase_hip_qmatmul_prepack(nncase_hip_ctx_t *ctx, const uint8_t *b_host, int32_t k, int32_t n,
                                          nncase_hip_quant_param_t b_qp, const int32_t *bias_host, int64_t expected_rows,
                                          nncase_hip_weights_t **weights) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, b_host && weights, -EINVAL, "qmatmul_prepack: null argument");
    NNHIP_REQUIRE(ctx, k > 0 && n > 0, -EINVAL, "qmatmul_prepack: non-positive dimension");
    // B[K,N] row-major is a 1x1 convolution's OIHW weight [N,K,1,1] transposed.
    std::vector<uint8_t> bt((size_t)k * n);
    for (int kk = 0; kk < k; kk++)
        for (int j = 0; j < n; j++) bt[(size_t)j * k + kk] = b_host[(size_t)kk * n + j];
    nncase_hip_conv2d_desc_t d;
    d.in_channels = k;
    d.out_channels = n;
    d.kernel_h = d.kernel_w = 1;
    d.groups = 1;
    d.w_qp = b_qp;
    d.expected_pixels = expected_rows;
    return nncase_hip_qconv2d_prepack(ctx, &d, bt.data(), bias_host, weights);
}

extern "C" int nncase_hip_qmatmul(nncase_hip_ctx_t *ctx, const uint8_t *a_dev, const nncase_hip_weights_t *w, void *y_dev,
                                  const nncase_hip_matmul_args_t *m) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, a_dev && w && y_dev && m, -EINVAL, "qmatmul: null argument");
    NNHIP_REQUIRE(ctx, m->m > 0, -EINVAL, "qmatmul: non-positive row count");
    NNHIP_REQUIRE(ctx, w->kind == nncase_hip_weights::kIgemm && w->kernel_h == 1 && w->kernel_w == 1 && w->groups == 1,
                  -NNCASE_HIP_ERR_SHAPE_MISMATCH, "qmatmul: weights were not packed by qmatmul_prepack");
    nncase_hip_conv2d_args_t c;
    memset(&c, 0, sizeof(c));
    c.batch = 1;
    c.in_h = m->m;
    c.in_w = 1;
    c.stride_h = c.stride_w = c.dilation_h = c.dilation_w = 1;
    c.x_qp = m->a_qp;
    c.y_qp = m->y_qp;
    c.clamp_min = m->clamp_min;
    c.clamp_max = m->clamp_max;
    c.out_dtype = m->out_dtype;
    return nncase_hip_qconv2d(ctx, a_dev, w, y_dev, &c);
}

extern "C" int nncase_hip_qglobal_avgpool_qconv2d(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, int32_t h, int32_t w_,
                                                  nncase_hip_quant_param_t x_qp, const nncase_hip_weights_t *w, void *y_dev,
                                                  const nncase_hip_conv2d_args_t *a) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && w && y_dev && a, -EINVAL, "qglobal_avgpool_qconv2d: null argument");
    NNHIP_REQUIRE(ctx, a->batch > 0 && h > 0 && w_ > 0 && a->in_h == 1 && a->in_w == 1, -EINVAL,
                  "qglobal_avgpool_qconv2d: the convolution reads one pooled pixel per image");
    NNHIP_REQUIRE(ctx, x_qp.zero_point >= 0 && x_qp.zero_point <= 255 && a->x_qp.zero_point >= 0 && a->x_qp.zero_point <= 255 &&
                           a->x_qp.scale != 0.f,
                  -EINVAL, "qglobal_avgpool_qconv2d: quantisation outside u8");
    nncase_hip_conv2d_args_t through_u8;
    if (a->dequantize_output != 0) {
        NNHIP_REQUIRE(ctx, a->out_dtype == NNCASE_HIP_DT_F32, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                      "qglobal_avgpool_qconv2d: dequantize_output needs out_dtype float32");
        through_u8 = *a;
        through_u8.out_dtype = NNCASE_HIP_DT_U8;
        a = &through_u8;
    }
    const int rc = check_out_dtype(ctx, a->out_dtype, a->y_qp, "qglobal_avgpool_qconv2d");
    if (rc) return rc;
    NNHIP_REQUIRE(ctx, rows_path_taken(w, a, 1, 1), -EINVAL,
                  "qglobal_avgpool_qconv2d: needs a dense 1x1 convolution packed for a few pixels (expected_pixels = batch at pre-pack "
                  "time), u8 or dequantised output, no residual");
    const PoolFront pool{h * w_, x_qp};
    return launch_qconv_rows(ctx, x_dev, w, y_dev, a, &pool);
}

extern "C" int nncase_hip_qglobal_avgpool_qconv2d_supported(const nncase_hip_weights_t *w, const nncase_hip_conv2d_args_t *a, int32_t h,
                                                            int32_t w_) {
    if (!w || !a || a->in_h != 1 || a->in_w != 1 || h <= 0 || w_ <= 0 || a->batch <= 0) return 0;
    if (!pool_front_pays(a->batch, h * w_, w->in_channels)) return 0;
    return rows_path_taken(w, a, 1, 1) ? 1 : 0;
}
