// Host side of the implicit-GEMM convolution: weight pre-packing into MFMA
// operand order, the tiling plan, and the launch dispatch.
#include "qconv_wide.hpp"

#include <algorithm>
#include <vector>

namespace nnhip {

static const int kAllowedTiles[] = {1, 2, 3, 4, 5, 6, 8, 9, 10, 12, 16};

static int round_tiles(int t) {
    for (int v : kAllowedTiles)
        if (v >= t) return v;
    return 16;
}

// Chooses the channel-chunk width T (in 16-channel tiles), the number of chunks and the
// LDS staging depth for a reduction of `ksteps` k-steps.  Wide chunks reuse every
// activation fragment for more output channels; narrow ones give more blocks.  With a
// pixel-count hint the widest chunk that still yields about two blocks per compute unit
// (at the smallest pixel tile) is taken; without one, the widest that fits the LDS budget.
// max_tiles bounds T (the byte-gather loader is only built for T <= 4).
static void plan_igemm(int g_oc, int ksteps, int max_tiles, int64_t pixels_hint, int compute_units, int *tiles, int *nchunks,
                       int *kc_steps) {
    const int tt = ceil_div(g_oc, 16);
    const long long target = 2LL * compute_units;
    int best_t = 1, best_kc = std::min(ksteps, kLdsFrags);
    for (int nc = 1; nc <= tt; nc++) {
        if (ceil_div(tt, nc) > 16) continue; // more tiles than the widest kernel
        const int t = round_tiles(ceil_div(tt, nc));
        if (t > max_tiles) continue;
        int kc;
        if (ksteps * t <= kLdsFrags) kc = ksteps;              // whole reduction resident
        else if (ksteps > 12 && t <= 4) kc = kLdsFrags / t;     // long reduction: staged in pieces
        else continue;
        best_t = t;
        best_kc = kc;
        if (pixels_hint <= 0 || t == 1) break;
        if ((long long)ceil_div((int)std::min<int64_t>(pixels_hint, 1 << 30), kWaves * 16) * ceil_div(tt, t) >= target) break;
    }
    *tiles = best_t;
    *nchunks = ceil_div(tt, best_t);
    *kc_steps = best_kc;
}

int prepack_igemm(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw, const int32_t *bias) {
    const int taps = w->kernel_h * w->kernel_w;
    NNHIP_REQUIRE(ctx, (int64_t)taps * w->g_ic < 65536, -EINVAL,
                  "qconv2d_prepack: reduction length %lld would overflow the int32 accumulator",
                  (long long)taps * w->g_ic);
    w->k = taps * w->g_ic;
    w->ksteps = ceil_div(w->k, 64);
    const int max_tiles = (w->g_ic % 4 == 0) ? 16 : 4;
    plan_igemm(w->g_oc, w->ksteps, max_tiles, w->pixels_hint, ctx->compute_units, &w->tiles, &w->nchunks, &w->kc_steps);
    // Long reductions over many pixels and at least 64 channels are bound by the matrix cores: they take the
    // wide-tile kernels (a wave owns 64 pixels x 64 or 128 channels) when the launch has a 256-pixel block for every
    // compute unit; smaller launches keep the small tiles, whose larger wave count fills the device better.
    {
        const long long ptiles = ceil_div((int)std::min<int64_t>(std::max<int64_t>(w->pixels_hint, 0), 1 << 30), 256);
        // 256-channel chunks (two waves side by side share the block's activations) where that still fills the device
        const int wide_tiles = w->g_oc <= 64 ? 4 : (w->g_oc > 128 && ptiles * ceil_div(w->g_oc, 256) >= ctx->compute_units ? 16 : 8);
        w->wide = w->g_ic % 16 == 0 && w->ksteps >= kWideMinKsteps && w->g_oc >= 64 &&
                  ptiles * ceil_div(w->g_oc, wide_tiles * 16) >= ctx->compute_units;
        if (w->wide) {
            w->tiles = wide_tiles;
            w->nchunks = ceil_div(w->g_oc, w->tiles * 16);
            w->kc_steps = std::min(w->ksteps, kLdsFrags / w->tiles);
        }
    }
    // Reductions of kSmallWideMinKsteps k-steps and more over fewer pixels take the same kernel with 128 x 64 blocks
    // (four waves of 32 pixels) or 64 x 32 ones: against the small tiles' per-lane loads of 16 pixels' slices, the
    // row-order fetch through LDS needs a quarter of the requests to the vector L1, which is what such launches
    // are bound by.
    if (!w->wide && w->g_ic % 16 == 0 && w->ksteps >= kSmallWideMinKsteps) {
        w->wide = 2;
        // (64 x 32 blocks of two waves while the larger ones would leave more than half of the compute units without a
        // block: the 512 x 1024 x 1024 product takes 7.0 us with them, 9.2 us with 64 blocks of 128 x 64)
        const long long blocks128 = (long long)ceil_div((int)std::min<int64_t>(std::max<int64_t>(w->pixels_hint, 1), 1 << 30), 128) * ceil_div(w->g_oc, 64);
        w->tiles = (w->g_oc <= 32 || (w->pixels_hint > 0 && 2 * blocks128 < ctx->compute_units)) ? 2 : 4;
        w->nchunks = ceil_div(w->g_oc, w->tiles * 16);
        w->kc_steps = std::min(w->ksteps, kLdsFrags / w->tiles);
    }
    // -(zw - 128) has to be an s8 value
    w->fold = w->ksteps == 1 && w->k <= 32 && w->zw >= 1;
    const size_t group_bytes = (size_t)w->nchunks * w->ksteps * w->tiles * 1024;
    w->packed_bytes = group_bytes * w->groups;
    std::vector<uint8_t> packed(w->packed_bytes);
    std::vector<int32_t> wsum(w->out_channels), hb(w->out_channels, 0);
    if (bias) std::copy(bias, bias + w->out_channels, hb.begin());
    for (int32_t b : hb) w->bias_absmax = std::max<long long>(w->bias_absmax, std::llabs((long long)b));
    const int g_ic = w->g_ic, kh = w->kernel_h, kw = w->kernel_w;
    for (int g = 0; g < w->groups; g++) {
        const uint8_t *wg = w_oihw + (size_t)g * w->g_oc * g_ic * kh * kw;
        auto w_at = [&](int oc, int kk) -> uint8_t {
            const int tap = kk / g_ic, ic = kk % g_ic;
            return wg[((size_t)oc * g_ic + ic) * kh * kw + tap]; // OIHW: tap = ky * kw + kx
        };
        pack_group(packed.data() + g * group_bytes, wsum.data() + (size_t)g * w->g_oc, w->g_oc, w->k, w->ksteps, w->tiles,
                   w->nchunks, w_at, w->fold != 0, 128 - w->zw);
    }
    NNHIP_HIP(ctx, hipMalloc(&w->d_packed, w->packed_bytes));
    NNHIP_HIP(ctx, hipMalloc((void **)&w->d_wsum, sizeof(int32_t) * w->out_channels));
    NNHIP_HIP(ctx, hipMalloc((void **)&w->d_bias, sizeof(int32_t) * w->out_channels));
    NNHIP_HIP(ctx, hipMemcpy(w->d_packed, packed.data(), w->packed_bytes, hipMemcpyHostToDevice));
    NNHIP_HIP(ctx, hipMemcpy(w->d_wsum, wsum.data(), sizeof(int32_t) * w->out_channels, hipMemcpyHostToDevice));
    NNHIP_HIP(ctx, hipMemcpy(w->d_bias, hb.data(), sizeof(int32_t) * w->out_channels, hipMemcpyHostToDevice));
    return 0;
}

int igemm_pixel_groups(const nncase_hip_ctx *ctx, const nncase_hip_weights *w, int m) {
    return choose_rg(ctx, w->tiles, w->nchunks, m);
}

int igemm_load_mode(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c, int out_h, int out_w) {
    const bool pointwise = w->kernel_h == 1 && w->kernel_w == 1 && c->stride_h == 1 && c->stride_w == 1 &&
                           c->pad_h_before == 0 && c->pad_w_before == 0 && out_h == c->in_h && out_w == c->in_w;
    if (w->g_ic % 16 == 0) return pointwise ? kRows16 : kVec16;
    // (the row loader reads 16 bytes at a time: the tensor has to hold that many)
    if (w->g_ic % 8 == 0) return pointwise && (int64_t)c->batch * c->in_h * c->in_w * w->in_channels >= 16 ? kRows8 : kVec8;
    if (w->g_ic % 4 == 0) return kVec4;
    return kBytes;
}

int launch_qconv_igemm(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                       const nncase_hip_conv2d_args_t *c, int out_h, int out_w) {
    const int64_t m64 = (int64_t)c->batch * out_h * out_w;
    const int64_t in_bytes = (int64_t)c->batch * c->in_h * c->in_w * w->in_channels;
    const int out_es = c->out_dtype == NNCASE_HIP_DT_U8 && !c->dequantize_output ? 1 : 4;
    NNHIP_REQUIRE(ctx, m64 > 0 && m64 < ((int64_t)1 << 30), -EINVAL, "qconv2d: %lld output pixels unsupported",
                  (long long)m64);
    NNHIP_REQUIRE(ctx, in_bytes < ((int64_t)1 << 31), -EINVAL, "qconv2d: input of %lld bytes exceeds 2 GiB",
                  (long long)in_bytes);
    NNHIP_REQUIRE(ctx, m64 * w->out_channels * out_es < ((int64_t)1 << 40), -EINVAL, "qconv2d: output too large");
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0,
                  -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION, "qconv2d: activation buffers must be 16-byte aligned");

    IgemmArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x;
    a.y = y;
    a.m = (int)m64;
    a.n = w->g_oc;
    a.k = w->k;
    a.ksteps = w->ksteps;
    a.kc_steps = w->kc_steps;
    a.ldx = w->in_channels;
    a.x_bytes = (size_t)c->batch * c->in_h * c->in_w * w->in_channels;
    a.ldy = c->out_channel_stride ? c->out_channel_stride : w->out_channels;
    a.ldr = w->out_channels;
    NNHIP_REQUIRE(ctx, c->out_channel_stride >= 0 && c->out_channel_offset >= 0 &&
                           (c->out_channel_stride ? c->out_channel_offset + w->out_channels <= c->out_channel_stride : c->out_channel_offset == 0),
                  -EINVAL, "qconv2d: %d output channels at offset %d do not fit a pixel stride of %d", w->out_channels, c->out_channel_offset,
                  c->out_channel_stride);
    NNHIP_REQUIRE(ctx, m64 * a.ldy * out_es < ((int64_t)1 << 40), -EINVAL, "qconv2d: output too large");
    a.g_ic = w->g_ic;
    a.in_h = c->in_h;
    a.in_w = c->in_w;
    a.kw = w->kernel_w;
    a.stride_h = c->stride_h;
    a.stride_w = c->stride_w;
    a.dil_h = c->dilation_h;
    a.dil_w = c->dilation_w;
    a.pad_h = c->pad_h_before;
    a.pad_w = c->pad_w_before;
    a.d_ohow = make_fastdiv((uint32_t)(out_h * out_w));
    a.d_ow = make_fastdiv((uint32_t)out_w);
    a.d_kw = make_fastdiv((uint32_t)w->kernel_w);
    a.d_gic = make_fastdiv((uint32_t)w->g_ic);
    a.zxp = c->x_qp.zero_point - 128;
    a.zwp = w->zw - 128;
    a.zwp_rows = w->fold ? 0 : a.zwp;
    a.kc_mask = w->fold ? 1 : -1;
    a.zx_splat = (uint32_t)(c->x_qp.zero_point & 0xff) * 0x01010101u;
    {
        const int rc = make_epilogue(ctx, &a.ep, c->x_qp.scale, w->sw, c->y_qp, c->clamp_min, c->clamp_max, c->out_dtype, "qconv2d");
        if (rc) return rc;
    }

    {
        const int rc = make_residual_epilogue(ctx, &a.rep, c, w);
        if (rc) return rc;
    }
    // every accumulator, the zero-point terms included, is at most |bias| + 4 K 128^2 in magnitude
    a.magic_ok = a.ep.magic && a.ep.full && w->bias_absmax + 4ll * w->k * 16384 <= a.ep.magic_limit;
    a.lut = c->out_dtype == NNCASE_HIP_DT_U8 ? w->d_post_lut : nullptr;
    if (c->dequantize_output != 0) { // (out_dtype is u8 here: the entry point has turned the call into its u8 form)
        const nncase_hip_quant_param_t last = c->residual_dev ? c->sum_qp : (w->d_post_lut ? w->post_lut_qp : c->y_qp);
        a.deq = 1, a.deq_zero = last.zero_point, a.deq_scale = last.scale;
    }
    const int mode = igemm_load_mode(w, c, out_h, out_w);

    const size_t group_bytes = (size_t)w->nchunks * w->ksteps * w->tiles * 1024;
    for (int g = 0; g < w->groups; g++) {
        a.wpk = reinterpret_cast<const uint8_t *>(w->d_packed) + g * group_bytes;
        a.wsum = w->d_wsum + (size_t)g * w->g_oc;
        a.bias = w->d_bias + (size_t)g * w->g_oc;
        a.x_coff = g * w->g_ic;
        a.y_coff = g * w->g_oc + c->out_channel_offset;
        a.r_coff = g * w->g_oc;
        int rc;
        if (w->wide == 2) {
            rc = mode == kRows16 ? launch_wide_small_rows16(ctx, a, w->tiles, w->nchunks) : launch_wide_small_vec16(ctx, a, w->tiles, w->nchunks);
            if (rc) return rc;
            continue;
        }
        if (w->wide) {
            rc = mode == kRows16 ? launch_wide_rows16(ctx, a, w->tiles, w->nchunks) : launch_wide_vec16(ctx, a, w->tiles, w->nchunks);
            if (rc) return rc;
            continue;
        }
        const int rg = choose_rg(ctx, w->tiles, w->nchunks, a.m);
        switch (mode) {
        case kRows16: rc = launch_igemm_rows16(ctx, a, w->tiles, w->nchunks, rg); break;
        case kVec16: rc = launch_igemm_vec16(ctx, a, w->tiles, w->nchunks, rg); break;
        case kVec8: rc = launch_igemm_vec8(ctx, a, w->tiles, w->nchunks, rg); break;
        case kRows8: rc = launch_igemm_rows8(ctx, a, w->tiles, w->nchunks, rg); break;
        case kVec4: rc = launch_igemm_vec4(ctx, a, w->tiles, w->nchunks, rg); break;
        default: rc = launch_igemm_bytes(ctx, a, w->tiles, w->nchunks, rg); break;
        }
        if (rc) return rc;
    }
    return 0;
}

} // namespace nnhip
