// Dense u8/u8 convolution for inputs with very few channels (the RGB stem of a
// classifier): 3 x 3 window, 1..4 input channels, any stride.
//
// With 3 channels the reduction is only 27 long, so an MFMA tile (K = 64) would be
// mostly padding and the implicit-GEMM gather degenerates to byte loads.  Here one
// thread owns one output pixel instead: in NHWC the KW * C bytes of a window row are
// contiguous, so the whole window is three (unaligned) 12-byte loads; the bytes are
// spliced into a packed s8 vector and every output channel is a short chain of
// v_dot4_i32_i8 against weights that all lanes read from the same LDS address
// (broadcast reads).  A thread produces all output channels of its pixel, i.e. a
// contiguous run of NHWC bytes, so stores are full 16-byte vectors.
// Zero points are folded exactly as in the implicit-GEMM kernel.
#include "qconv.hpp"

#include <algorithm>
#include <vector>

namespace nnhip {

constexpr int kScThreads = 256;

struct SmallCArgs {
    const uint8_t *x;
    void *y;
    const int32_t *wpk;  // [oc_pad][KDP] packed s8 weights (dwords)
    const int32_t *wsum; // [oc]
    const int32_t *bias; // [oc]
    int m, oc, oc_pad;
    int in_h, in_w, out_w;
    int stride_h, stride_w, pad_h, pad_w;
    long long in_bytes;
    FastDiv d_ohow, d_ow;
    int k, zxp, zwp;
    uint32_t zx_splat;
    Epilogue ep;
};

struct __attribute__((packed, aligned(1))) Bytes12 {
    uint32_t d[3];
};

template <int C, int KW, int KH> __global__ __launch_bounds__(kScThreads) void qconv_smallc_kernel(const SmallCArgs a) {
    constexpr int KWC = KW * C;          // bytes per window row
    constexpr int KB = KWC * KH;         // reduction length
    constexpr int KD = (KB + 3) / 4;     // ... in dwords
    constexpr int KDP = (KD + 3) / 4 * 4; // padded to whole 16-byte LDS reads
    static_assert(KWC <= 12, "a window row must fit three dwords");
    extern __shared__ __attribute__((aligned(16))) int32_t sc_lds[];
    int32_t *wl = sc_lds;                    // [oc_pad][KDP]
    int32_t *cterm = sc_lds + a.oc_pad * KDP; // [oc_pad]
    for (int i = threadIdx.x; i < a.oc_pad * KDP; i += kScThreads) wl[i] = a.wpk[i];
    for (int i = threadIdx.x; i < a.oc_pad; i += kScThreads)
        cterm[i] = i < a.oc ? a.bias[i] - a.zxp * a.wsum[i] + a.k * a.zxp * a.zwp : 0;
    __syncthreads();

    const int p = blockIdx.x * kScThreads + threadIdx.x;
    if (p >= a.m) return;
    const uint32_t img = fastdiv((uint32_t)p, a.d_ohow);
    const uint32_t rem = (uint32_t)p - img * a.d_ohow.div;
    const uint32_t oy = fastdiv(rem, a.d_ow);
    const uint32_t ox = rem - oy * a.d_ow.div;
    const int iy0 = (int)oy * a.stride_h - a.pad_h;
    const int ix0 = (int)ox * a.stride_w - a.pad_w;

    // which of the 12 loaded bytes of a row belong to a pixel inside the image
    uint32_t vmask[3] = {0, 0, 0};
#pragma unroll
    for (int kx = 0; kx < KW; kx++) {
        const bool ok = (unsigned)(ix0 + kx) < (unsigned)a.in_w;
#pragma unroll
        for (int c = 0; c < C; c++) {
            const int b = kx * C + c;
            if (ok) vmask[b / 4] |= 0xffu << (8 * (b % 4));
        }
    }

    uint8_t stream[KD * 4]; // the window, row after row (registers after unrolling)
#pragma unroll
    for (int i = 0; i < KD * 4; i++) stream[i] = 0x80; // x' = 0 past the end of the reduction
#pragma unroll
    for (int ky = 0; ky < KH; ky++) {
        const int iy = iy0 + ky;
        uint32_t r[3] = {a.zx_splat, a.zx_splat, a.zx_splat};
        if ((unsigned)iy < (unsigned)a.in_h) {
            const long long s = ((long long)((int)img * a.in_h + iy) * a.in_w + ix0) * C;
            if (s >= 0 && s + 12 <= a.in_bytes) {
                const Bytes12 v = *reinterpret_cast<const Bytes12 *>(a.x + s);
#pragma unroll
                for (int d = 0; d < 3; d++) r[d] = (v.d[d] & vmask[d]) | (a.zx_splat & ~vmask[d]);
            } else { // first / last bytes of the tensor: stay inside it
#pragma unroll
                for (int b = 0; b < KWC; b++) {
                    const long long idx = s + b;
                    if ((vmask[b / 4] >> (8 * (b % 4))) & 1u)
                        if (idx >= 0 && idx < a.in_bytes)
                            r[b / 4] = (r[b / 4] & ~(0xffu << (8 * (b % 4)))) | ((uint32_t)a.x[idx] << (8 * (b % 4)));
                }
            }
        }
#pragma unroll
        for (int b = 0; b < KWC; b++) stream[ky * KWC + b] = (uint8_t)(r[b / 4] >> (8 * (b % 4)));
    }
    int32_t xs[KD];
#pragma unroll
    for (int i = 0; i < KD; i++) {
        const uint32_t v = (uint32_t)stream[4 * i] | ((uint32_t)stream[4 * i + 1] << 8) | ((uint32_t)stream[4 * i + 2] << 16) |
                           ((uint32_t)stream[4 * i + 3] << 24);
        xs[i] = (int32_t)(v ^ 0x80808080u);
    }
    int32_t rowsum = 0;
#pragma unroll
    for (int i = 0; i < KD; i++) rowsum = __builtin_amdgcn_sdot4(xs[i], 0x01010101, rowsum, false);
    const int32_t nrsz = -a.zwp * rowsum;

    const size_t obase = (size_t)p * a.oc;
    for (int ocb = 0; ocb < a.oc; ocb += 16) {
        int32_t acc[16];
#pragma unroll
        for (int o = 0; o < 16; o++) {
            const int32_t *wrow = wl + (ocb + o) * KDP;
            int32_t s = cterm[ocb + o] + nrsz;
#pragma unroll
            for (int i4 = 0; i4 < KDP; i4 += 4) {
                const int4 wv = *reinterpret_cast<const int4 *>(wrow + i4);
                if (i4 + 0 < KD) s = __builtin_amdgcn_sdot4(xs[i4 + 0 < KD ? i4 + 0 : 0], wv.x, s, false);
                if (i4 + 1 < KD) s = __builtin_amdgcn_sdot4(xs[i4 + 1 < KD ? i4 + 1 : 0], wv.y, s, false);
                if (i4 + 2 < KD) s = __builtin_amdgcn_sdot4(xs[i4 + 2 < KD ? i4 + 2 : 0], wv.z, s, false);
                if (i4 + 3 < KD) s = __builtin_amdgcn_sdot4(xs[i4 + 3 < KD ? i4 + 3 : 0], wv.w, s, false);
            }
            acc[o] = s;
        }
        const int nvalid = min(16, a.oc - ocb); // multiple of 4
        if (a.ep.out_mode == kOutU8) {
            uint32_t q[4];
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const int32_t v4[4] = {acc[d * 4], acc[d * 4 + 1], acc[d * 4 + 2], acc[d * 4 + 3]};
                q[d] = requant4_u8_packed(v4, a.ep);
            }
            uint8_t *yo = reinterpret_cast<uint8_t *>(a.y) + obase + ocb;
            if (nvalid == 16 && (a.oc & 15) == 0) {
                *reinterpret_cast<uint4 *>(yo) = uint4{q[0], q[1], q[2], q[3]};
            } else {
#pragma unroll
                for (int d = 0; d < 4; d++)
                    if (d * 4 < nvalid) *reinterpret_cast<uint32_t *>(yo + d * 4) = q[d];
            }
        } else {
            uint32_t *yo = reinterpret_cast<uint32_t *>(a.y) + obase + ocb;
#pragma unroll
            for (int o = 0; o < 16; o++)
                if (o < nvalid)
                    yo[o] = a.ep.out_mode == kOutI32
                                ? (uint32_t)acc[o]
                                : __float_as_uint(clamp_ref((float)acc[o] * a.ep.mult, a.ep.lo, a.ep.hi));
        }
    }
}

bool smallc_supported(const nncase_hip_weights *w) {
    return w->groups == 1 && w->kernel_h == 3 && w->kernel_w == 3 && w->in_channels >= 1 && w->in_channels <= 4 &&
           w->out_channels % 4 == 0 && w->out_channels <= 512;
}

int prepack_smallc(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw) {
    const int c = w->in_channels, kh = w->kernel_h, kw = w->kernel_w;
    const int kb = c * kh * kw, kd = ceil_div(kb, 4), kdp = ceil_div(kd, 4) * 4;
    const int oc_pad = ceil_div(w->out_channels, 16) * 16;
    std::vector<int32_t> packed((size_t)oc_pad * kdp, 0);
    for (int oc = 0; oc < w->out_channels; oc++)
        for (int kk = 0; kk < kb; kk++) {
            const int tap = kk / c, ic = kk % c; // k = (ky * kw + kx) * c + ic
            const uint8_t v = (uint8_t)(w_oihw[((size_t)oc * c + ic) * kh * kw + tap] ^ 0x80);
            packed[(size_t)oc * kdp + kk / 4] |= (int32_t)((uint32_t)v << (8 * (kk % 4)));
        }
    w->smallc_bytes = packed.size() * sizeof(int32_t);
    NNHIP_HIP(ctx, hipMalloc(&w->d_smallc, w->smallc_bytes));
    NNHIP_HIP(ctx, hipMemcpy(w->d_smallc, packed.data(), w->smallc_bytes, hipMemcpyHostToDevice));
    return 0;
}

int launch_qconv_smallc(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                        const nncase_hip_conv2d_args_t *c, int out_h, int out_w) {
    const int64_t m64 = (int64_t)c->batch * out_h * out_w;
    NNHIP_REQUIRE(ctx, m64 > 0 && m64 < ((int64_t)1 << 30), -EINVAL, "qconv2d: %lld output pixels unsupported", (long long)m64);
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(y) & 15u) == 0, -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION,
                  "qconv2d: activation buffers must be 16-byte aligned");
    SmallCArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x;
    a.y = y;
    a.wpk = reinterpret_cast<const int32_t *>(w->d_smallc);
    a.wsum = w->d_wsum;
    a.bias = w->d_bias;
    a.m = (int)m64;
    a.oc = w->out_channels;
    a.oc_pad = ceil_div(w->out_channels, 16) * 16;
    a.in_h = c->in_h;
    a.in_w = c->in_w;
    a.out_w = out_w;
    a.stride_h = c->stride_h;
    a.stride_w = c->stride_w;
    a.pad_h = c->pad_h_before;
    a.pad_w = c->pad_w_before;
    a.in_bytes = (long long)c->batch * c->in_h * c->in_w * w->in_channels;
    a.d_ohow = make_fastdiv((uint32_t)(out_h * out_w));
    a.d_ow = make_fastdiv((uint32_t)out_w);
    a.k = w->k;
    a.zxp = c->x_qp.zero_point - 128;
    a.zwp = w->zw - 128;
    a.zx_splat = (uint32_t)(c->x_qp.zero_point & 0xff) * 0x01010101u;
    const int rc = make_epilogue(ctx, &a.ep, c->x_qp.scale, w->sw, c->y_qp, c->clamp_min, c->clamp_max, c->out_dtype, "qconv2d");
    if (rc) return rc;
    const int kb = w->in_channels * 9, kdp = ceil_div(ceil_div(kb, 4), 4) * 4;
    const size_t lds = ((size_t)a.oc_pad * kdp + a.oc_pad) * sizeof(int32_t);
    const dim3 grid(ceil_div(a.m, kScThreads));
    switch (w->in_channels) {
    case 1: hipLaunchKernelGGL((qconv_smallc_kernel<1, 3, 3>), grid, dim3(kScThreads), lds, ctx->stream, a); break;
    case 2: hipLaunchKernelGGL((qconv_smallc_kernel<2, 3, 3>), grid, dim3(kScThreads), lds, ctx->stream, a); break;
    case 3: hipLaunchKernelGGL((qconv_smallc_kernel<3, 3, 3>), grid, dim3(kScThreads), lds, ctx->stream, a); break;
    default: hipLaunchKernelGGL((qconv_smallc_kernel<4, 3, 3>), grid, dim3(kScThreads), lds, ctx->stream, a); break;
    }
    NNHIP_LAUNCH_CHECK(ctx, "qconv_smallc_kernel");
    return 0;
}

} // namespace nnhip
