// Depthwise u8/u8 convolution (groups == channels), NHWC.  Bandwidth-bound:
// 2 bytes of HBM traffic per output for 9 multiply-adds, so no matrix cores;
// the work is laid out so that every global access is a dword holding 4
// adjacent channels of one pixel and adjacent lanes hold adjacent channels.
//
//   acc[c] = bias[c] + sum_t (x_t[c] - zx) * (w_t[c] - zw)
//          = sum_t x_t[c] * w''_t[c] + (bias[c] - zx * sum_t w''_t[c]),   w'' = w - zw
// where a padding tap is read as x = zx (contributes nothing).  w'' and its
// tap sum are pack-time constants.  The requantisation epilogue is the same
// fp32 sequence as the dense kernel's.
//
// dw3x3_kernel: a thread owns 4 channels x 4 output columns and walks down a
// strip of output rows keeping the last three input rows unpacked in
// registers, so each input byte is loaded from memory once per strip (plus a
// two-row halo) and unpacked once.
// dw_generic_kernel: any kernel size / stride / dilation / channel count.
#include "qconv.hpp"

#include <algorithm>
#include <vector>

namespace nnhip {

constexpr int kDwThreads = 256;
constexpr int kDwCols = 4;  // output columns per thread
constexpr int kDwMaxRows = 8; // most output rows one thread walks down (3x3 kernel)

struct DwArgs {
    const uint8_t *x;
    void *y;
    const int16_t *w; // [taps][channels], w - zw
    const int32_t *wsum;
    const int32_t *bias;
    int batch, in_h, in_w, channels, out_h, out_w;
    int kh, kw, stride_h, stride_w, dil_h, dil_w, pad_h, pad_w;
    int zx;
    uint32_t zx_splat;
    int cq;          // channel vectors per pixel
    int strips;      // column strips per row
    int row_chunks;  // row chunks per image (3x3 kernel)
    int rows;        // output rows per thread (3x3 kernel)
    FastDiv d_cq, d_strips, d_rows, d_ow, d_oh;
    long long total; // threads of useful work
    Epilogue ep;
};

// A conditional between two named objects is an lvalue in C++, which the compiler may turn
// into a load through a selected address (private memory); taking the operands by value
// keeps the choice a register select.
__device__ __forceinline__ uint32_t select_u32(bool c, uint32_t yes, uint32_t no) { return c ? yes : no; }

// Stores 4 adjacent channels of one output pixel; `o` is the element offset of the first.
__device__ __forceinline__ void dw_store4(const DwArgs &a, uint32_t o, const int32_t (&v)[4]) {
    if (a.ep.out_mode == kOutU8) {
        *reinterpret_cast<uint32_t *>(reinterpret_cast<uint8_t *>(a.y) + o) = requant4_u8_packed(v, a.ep);
    } else if (a.ep.out_mode == kOutI32) {
        *reinterpret_cast<int4 *>(reinterpret_cast<int32_t *>(a.y) + o) = int4{v[0], v[1], v[2], v[3]};
    } else {
        float4 f;
        f.x = clamp_ref((float)v[0] * a.ep.mult, a.ep.lo, a.ep.hi);
        f.y = clamp_ref((float)v[1] * a.ep.mult, a.ep.lo, a.ep.hi);
        f.z = clamp_ref((float)v[2] * a.ep.mult, a.ep.lo, a.ep.hi);
        f.w = clamp_ref((float)v[3] * a.ep.mult, a.ep.lo, a.ep.hi);
        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.y) + o) = f;
    }
}

// Stores one output row of a thread: kDwCols pixels of 4 adjacent channels each; `o` is the element offset of the
// first.  u8 rows are stored without predicates (a predicated memory instruction sits behind a branch, and
// operations behind branches cannot be counted by the waits of the rows that follow): a pixel outside the image
// is replaced by the first pixel of the thread's first row, address and value, which always exists, is written
// by this thread alone and so is merely written again.  `safe_off` / `safe_val` carry that pixel; `first` is
// uniform.
template <bool FF, bool MG, typename T>
__device__ __forceinline__ void dw_store_row(const DwArgs &a, uint32_t o, const T (&v)[kDwCols][4], const bool (&col_stored)[kDwCols],
                                             bool row_stored, bool first, uint32_t &safe_off, uint32_t &safe_val) {
    if (FF || std::is_same<T, float>::value || a.ep.out_mode == kOutU8) { // (fp32 sums are used for u8 outputs only)
        uint32_t q[kDwCols];
#pragma unroll
        for (int c = 0; c < kDwCols; c++) {
            if constexpr (MG && std::is_same<T, int32_t>::value) q[c] = requant4_u8_packed_magic(v[c], a.ep);
            else q[c] = FF ? requant4_u8_packed_direct(v[c], a.ep) : requant4_u8_packed(v[c], a.ep);
        }
        safe_off = first ? o : safe_off;
        safe_val = first ? q[0] : safe_val;
#pragma unroll
        for (int c = 0; c < kDwCols; c++) {
            const bool sel = row_stored && col_stored[c];
            const uint32_t off = select_u32(sel, o + (uint32_t)(c * a.channels), safe_off);
            *reinterpret_cast<uint32_t *>(reinterpret_cast<uint8_t *>(a.y) + off) = select_u32(sel, q[c], safe_val);
        }
    } else if (a.ep.out_mode == kOutI32) {
#pragma unroll
        for (int c = 0; c < kDwCols; c++)
            if (row_stored && col_stored[c])
                *reinterpret_cast<int4 *>(reinterpret_cast<int32_t *>(a.y) + o + (uint32_t)(c * a.channels)) =
                    int4{(int32_t)v[c][0], (int32_t)v[c][1], (int32_t)v[c][2], (int32_t)v[c][3]};
    } else {
#pragma unroll
        for (int c = 0; c < kDwCols; c++) {
            float4 f;
            f.x = clamp_ref((float)v[c][0] * a.ep.mult, a.ep.lo, a.ep.hi);
            f.y = clamp_ref((float)v[c][1] * a.ep.mult, a.ep.lo, a.ep.hi);
            f.z = clamp_ref((float)v[c][2] * a.ep.mult, a.ep.lo, a.ep.hi);
            f.w = clamp_ref((float)v[c][3] * a.ep.mult, a.ep.lo, a.ep.hi);
            if (row_stored && col_stored[c]) *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.y) + o + (uint32_t)(c * a.channels)) = f;
        }
    }
}

// All offsets are 32-bit element offsets from the (uniform) tensor bases, advanced by
// additions only; the host checks that both tensors stay below 2^31 elements.
// The loads of the rows the NEXT output row needs are issued before the current row is
// computed, so a whole row of arithmetic covers their latency.
// The stride-2 kernel holds nine input columns per row; asking for three blocks per CU keeps it
// at 3 waves per SIMD (without the bound the allocator takes 176 VGPRs and drops to 2).
//
// FP: the sums are kept in fp32.  The host picks this form for u8 outputs when every partial sum, the
// per-channel constant included, stays below 2^24 in magnitude: all of them are then integers that fp32 holds
// exactly, the result is the integer form's bit for bit, and the multiply-adds run at the full rate of the
// vector unit (v_fma_f32) instead of the integer multiplier's lower one; the accumulators need no conversion
// before they are requantised either.
// FF: the layer's epilogue is the one-instruction requantisation to u8 (fast and full), fixed at compile time.
// MG (integer sums): they start from kMagicBias and are requantised as floats without a conversion (Epilogue::magic).
template <int S, bool FP, bool FF, bool MG = false> __global__ __launch_bounds__(kDwThreads, (S == 2 && !FP ? 3 : 1)) void dw3x3_kernel(const DwArgs a) {
    static_assert(!MG || (FF && !FP), "the magic-bias form replaces the conversion of integer sums in the one-instruction epilogue");
    using acc_t = typename std::conditional<FP, float, int32_t>::type;
    constexpr int NCOL = (kDwCols - 1) * S + 3;
    // Workgroups are dealt to the 8 XCDs round-robin, each XCD with an L2 of its own.  Renumber them
    // so that every XCD works on one contiguous run of the tensor: vertically adjacent row chunks,
    // which share two input rows, then meet in the same L2 instead of being fetched once per XCD.
    const uint32_t nblk = gridDim.x, per = nblk >> 3, rem = nblk & 7u;
    const uint32_t xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const uint32_t blk = xcd * per + min(xcd, rem) + slot;
    const uint32_t gid = blk * kDwThreads + threadIdx.x;
    if (gid >= (uint32_t)a.total) return;
    // gid -> (image, row chunk, strip, channel quad), channel quad fastest
    uint32_t t = gid;
    uint32_t q = fastdiv(t, a.d_cq);
    const int cq = (int)(t - q * a.d_cq.div);
    t = q;
    q = fastdiv(t, a.d_strips);
    const int strip = (int)(t - q * a.d_strips.div);
    t = q;
    q = fastdiv(t, a.d_rows);
    const int rchunk = (int)(t - q * a.d_rows.div);
    const int img = (int)q;

    const uint32_t zx_splat = a.zx_splat;
    const int c0 = cq * 4;
    const int ox0 = strip * kDwCols;
    const int oy0 = rchunk * a.rows;
    const int ix0 = ox0 * S - a.pad_w;
    const int iy_first = oy0 * S - a.pad_h;

    uint32_t w01[9], w23[9]; // (w - zw) of channels (0,1) and (2,3) as int16 pairs, per tap
    float wf[9][4];          // FP: the same as floats
    acc_t ct[4];
#pragma unroll
    for (int tap = 0; tap < 9; tap++) {
        const uint2 raw = *reinterpret_cast<const uint2 *>(a.w + (uint32_t)(tap * a.channels + c0));
        if constexpr (FP) {
            wf[tap][0] = (float)(int16_t)(raw.x & 0xffffu);
            wf[tap][1] = (float)((int32_t)raw.x >> 16);
            wf[tap][2] = (float)(int16_t)(raw.y & 0xffffu);
            wf[tap][3] = (float)((int32_t)raw.y >> 16);
        } else {
            w01[tap] = raw.x;
            w23[tap] = raw.y;
        }
    }
    {
        const int4 b = *reinterpret_cast<const int4 *>(a.bias + c0);
        const int4 s = *reinterpret_cast<const int4 *>(a.wsum + c0);
        constexpr int32_t start = MG ? kMagicBias : 0;
        ct[0] = (acc_t)(b.x - a.zx * s.x + start);
        ct[1] = (acc_t)(b.y - a.zx * s.y + start);
        ct[2] = (acc_t)(b.z - a.zx * s.z + start);
        ct[3] = (acc_t)(b.w - a.zx * s.w + start);
    }

    const uint32_t in_row = (uint32_t)(a.in_w * a.channels); // elements per input row
    const uint32_t in_base = (uint32_t)img * (uint32_t)a.in_h * in_row + (uint32_t)c0; // (img, row 0, column 0, c0)
    // Loads are unconditional: a tap outside the image reads the nearest pixel inside it
    // (always a valid address) and the value is replaced by the zero point afterwards, so
    // the border handling costs one select per load and no divergent branches.
    bool col_ok[NCOL];
    uint32_t col_off[NCOL];
#pragma unroll
    for (int col = 0; col < NCOL; col++) {
        const int ix = ix0 + col;
        col_ok[col] = (unsigned)ix < (unsigned)a.in_w;
        col_off[col] = (uint32_t)(min(max(ix, 0), a.in_w - 1) * a.channels);
    }

    uint32_t r01[3][NCOL], r23[3][NCOL]; // three most recent input rows, two channels per register
    float rf[3][NCOL][4];                // FP: one channel per register
    int next_iy = iy_first;             // rows are fetched strictly in order
    // fetch_row only issues the loads (nothing depends on their data); unpack_row, called one
    // output row later, applies the border replacement and splits the bytes.
    auto fetch_row = [&](uint32_t (&raw)[NCOL], bool &row_ok) {
        row_ok = (unsigned)next_iy < (unsigned)a.in_h;
        const uint32_t row_off = in_base + (uint32_t)min(max(next_iy, 0), a.in_h - 1) * in_row;
#pragma unroll
        for (int col = 0; col < NCOL; col++) raw[col] = *reinterpret_cast<const uint32_t *>(a.x + (row_off + col_off[col]));
        next_iy++;
    };
    auto unpack_row = [&](int buf, const uint32_t (&raw)[NCOL], bool row_ok) {
#pragma unroll
        for (int col = 0; col < NCOL; col++) {
            const uint32_t d = select_u32(row_ok && col_ok[col], raw[col], zx_splat);
            if constexpr (FP) {
#pragma unroll
                for (int c = 0; c < 4; c++) rf[buf][col][c] = (float)((d >> (8 * c)) & 0xffu); // v_cvt_f32_ubyte<c>
            } else {
                r01[buf][col] = __builtin_amdgcn_perm(0u, d, 0x0c010c00u); // [b0, 0, b1, 0]
                r23[buf][col] = __builtin_amdgcn_perm(0u, d, 0x0c030c02u); // [b2, 0, b3, 0]
            }
        }
    };

    const uint32_t out_row = (uint32_t)(a.out_w * a.channels);
    uint32_t out_off = ((uint32_t)img * (uint32_t)a.out_h + (uint32_t)oy0) * out_row + (uint32_t)(ox0 * a.channels + c0);

    // Output row t (relative) reads input rows t*S + {0,1,2} (relative), kept in
    // buffer (row index mod 3).  The loop is unrolled by 3 so every buffer index
    // is a compile-time constant.
    //
    // Memory operations complete in order and the wait before a row is unpacked is a count of younger
    // operations that may still be in flight: only operations issued on every path can be counted.  So the
    // loop issues the same loads and stores for every thread: all threads walk a.rows rows (rows below the
    // image are computed from clamped input rows and not stored), the loads are never predicated (addresses
    // are clamped into the image), and the predicate of a store guards the store instruction alone, after
    // all of its row has been requantised.  The wait for a row's loads then leaves the previous row's stores
    // in flight instead of waiting for their acknowledgement, which used to cost a memory round trip per row.
    //
    // Stride 1 fetches two output rows ahead (a row of arithmetic is shorter than a trip to memory); the rows
    // in flight rotate through three register sets so that, like the row buffers, they are named by the phase.
    constexpr int DEPTH = S == 1 ? 2 : 1;
    constexpr int NPRE = DEPTH == 2 ? 3 : 1;
    uint32_t pre[NPRE][S][NCOL]; // rows fetched ahead
    bool pre_ok[NPRE][S];
    {
        uint32_t raw[3 - S][NCOL];
        bool ok[3 - S];
#pragma unroll
        for (int b = 0; b < 3 - S; b++) fetch_row(raw[b], ok[b]);
#pragma unroll
        for (int d = 0; d < DEPTH; d++)
#pragma unroll
            for (int nr = 0; nr < S; nr++) fetch_row(pre[d][nr], pre_ok[d][nr]);
#pragma unroll
        for (int b = 0; b < 3 - S; b++) unpack_row(b, raw[b], ok[b]);
    }
    const int nrows = a.rows;              // uniform
    const int rows_here = a.out_h - oy0;   // rows of this thread that exist (>= 1)
    uint32_t safe_off = 0, safe_val = 0;
    bool col_stored[kDwCols];
#pragma unroll
    for (int o = 0; o < kDwCols; o++) col_stored[o] = ox0 + o < a.out_w;
    for (int t0 = 0; t0 < nrows; t0 += 3) {
#pragma unroll
        for (int ph = 0; ph < 3; ph++) {
            const int tt = t0 + ph;
            if (tt < nrows) {
                // input rows tt*S + 3 - S + nr; tt % 3 == ph fixes their residue mod 3
#pragma unroll
                for (int nr = 0; nr < S; nr++) unpack_row((ph * S + 3 - S + nr) % 3, pre[DEPTH == 2 ? ph : 0][nr], pre_ok[DEPTH == 2 ? ph : 0][nr]);
                // (also issued by the last rows, which need nothing more: a load that only some paths issue
                // could not be counted either, and its address is clamped into the image like any other)
#pragma unroll
                for (int nr = 0; nr < S; nr++) fetch_row(pre[DEPTH == 2 ? (ph + 2) % 3 : 0][nr], pre_ok[DEPTH == 2 ? (ph + 2) % 3 : 0][nr]);
                acc_t acc[kDwCols][4];
#pragma unroll
                for (int o = 0; o < kDwCols; o++)
#pragma unroll
                    for (int c = 0; c < 4; c++) acc[o][c] = ct[c];
#pragma unroll
                for (int ky = 0; ky < 3; ky++) {
                    const int buf = (ph * S + ky) % 3;
#pragma unroll
                    for (int kx = 0; kx < 3; kx++)
#pragma unroll
                        for (int o = 0; o < kDwCols; o++) {
                            const int col = o * S + kx, tap = ky * 3 + kx;
                            if constexpr (FP) {
#pragma unroll
                                for (int c = 0; c < 4; c++) acc[o][c] = __builtin_fmaf(rf[buf][col][c], wf[tap][c], acc[o][c]);
                            } else {
                                acc[o][0] = mad16_lo(r01[buf][col], w01[tap], acc[o][0]);
                                acc[o][1] = mad16_hi(r01[buf][col], w01[tap], acc[o][1]);
                                acc[o][2] = mad16_lo(r23[buf][col], w23[tap], acc[o][2]);
                                acc[o][3] = mad16_hi(r23[buf][col], w23[tap], acc[o][3]);
                            }
                        }
                }
                dw_store_row<FF, MG>(a, out_off, acc, col_stored, tt < rows_here, tt == 0, safe_off, safe_val);
                out_off += out_row;
            }
        }
    }
}

template <int VEC> __global__ __launch_bounds__(kDwThreads) void dw_generic_kernel(const DwArgs a) {
    const long long gid = (long long)blockIdx.x * kDwThreads + threadIdx.x;
    if (gid >= a.total) return;
    uint32_t t = (uint32_t)gid;
    uint32_t q = fastdiv(t, a.d_cq);
    const int c0 = (int)(t - q * a.d_cq.div) * VEC;
    t = q;
    q = fastdiv(t, a.d_ow);
    const int ox = (int)(t - q * a.d_ow.div);
    t = q;
    q = fastdiv(t, a.d_oh);
    const int oy = (int)(t - q * a.d_oh.div);
    const int img = (int)q;

    int32_t acc[VEC];
#pragma unroll
    for (int c = 0; c < VEC; c++) acc[c] = a.bias[c0 + c] - a.zx * a.wsum[c0 + c];
    const uint8_t *ximg = a.x + (size_t)img * a.in_h * a.in_w * a.channels + c0;
    for (int ky = 0; ky < a.kh; ky++) {
        const int iy = oy * a.stride_h - a.pad_h + ky * a.dil_h;
        for (int kx = 0; kx < a.kw; kx++) {
            const int ix = ox * a.stride_w - a.pad_w + kx * a.dil_w;
            const bool ok = (unsigned)iy < (unsigned)a.in_h && (unsigned)ix < (unsigned)a.in_w;
            const int16_t *wt = a.w + (size_t)(ky * a.kw + kx) * a.channels + c0;
            if (VEC == 4) {
                uint32_t d = a.zx_splat;
                if (ok) d = *reinterpret_cast<const uint32_t *>(ximg + ((size_t)iy * a.in_w + ix) * a.channels);
#pragma unroll
                for (int c = 0; c < VEC; c++) acc[c] += __mul24((int)((d >> (8 * c)) & 0xff), (int)wt[c]);
            } else {
                int xv = a.zx;
                if (ok) xv = ximg[((size_t)iy * a.in_w + ix) * a.channels];
                acc[0] += __mul24(xv, (int)wt[0]);
            }
        }
    }
    const uint32_t o = (((uint32_t)img * a.out_h + oy) * a.out_w + ox) * a.channels + c0;
    if (VEC == 4) {
        int32_t v[4];
#pragma unroll
        for (int c = 0; c < 4; c++) v[c] = acc[c < VEC ? c : 0];
        dw_store4(a, o, v);
    } else {
        if (a.ep.out_mode == kOutU8)
            reinterpret_cast<uint8_t *>(a.y)[o] = (uint8_t)requant_u8_lowbyte((float)acc[0] * a.ep.mult, a.ep);
        else if (a.ep.out_mode == kOutI32) reinterpret_cast<int32_t *>(a.y)[o] = acc[0];
        else reinterpret_cast<float *>(a.y)[o] = clamp_ref((float)acc[0] * a.ep.mult, a.ep.lo, a.ep.hi);
    }
}

int prepack_depthwise(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw, const int32_t *bias) {
    const int taps = w->kernel_h * w->kernel_w, ch = w->out_channels;
    w->k = taps;
    std::vector<int16_t> packed((size_t)taps * ch);
    std::vector<int32_t> wsum(ch, 0), hb(ch, 0);
    if (bias) std::copy(bias, bias + ch, hb.begin());
    for (int c = 0; c < ch; c++)
        for (int t = 0; t < taps; t++) {
            const int v = (int)w_oihw[(size_t)c * taps + t] - w->zw; // OIHW with I == 1
            packed[(size_t)t * ch + c] = (int16_t)v;
            wsum[c] += v;
        }
    w->dw_const_bound = 0;
    for (int c = 0; c < ch; c++)
        w->dw_const_bound = std::max<long long>(w->dw_const_bound, std::llabs((long long)hb[c]) + 255ll * std::llabs((long long)wsum[c]));
    w->packed_bytes = packed.size() * sizeof(int16_t);
    NNHIP_HIP(ctx, hipMalloc(&w->d_packed, w->packed_bytes));
    NNHIP_HIP(ctx, hipMalloc((void **)&w->d_wsum, sizeof(int32_t) * ch));
    NNHIP_HIP(ctx, hipMalloc((void **)&w->d_bias, sizeof(int32_t) * ch));
    NNHIP_HIP(ctx, hipMemcpy(w->d_packed, packed.data(), w->packed_bytes, hipMemcpyHostToDevice));
    NNHIP_HIP(ctx, hipMemcpy(w->d_wsum, wsum.data(), sizeof(int32_t) * ch, hipMemcpyHostToDevice));
    NNHIP_HIP(ctx, hipMemcpy(w->d_bias, hb.data(), sizeof(int32_t) * ch, hipMemcpyHostToDevice));
    return 0;
}

bool depthwise_uses_3x3(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c) {
    return w->out_channels % 4 == 0 && w->kernel_h == 3 && w->kernel_w == 3 && c->dilation_h == 1 && c->dilation_w == 1 &&
           c->stride_h == c->stride_w && (c->stride_h == 1 || c->stride_h == 2);
}

int launch_qconv_depthwise(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y,
                           const nncase_hip_conv2d_args_t *c, int out_h, int out_w) {
    const int ch = w->out_channels;
    const int64_t in_elems = (int64_t)c->batch * c->in_h * c->in_w * ch;
    const int64_t out_elems = (int64_t)c->batch * out_h * out_w * ch;
    NNHIP_REQUIRE(ctx, out_elems > 0, -EINVAL, "qconv2d(depthwise): empty output");
    NNHIP_REQUIRE(ctx, in_elems < ((int64_t)1 << 31) && out_elems < ((int64_t)1 << 31), -EINVAL,
                  "qconv2d(depthwise): tensors of 2^31 elements or more are not supported");
    NNHIP_REQUIRE(ctx, w->kernel_h * w->kernel_w <= 258, -EINVAL, "qconv2d(depthwise): window too large");

    DwArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x;
    a.y = y;
    a.w = reinterpret_cast<const int16_t *>(w->d_packed);
    a.wsum = w->d_wsum;
    a.bias = w->d_bias;
    a.batch = c->batch;
    a.in_h = c->in_h;
    a.in_w = c->in_w;
    a.channels = ch;
    a.out_h = out_h;
    a.out_w = out_w;
    a.kh = w->kernel_h;
    a.kw = w->kernel_w;
    a.stride_h = c->stride_h;
    a.stride_w = c->stride_w;
    a.dil_h = c->dilation_h;
    a.dil_w = c->dilation_w;
    a.pad_h = c->pad_h_before;
    a.pad_w = c->pad_w_before;
    a.zx = c->x_qp.zero_point;
    a.zx_splat = (uint32_t)(c->x_qp.zero_point & 0xff) * 0x01010101u;
    {
        const int rc = make_epilogue(ctx, &a.ep, c->x_qp.scale, w->sw, c->y_qp, c->clamp_min, c->clamp_max, c->out_dtype, "qconv2d");
        if (rc) return rc;
    }

    const bool vec4 = (ch % 4 == 0) && ((reinterpret_cast<uintptr_t>(x) & 3u) == 0) &&
                      ((reinterpret_cast<uintptr_t>(y) & 15u) == 0);
    const bool k3 = vec4 && depthwise_uses_3x3(w, c);
    if (k3) {
        a.cq = ch / 4;
        a.strips = ceil_div(out_w, kDwCols);
        // Rows per thread.  Long strips amortise the two-row halo and the per-thread set-up;
        // short ones give more waves.  While every SIMD gets at least a few waves, the waves are
        // dealt out in whole numbers, so the length that minimises (waves per SIMD, rounded up)
        // x (work per wave) wins; smaller problems are latency-bound and take the shortest
        // strips that still leave two waves per SIMD.
        {
            const long long simds = (long long)ctx->compute_units * 4;
            auto waves_for = [&](int rows) {
                return ((long long)c->batch * ceil_div(out_h, rows) * a.strips * a.cq + 63) / 64;
            };
            if (waves_for(kDwMaxRows) >= 3 * simds) {
                long long best_cost = -1;
                for (int rows = 2; rows <= kDwMaxRows; rows++) {
                    const long long per_simd = (waves_for(rows) + simds - 1) / simds;
                    const long long cost = per_simd * (rows * 340 + 100);
                    if (best_cost < 0 || cost < best_cost) {
                        best_cost = cost;
                        a.rows = rows;
                    }
                }
            } else {
                a.rows = kDwMaxRows;
                while (a.rows > 1 && waves_for(a.rows) < 2 * simds) a.rows /= 2;
            }
        }
        a.row_chunks = ceil_div(out_h, a.rows);
        a.d_cq = make_fastdiv((uint32_t)a.cq);
        a.d_strips = make_fastdiv((uint32_t)a.strips);
        a.d_rows = make_fastdiv((uint32_t)a.row_chunks);
        a.total = (long long)c->batch * a.row_chunks * a.strips * a.cq;
        NNHIP_REQUIRE(ctx, a.total < ((long long)1 << 31), -EINVAL, "qconv2d(depthwise): too many work items");
        const int grid = (int)((a.total + kDwThreads - 1) / kDwThreads);
        // Every partial sum is an integer of magnitude at most |bias - zx * sum(w')| + 9 * 255 * 255.
        const bool fp = a.ep.out_mode == kOutU8 && w->dw_const_bound + 9 * 255 * 255 <= (1 << 24);
        const bool ff = a.ep.out_mode == kOutU8 && a.ep.fast && a.ep.full;
        const dim3 g(grid), t(kDwThreads);
        if (c->stride_h == 1) {
            if (fp && ff) hipLaunchKernelGGL((dw3x3_kernel<1, true, true>), g, t, 0, ctx->stream, a);
            else if (fp) hipLaunchKernelGGL((dw3x3_kernel<1, true, false>), g, t, 0, ctx->stream, a);
            else if (ff) hipLaunchKernelGGL((dw3x3_kernel<1, false, true>), g, t, 0, ctx->stream, a);
            else hipLaunchKernelGGL((dw3x3_kernel<1, false, false>), g, t, 0, ctx->stream, a);
        } else {
            // (stride 2 holds nine input columns per row: as floats they leave room for two waves per SIMD only,
            // and the largest stride-2 layer of MobileNetV2 runs 15 % slower that way)
            const bool mg = ff && a.ep.magic && w->dw_const_bound + 9 * 255 * 255 <= a.ep.magic_limit;
            if (mg) hipLaunchKernelGGL((dw3x3_kernel<2, false, true, true>), g, t, 0, ctx->stream, a);
            else if (ff) hipLaunchKernelGGL((dw3x3_kernel<2, false, true>), g, t, 0, ctx->stream, a);
            else hipLaunchKernelGGL((dw3x3_kernel<2, false, false>), g, t, 0, ctx->stream, a);
        }
        NNHIP_LAUNCH_CHECK(ctx, "dw3x3_kernel");
        return 0;
    }
    const int vec = vec4 ? 4 : 1;
    a.cq = ch / vec;
    a.d_cq = make_fastdiv((uint32_t)a.cq);
    a.d_ow = make_fastdiv((uint32_t)out_w);
    a.d_oh = make_fastdiv((uint32_t)out_h);
    a.total = (long long)c->batch * out_h * out_w * a.cq;
    NNHIP_REQUIRE(ctx, a.total < ((long long)1 << 31), -EINVAL, "qconv2d(depthwise): too many work items");
    const int grid = (int)((a.total + kDwThreads - 1) / kDwThreads);
    if (vec == 4) hipLaunchKernelGGL(dw_generic_kernel<4>, dim3(grid), dim3(kDwThreads), 0, ctx->stream, a);
    else hipLaunchKernelGGL(dw_generic_kernel<1>, dim3(grid), dim3(kDwThreads), 0, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "dw_generic_kernel");
    return 0;
}

} // namespace nnhip
