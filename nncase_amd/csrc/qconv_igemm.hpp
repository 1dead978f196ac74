// u8/u8 convolution and matmul as an implicit GEMM on the gfx950 int8 matrix
// cores (v_mfma_i32_16x16x64_i8), int32 accumulation, zero points folded in as
// sums, fp32 requantisation fused in the epilogue.
//
// Orientation.  The MFMA "A" operand (rows) is a 16-channel slice of the
// pre-packed weights, the "B" operand (columns) is a group of 16 output
// pixels, so after the multiply every lane owns 4 consecutive output channels
// of ONE pixel per tile and, because the weight rows were permuted at pack
// time, 4*T consecutive channels over the T tiles of its chunk: the epilogue
// writes NHWC bytes with dword / dwordx4 stores and no cross-lane traffic.
//
// Zero points.  u8 values are re-biased to s8 with x' = x ^ 0x80 (= x - 128):
//   sum (x - zx)(w - zw) = sum x'w' - zw' * sum_k x' - zx' * sum_k w' + K zx' zw'
// with zx' = zx - 128, zw' = zw - 128.  sum_k w' is a pack-time constant;
// sum_k x' (per pixel) comes from one extra MFMA per k-step against an
// all-ones weight fragment held in registers, which leaves the sum in every
// lane that needs it.  Padding taps are loaded as x = zx (they contribute
// nothing); k positions past the end of the reduction load as x' = 0 and hit
// zero weights.
//
// Data movement.  A block owns one chunk of output channels: it copies that
// chunk's weight fragments into LDS once and then walks pixel tiles with a
// grid stride, streaming activations global -> registers (each activation
// fragment feeds all T tiles) while the previous fragment is being multiplied.
//
// The activation loader is a template parameter (one translation unit per
// mode so the instantiations compile in parallel):
//   kRows16  1x1 / stride 1 / no padding, channels % 16 == 0: a pixel's
//            reduction row is contiguous, one 16-byte load per lane and k-step
//   kRows8   the same for channels % 8 == 0: the last load of a row is half used
//   kVec16/8/4  any window; channels % VW == 0, so a VW-byte piece of the
//            reduction never straddles two taps
//   kBytes   anything else (e.g. 3 input channels): byte gathers
#pragma once

#include <mutex>
#include <type_traits>

#include "qconv.hpp"

namespace nnhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = 4;
constexpr int kLdsFrags = 48; // weight fragments (1 KiB each) resident in LDS per block

enum LoadMode { kRows16 = 0, kVec16 = 1, kVec8 = 2, kVec4 = 3, kBytes = 4, kRows8 = 5 };
constexpr bool loads_rows(int mode) { return mode == kRows16 || mode == kRows8; }

struct IgemmArgs {
    const uint8_t *x;
    void *y;
    const uint8_t *wpk;    // fragments of this group: [nchunks][ksteps][T][1024]
    const int32_t *wsum;   // [n] of this group
    const int32_t *bias;   // [n] of this group
    int m;                 // output pixels
    int n;                 // output channels of this group
    int k;                 // reduction length
    int ksteps, kc_steps;  // total k-steps, k-steps per LDS stage
    int ldx, x_coff;       // input pixel stride / channel offset of the group (bytes)
    size_t x_bytes;        // size of the input tensor
    int ldy, y_coff;       // output pixel stride / channel offset (elements)
    int ldr, r_coff;       // the same for the (dense) residual tensor
    int g_ic;
    int in_h, in_w;
    int kw, stride_h, stride_w, dil_h, dil_w, pad_h, pad_w;
    FastDiv d_ohow, d_ow, d_kw, d_gic;
    int zxp, zwp;          // zx - 128, zw - 128
    int zwp_rows;          // zwp where the kernel still owes -zwp * (sum of x') per pixel, 0 where the weights carry it
    int kc_mask;           // applied to the index of the 16-byte slice a lane loads: 1 with such weights, else all ones
    uint32_t zx_splat;     // zx in all four bytes
    int num_mtiles;
    Epilogue ep;
    ResidualEpilogue rep;
    const uint32_t *lut;   // 256-entry byte table applied to the requantised byte (before the residual add), or null
    int magic_ok;          // the epilogue's magic-bias pair exists and every accumulator of this layer stays within its range
    int deq;               // the u8 result is stored as float32: (q - deq_zero) * deq_scale
    int deq_zero;
    float deq_scale;
};

// Packs one group's weights into MFMA operand order.
//   w_at(oc, k) -> u8 weight of output channel oc (within the group) at
//   reduction index k = (ky * kw + kx) * g_ic + ic.
// Fragment (chunk, ks, nt): byte (kg * 16 + i) * 16 + b holds the weight of
//   channel chunk*16T + (i / 4) * 4T + nt * 4 + (i % 4) at k = ks*64 + kg*16 + b,
// re-biased to s8, or 0 outside the real channel / reduction range.  With fold (k <= 32, one k-step) the slots
// 32 + kk, kk < k, hold the s8 value fold_value instead: the kernel feeds them a second copy of the activations.
template <typename WAt>
inline void pack_group(uint8_t *dst, int32_t *wsum, int g_oc, int k, int ksteps, int tiles, int nchunks, WAt w_at, bool fold = false,
                       int fold_value = 0) {
    for (int oc = 0; oc < g_oc; oc++) {
        int32_t s = 0;
        for (int kk = 0; kk < k; kk++) s += (int32_t)(int8_t)(w_at(oc, kk) ^ 0x80);
        wsum[oc] = s;
    }
    for (int chunk = 0; chunk < nchunks; chunk++)
        for (int ks = 0; ks < ksteps; ks++)
            for (int nt = 0; nt < tiles; nt++) {
                uint8_t *frag = dst + (((size_t)chunk * ksteps + ks) * tiles + nt) * 1024;
                for (int kg = 0; kg < 4; kg++)
                    for (int i = 0; i < 16; i++) {
                        const int oc = chunk * 16 * tiles + (i / 4) * 4 * tiles + nt * 4 + (i % 4);
                        for (int b = 0; b < 16; b++) {
                            const int kk = ks * 64 + kg * 16 + b;
                            uint8_t v = 0;
                            if (oc < g_oc && kk < k) v = (uint8_t)(w_at(oc, kk) ^ 0x80);
                            if (fold && kk >= 32 && kk - 32 < k) v = (uint8_t)(int8_t)fold_value;
                            frag[(kg * 16 + i) * 16 + b] = v;
                        }
                    }
            }
}

// f(std::integral_constant<int, I>) for I = first .. N - 1, as straight-line code: an index into a register array
// stays a compile-time constant even where the optimiser would decline to unroll a loop of this size.
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>());
        static_for<I + 1, N>(f);
    }
}

struct PixInfo {
    int base; // kRows16: pixel index; other modes: pixel index of the image origin; < 0: no such pixel
    int iy0, ix0;
};

// One of two pixel records by value: a conditional expression over the named records would be an lvalue
// and could be placed in memory.
__device__ __forceinline__ PixInfo select_pix(bool first, PixInfo a, PixInfo b) {
    PixInfo r;
    r.base = first ? a.base : b.base;
    r.iy0 = first ? a.iy0 : b.iy0;
    r.ix0 = first ? a.ix0 : b.ix0;
    return r;
}

template <int MODE> __device__ __forceinline__ PixInfo pix_info(const IgemmArgs &a, int p) {
    PixInfo pi;
    pi.iy0 = pi.ix0 = 0;
    if (p >= a.m) {
        pi.base = -1;
        return pi;
    }
    if (loads_rows(MODE)) {
        pi.base = p;
        return pi;
    }
    const uint32_t img = fastdiv((uint32_t)p, a.d_ohow);
    const uint32_t rem = (uint32_t)p - img * a.d_ohow.div;
    const uint32_t oy = fastdiv(rem, a.d_ow);
    const uint32_t ox = rem - oy * a.d_ow.div;
    pi.base = (int)img * a.in_h * a.in_w;
    pi.iy0 = (int)oy * a.stride_h - a.pad_h;
    pi.ix0 = (int)ox * a.stride_w - a.pad_w;
    return pi;
}

// Location of the input element that reduction index kk of pixel `pi` reads.  The returned
// offset is always inside the tensor (coordinates are clamped); `inside` tells whether the
// tap really lies in the image or in the padding.
__device__ __forceinline__ uint32_t tap_offset(const IgemmArgs &a, const PixInfo &pi, int kk, bool *inside) {
    const uint32_t tap = fastdiv((uint32_t)kk, a.d_gic);
    const int c = kk - (int)tap * a.g_ic;
    const uint32_t ky = fastdiv(tap, a.d_kw);
    const int kx = (int)tap - (int)ky * a.kw;
    const int iy = pi.iy0 + (int)ky * a.dil_h;
    const int ix = pi.ix0 + kx * a.dil_w;
    *inside = (unsigned)iy < (unsigned)a.in_h && (unsigned)ix < (unsigned)a.in_w;
    const int cy = min(max(iy, 0), a.in_h - 1), cx = min(max(ix, 0), a.in_w - 1);
    return (uint32_t)(pi.base + cy * a.in_w + cx) * (uint32_t)a.ldx + a.x_coff + c;
}

// A 16-byte slice of the activation operand in flight.  The load is issued
// unconditionally from an address that is always valid; what the slice should have
// contained where the load does not apply (padding taps: the zero point; reduction
// indices past K or pixels past M: x' = 0) is kept in `fill` / `take` and applied only
// when the slice is consumed, so nothing depends on the loaded data until then and the
// load stays in flight across the multiply of the previous slice.
struct ActFrag {
    u32x4 raw;     // loaded bytes
    u32x4 fill;    // replacement per dword
    uint32_t take; // bit d set: dword d comes from raw
};

__device__ __forceinline__ v4i finish_act(const ActFrag &f) {
    u32x4 r;
    r[0] = (f.take & 1u) ? f.raw[0] : f.fill[0];
    r[1] = (f.take & 2u) ? f.raw[1] : f.fill[1];
    r[2] = (f.take & 4u) ? f.raw[2] : f.fill[2];
    r[3] = (f.take & 8u) ? f.raw[3] : f.fill[3];
    r ^= 0x80808080u;
    return __builtin_bit_cast(v4i, r);
}

template <int MODE> __device__ __forceinline__ ActFrag load_act(const IgemmArgs &a, const PixInfo &pi, int kc) {
    const u32x4 zero_s8 = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u}; // x' = 0
    ActFrag f;
    f.take = 0;
    f.raw = zero_s8;
    f.fill = zero_s8;
    const bool pix_ok = pi.base >= 0;
    PixInfo sp = pi; // any valid pixel for the address
    if (!pix_ok) sp.base = 0, sp.iy0 = 0, sp.ix0 = 0;
    if (loads_rows(MODE)) {
        const bool in_k = kc * 16 < a.k;
        const int kcc = in_k ? kc : 0;
        const uint32_t off = (uint32_t)sp.base * (uint32_t)a.ldx + a.x_coff + kcc * 16;
        if (MODE == kRows16) {
            f.raw = *reinterpret_cast<const u32x4 *>(a.x + (size_t)off);
            f.take = (pix_ok && in_k) ? 0xfu : 0u;
        } else {
            // The last slice of a pixel ends 8 bytes past its channels,
            // in the next pixel (those two dwords are replaced) or, for the tensor's last pixel, past the tensor:
            // that one slice is read 8 bytes lower and moved up, so that nothing outside the tensor is touched.
            const bool over = (size_t)off + 16 > a.x_bytes;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(a.x + (size_t)(over ? off - 8 : off));
            f.raw = u32x4{over ? v[2] : v[0], over ? v[3] : v[1], v[2], v[3]};
            f.take = (pix_ok && in_k) ? (a.k - kcc * 16 >= 16 ? 0xfu : 0x3u) : 0u;
        }
    } else if (MODE == kBytes) {
        // byte gathers: assembled immediately (this loader does not overlap with the multiply)
        uint32_t w0 = 0x80808080u, w1 = 0x80808080u, w2 = 0x80808080u, w3 = 0x80808080u;
        if (pix_ok) {
#pragma unroll
            for (int b = 0; b < 16; b++) {
                const int kk = kc * 16 + b;
                if (kk < a.k) {
                    bool inside;
                    const uint32_t off = tap_offset(a, pi, kk, &inside);
                    const uint32_t byte = inside ? (uint32_t)a.x[(size_t)off] : (a.zx_splat & 0xffu);
                    const uint32_t clr = ~(0xffu << (8 * (b & 3))), ins = byte << (8 * (b & 3));
                    if ((b >> 2) == 0) w0 = (w0 & clr) | ins;
                    if ((b >> 2) == 1) w1 = (w1 & clr) | ins;
                    if ((b >> 2) == 2) w2 = (w2 & clr) | ins;
                    if ((b >> 2) == 3) w3 = (w3 & clr) | ins;
                }
            }
        }
        f.fill = u32x4{w0, w1, w2, w3};
    } else {
        constexpr int VW = MODE == kVec16 ? 16 : (MODE == kVec8 ? 8 : 4);
#pragma unroll
        for (int piece = 0; piece < 16 / VW; piece++) {
            const int kk = kc * 16 + piece * VW;
            const bool in_k = kk < a.k;
            bool inside;
            const uint32_t off = tap_offset(a, sp, in_k ? kk : 0, &inside);
            const bool ok = pix_ok && in_k && inside;
            const uint32_t fill = (pix_ok && in_k) ? a.zx_splat : 0x80808080u; // padding tap : outside the problem
            if (VW == 16) {
                f.raw = *reinterpret_cast<const u32x4 *>(a.x + (size_t)off);
                f.fill = u32x4{fill, fill, fill, fill};
                f.take = ok ? 0xfu : 0u;
            } else if (VW == 8) {
                const u32x2 v = *reinterpret_cast<const u32x2 *>(a.x + (size_t)off);
                f.raw[piece * 2] = v[0], f.raw[piece * 2 + 1] = v[1];
                f.fill[piece * 2] = fill, f.fill[piece * 2 + 1] = fill;
                f.take |= ok ? (3u << (piece * 2)) : 0u;
            } else {
                f.raw[piece] = *reinterpret_cast<const uint32_t *>(a.x + (size_t)off);
                f.fill[piece] = fill;
                f.take |= ok ? (1u << piece) : 0u;
            }
        }
    }
    return f;
}

struct ActSlice { // vec16 / rows16: one 16-byte load per k-step, one fill value
    u32x4 raw;
    uint32_t fill;
    uint32_t take; // 0 or ~0
};

template <int MODE> __device__ __forceinline__ ActSlice load_slice(const IgemmArgs &a, const PixInfo &pi, int kc) {
    static_assert(MODE == kRows16 || MODE == kVec16, "one 16-byte piece per slice");
    ActSlice f;
    const bool pix_ok = pi.base >= 0;
    PixInfo sp = pi;
    if (!pix_ok) sp.base = 0, sp.iy0 = 0, sp.ix0 = 0;
    const bool in_k = kc * 16 < a.k;
    if (MODE == kRows16) {
        f.raw = *reinterpret_cast<const u32x4 *>(a.x + (size_t)((uint32_t)sp.base * (uint32_t)a.ldx + a.x_coff + (in_k ? kc : 0) * 16));
        f.fill = 0x80808080u;
        f.take = (pix_ok && in_k) ? ~0u : 0u;
    } else {
        bool inside;
        const uint32_t off = tap_offset(a, sp, in_k ? kc * 16 : 0, &inside);
        f.raw = *reinterpret_cast<const u32x4 *>(a.x + (size_t)off);
        f.fill = (pix_ok && in_k) ? a.zx_splat : 0x80808080u; // padding tap : outside the problem
        f.take = (pix_ok && in_k && inside) ? ~0u : 0u;
    }
    return f;
}

__device__ __forceinline__ v4i finish_slice(const ActSlice &f) {
    u32x4 r;
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = ((f.raw[d] & f.take) | (f.fill & ~f.take)) ^ 0x80808080u;
    return __builtin_bit_cast(v4i, r);
}

// The activation operand in flight, by loader: the 16-byte loaders need one fill value and an all-or-nothing mask
// (one bit operation and one xor per dword when the slice is consumed), the gathering loaders a fill and a bit per dword.
template <int MODE> struct ActOf {
    using type = ActFrag;
};
template <> struct ActOf<kRows16> {
    using type = ActSlice;
};
template <> struct ActOf<kVec16> {
    using type = ActSlice;
};
template <int MODE> __device__ __forceinline__ typename ActOf<MODE>::type load_operand(const IgemmArgs &a, const PixInfo &pi, int kc) {
    if constexpr (MODE == kRows16 || MODE == kVec16) return load_slice<MODE>(a, pi, kc);
    else return load_act<MODE>(a, pi, kc);
}
__device__ __forceinline__ v4i finish_operand(const ActFrag &f) { return finish_act(f); }
__device__ __forceinline__ v4i finish_operand(const ActSlice &f) { return finish_slice(f); }
__device__ __forceinline__ void clear_operand(ActFrag &f) {
    f.raw = f.fill = u32x4{0, 0, 0, 0};
    f.take = 0;
}
__device__ __forceinline__ void clear_operand(ActSlice &f) {
    f.raw = u32x4{0, 0, 0, 0};
    f.fill = 0, f.take = 0;
}

struct __attribute__((packed, aligned(1))) U32Unaligned {
    uint32_t v;
};

// Epilogue of one 16-pixel x 16T-channel tile of a wave: zero-point correction, requantisation
// (optionally a byte table and a residual add behind it), NHWC store.  Lane (j, gq) holds pixel p
// and the 4T consecutive channels from ch0 on; rowsum is the pixel's sum of x' over the reduction.
// OWED says what acc still lacks: kOwesAll, the channel constant (read at cterm) and -zwp * rowsum; kOwesRows, only
// -zwp_rows * rowsum; kOwesNothing.
enum { kOwesAll = 0, kOwesRows = 1, kOwesNothing = 2 };
// PLAIN: the launch has been checked to need none of the options -- u8 output by the one-instruction requantisation
// (Epilogue::fast and ::full), no byte table, no residual, whole groups of 4T channels, dword-aligned rows -- so the
// tile is converted and stored without a single test of them.
// Dword outputs (float32 / int32) of a wave's 16 pixels x 16T channels.  A lane holds 4T consecutive channels of one
// pixel, so a 16-byte store of all lanes touches 64 different places, 16 bytes each (measured on the 255-channel
// detection heads: 1.6 TB/s).  Instead, four channel tiles at a time, every lane puts its 64 bytes into the wave's LDS
// staging area and the wave writes them out with four lanes per 64-byte run: a store instruction then covers 16
// whole 64-byte runs.  LDS operations of a wave execute in order, so the phases need neither a barrier nor a wait
// beyond the one in front of the first use of the data read back.
constexpr bool staged_store_built(int T) { return T % 4 == 0; }
constexpr int kStagedRun = 64 + 16;                       // a lane's run and its padding against bank conflicts
constexpr int staged_store_bytes() { return 64 * kStagedRun; } // per wave

// o: the lane's values of channel tiles 4g .. 4g + 3 (channels ch0 + 16 g + [0, 16) of pixel p)
__device__ __forceinline__ void store_dword_group(const IgemmArgs &a, const uint32_t (&o)[4][4], int g, int p, int ch0, int gq, uint8_t *stage,
                                                  int quarter_stride) {
    // (quarter_stride: channels between the lanes' quarters, 4T unless waves side by side share the chunk)
    const int lane = threadIdx.x & 63;
    const int j = lane & 15;
    const int p_first = p - j, ch_first = ch0 - gq * quarter_stride;
    uint32_t *yo = reinterpret_cast<uint32_t *>(a.y);
#pragma unroll
    for (int k = 0; k < 4; k++) *reinterpret_cast<u32x4 *>(stage + (j * 4 + gq) * kStagedRun + k * 16) = u32x4{o[k][0], o[k][1], o[k][2], o[k][3]};
    const int u = lane & 3, qq = (lane >> 2) & 3, psub = lane >> 4;
    const int ch = ch_first + qq * quarter_stride + g * 16 + u * 4;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int row = it * 4 + psub;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + (row * 4 + qq) * kStagedRun + u * 16);
        const int pp = p_first + row;
        if (pp < a.m) {
            uint32_t *dst = yo + ((size_t)pp * a.ldy + a.y_coff + ch);
            if (ch + 4 <= a.n) {
                *reinterpret_cast<u32x4_a4 *>(dst) = u32x4_a4{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (ch + r < a.n) dst[r] = v[r];
            }
        }
    }
}

// STAGED: the kernel has a staging area per wave for the dword outputs (store_dword_group); the lane-by-lane dword
// stores are then not built.
// MAGIC (with PLAIN): the accumulators were started from kMagicBias and are requantised as floats (Epilogue::magic).
template <int T, int OWED = kOwesAll, bool PLAIN = false, bool STAGED = false, bool MAGIC = false>
__device__ __forceinline__ void igemm_store_tile(const IgemmArgs &a, const v4i (&acc)[T], int32_t rowsum, int p, int ch0, int gq,
                                                 const int32_t *cterm, const uint8_t *lutl, uint8_t *stage = nullptr,
                                                 int quarter_stride = 4 * T) {
    static_assert(!STAGED || (!PLAIN && staged_store_built(T)), "staged stores move four channel tiles at a time");
    static_assert(!MAGIC || PLAIN, "the magic-bias form exists for the option-free epilogue only");
    // (with a staging area every lane of the wave takes part in the stores, whatever it holds itself)
    const bool staged = STAGED && (a.deq || a.ep.out_mode != kOutU8);
    const bool live = p < a.m && ch0 < a.n;
    if (!live && !staged) return;
    const int32_t nrsz = OWED == kOwesAll ? -a.zwp * rowsum : (OWED == kOwesRows ? -a.zwp_rows * rowsum : 0);
    const size_t obase = (size_t)p * a.ldy + a.y_coff + ch0;
    if constexpr (PLAIN) {
        uint32_t *yo = reinterpret_cast<uint32_t *>(reinterpret_cast<uint8_t *>(a.y) + obase);
        uint32_t packed[T];
#pragma unroll
        for (int nt = 0; nt < T; nt++) {
            v4i ct = {0, 0, 0, 0};
            if (OWED == kOwesAll) ct = *reinterpret_cast<const v4i *>(cterm + gq * (4 * T) + nt * 4);
            int32_t v[4];
#pragma unroll
            for (int r = 0; r < 4; r++)
                v[r] = OWED == kOwesAll ? add3(acc[nt][r], ct[r], nrsz) : (OWED == kOwesRows ? acc[nt][r] + nrsz : acc[nt][r]);
            packed[nt] = MAGIC ? requant4_u8_packed_magic(v, a.ep) : requant4_u8_packed_direct(v, a.ep);
        }
#pragma unroll
        for (int nt = 0; nt + 4 <= T; nt += 4)
            *reinterpret_cast<u32x4_a4 *>(yo + nt) = u32x4_a4{packed[nt], packed[nt + 1], packed[nt + 2], packed[nt + 3]};
#pragma unroll
        for (int nt = T / 4 * 4; nt < T; nt++) yo[nt] = packed[nt];
        return;
    }
    if (a.ep.out_mode == kOutU8) {
        uint8_t *yo = reinterpret_cast<uint8_t *>(a.y) + obase;
        uint32_t packed[T];
#pragma unroll
        for (int nt = 0; nt < T; nt++) {
            v4i ct = {0, 0, 0, 0};
            if (OWED == kOwesAll) ct = *reinterpret_cast<const v4i *>(cterm + gq * (4 * T) + nt * 4);
            int32_t v[4];
#pragma unroll
            for (int r = 0; r < 4; r++)
                v[r] = OWED == kOwesAll ? add3(acc[nt][r], ct[r], nrsz) : (OWED == kOwesRows ? acc[nt][r] + nrsz : acc[nt][r]);
            packed[nt] = requant4_u8_packed(v, a.ep);
        }
        if (a.lut) { // fused unary operator: one LDS byte read per output
#pragma unroll
            for (int nt = 0; nt < T; nt++) {
                const uint32_t v = packed[nt];
                packed[nt] = (uint32_t)lutl[v & 0xffu] | ((uint32_t)lutl[(v >> 8) & 0xffu] << 8) |
                             ((uint32_t)lutl[(v >> 16) & 0xffu] << 16) | ((uint32_t)lutl[v >> 24] << 24);
            }
        }
        if (a.rep.res && live) { // fused residual add on the requantised bytes
            const uint8_t *ro = a.rep.res + ((size_t)p * a.ldr + a.r_coff + ch0);
            const bool whole = ((a.ldr | a.r_coff) & 3) == 0 && ch0 + 4 * T <= a.n;
#pragma unroll
            for (int nt = 0; nt < T; nt++) {
                uint32_t rv = 0;
                if (whole) {
                    rv = *reinterpret_cast<const uint32_t *>(ro + nt * 4);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (ch0 + nt * 4 + r < a.n) rv |= (uint32_t)ro[nt * 4 + r] << (8 * r);
                }
                packed[nt] = residual4_packed(packed[nt], rv, a.rep);
            }
        }
        if (a.deq) { // the Dequantize behind the convolution: one float per channel
            if constexpr (STAGED) {
#pragma unroll
                for (int g = 0; g < T / 4; g++) {
                    uint32_t o[4][4];
#pragma unroll
                    for (int k = 0; k < 4; k++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            o[k][r] = __float_as_uint((float)((int)((packed[g * 4 + k] >> (8 * r)) & 0xffu) - a.deq_zero) * a.deq_scale);
                    store_dword_group(a, o, g, p, ch0, gq, stage, quarter_stride);
                }
            } else {
                float *fo = reinterpret_cast<float *>(a.y) + obase;
#pragma unroll
                for (int nt = 0; nt < T; nt++) {
                    uint32_t o[4];
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        o[r] = __float_as_uint((float)((int)((packed[nt] >> (8 * r)) & 0xffu) - a.deq_zero) * a.deq_scale);
                    if (ch0 + nt * 4 + 4 <= a.n) {
                        *reinterpret_cast<u32x4_a4 *>(fo + nt * 4) = u32x4_a4{o[0], o[1], o[2], o[3]};
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (ch0 + nt * 4 + r < a.n) fo[nt * 4 + r] = __uint_as_float(o[r]);
                    }
                }
            }
            return;
        }
        if (((a.ldy | a.y_coff) & 3) == 0 && ch0 + 4 * T <= a.n) {
#pragma unroll
            for (int nt = 0; nt < T; nt += 4) {
                if (nt + 4 <= T) {
                    *reinterpret_cast<u32x4_a4 *>(yo + nt * 4) =
                        u32x4_a4{packed[nt], packed[nt + 1 < T ? nt + 1 : nt], packed[nt + 2 < T ? nt + 2 : nt],
                                 packed[nt + 3 < T ? nt + 3 : nt]};
                } else {
#pragma unroll
                    for (int e = nt; e < T; e++) *reinterpret_cast<uint32_t *>(yo + e * 4) = packed[e];
                }
            }
        } else if (ch0 + 4 * T <= a.n) {
            // a channel count that is no multiple of 4 (255-channel detection heads): pixel rows start at
            // any byte, the lane's 4T bytes still go out as dwords (the memory system takes unaligned dwords)
#pragma unroll
            for (int nt = 0; nt < T; nt++) reinterpret_cast<U32Unaligned *>(yo + nt * 4)->v = packed[nt];
        } else {
#pragma unroll
            for (int nt = 0; nt < T; nt++)
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (ch0 + nt * 4 + r < a.n) yo[nt * 4 + r] = (uint8_t)(packed[nt] >> (8 * r));
        }
    } else {
        // int32 accumulators or clamped fp32, one dword per channel
        auto value = [&](int nt, int r) __attribute__((always_inline)) -> uint32_t {
            const int32_t ct = OWED == kOwesAll ? cterm[gq * (4 * T) + nt * 4 + r] : 0;
            const int32_t v = OWED == kOwesAll ? add3(acc[nt][r], ct, nrsz) : (OWED == kOwesRows ? acc[nt][r] + nrsz : acc[nt][r]);
            return a.ep.out_mode == kOutI32 ? (uint32_t)v : __float_as_uint(clamp_ref((float)v * a.ep.mult, a.ep.lo, a.ep.hi));
        };
        if constexpr (STAGED) {
#pragma unroll
            for (int g = 0; g < T / 4; g++) {
                uint32_t o[4][4];
#pragma unroll
                for (int k = 0; k < 4; k++)
#pragma unroll
                    for (int r = 0; r < 4; r++) o[k][r] = value(g * 4 + k, r);
                store_dword_group(a, o, g, p, ch0, gq, stage, quarter_stride);
            }
        } else {
            uint32_t *yo = reinterpret_cast<uint32_t *>(a.y) + obase;
#pragma unroll
            for (int nt = 0; nt < T; nt++) {
                uint32_t o[4];
#pragma unroll
                for (int r = 0; r < 4; r++) o[r] = value(nt, r);
                if (ch0 + nt * 4 + 4 <= a.n) {
                    *reinterpret_cast<u32x4_a4 *>(yo + nt * 4) = u32x4_a4{o[0], o[1], o[2], o[3]};
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (ch0 + nt * 4 + r < a.n) yo[nt * 4 + r] = o[r];
                }
            }
        }
    }
}

// Blocks per compute unit the register allocation has to leave room for: four (at most 128 registers) for the
// shapes that fit comfortably, so that the scheduler does not trade the occupancy away for longer live ranges.
// STAGED: built for dword outputs (float32 / int32 / the dequantised u8 result), which go through a staging area per
// wave behind the weights; a kernel of its own because the staged stores raise the register count of the whole kernel.
template <int T, int RG, int MODE, bool PLAIN = false, bool STAGED = false>
__global__ void __launch_bounds__(kThreads, (STAGED && T >= 12) ? 2 : (((RG == 1 && T <= 12) || loads_rows(MODE)) ? 4 : 2)) qconv_igemm_kernel(const IgemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int32_t *cterm = reinterpret_cast<int32_t *>(smem); // [T * 16]
    uint8_t *lutl = smem + T * 16 * sizeof(int32_t);    // [256] byte table of the fused unary operator
    uint8_t *wlds = lutl + 256;                         // [kc_steps][T][1024]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    // dword outputs: a staging area per wave behind the weights (see store_dword_rows), when the launch asked for one
    static_assert(!STAGED || (!PLAIN && staged_store_built(T)), "staged stores move four channel tiles at a time");
    uint8_t *const stage = wlds + (size_t)a.kc_steps * T * 1024 + wave * staged_store_bytes(); // (reserved by the launch of a STAGED kernel)
    const int j = lane & 15;  // pixel within a group of 16
    const int gq = lane >> 4; // k-quarter on the load side, channel quarter on the store side
    const int chunk = blockIdx.y;
    const int ch_base = chunk * (T * 16);
    const uint8_t *wsrc = a.wpk + (size_t)chunk * a.ksteps * T * 1024;
    const int nkc = (a.ksteps + a.kc_steps - 1) / a.kc_steps;

    // ---- set-up: every load it needs is issued before the first is used, in the order of use (constants, table,
    // weights, first activation slices): a block with one or two pixel tiles is a chain of memory round trips,
    // and this makes the set-up one of them ----
    auto stage_weights = [&](int kci, int first) {
        const int s0 = kci * a.kc_steps;
        const int steps = min(a.kc_steps, a.ksteps - s0);
        const u32x4 *src = reinterpret_cast<const u32x4 *>(wsrc + (size_t)s0 * T * 1024);
        u32x4 *dst = reinterpret_cast<u32x4 *>(wlds);
        // four loads in flight per thread before the first is stored
        const int n = steps * T * 64;
        for (int i = first + threadIdx.x; i < n; i += 4 * kThreads) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * kThreads < n) v[u] = src[i + u * kThreads];
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * kThreads < n) dst[i + u * kThreads] = v[u];
        }
    };
    // per-channel constant of the zero-point identity, in the lane order the epilogue reads it:
    // position gq' * 4T + nt * 4 + r <-> channel ch_base + same (T * 16 <= kThreads: one per thread)
    static_assert(T * 16 <= kThreads, "one constant per thread");
    int32_t c_bias = 0, c_wsum = 0;
    const bool c_mine = (int)threadIdx.x < T * 16, c_real = c_mine && ch_base + (int)threadIdx.x < a.n;
    if (c_real) c_bias = a.bias[ch_base + threadIdx.x], c_wsum = a.wsum[ch_base + threadIdx.x];
    uint32_t lut_word = 0;
    const bool lut_mine = a.lut && threadIdx.x < 64;
    if (lut_mine) lut_word = a.lut[threadIdx.x];
    u32x4 w_first[4];
    const int n_first = nkc == 1 ? a.ksteps * T * 64 : 0; // the first 4 * kThreads fragments' vectors of a resident chunk
#pragma unroll
    for (int u = 0; u < 4; u++)
        if ((int)threadIdx.x + u * kThreads < n_first) w_first[u] = reinterpret_cast<const u32x4 *>(wsrc)[threadIdx.x + u * kThreads];

    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    constexpr int pix_per_block = kWaves * RG * 16;

    PixInfo pcur[RG], pnxt[RG];
    using Act = typename ActOf<MODE>::type;
    Act fcur[RG], fnxt[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        pnxt[rg].base = -1;
        pnxt[rg].iy0 = pnxt[rg].ix0 = 0;
        clear_operand(fnxt[rg]);
    }
    int mt = blockIdx.x;
    if (mt < a.num_mtiles) {
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            pcur[rg] = pix_info<MODE>(a, mt * pix_per_block + (wave * RG + rg) * 16 + j);
            fcur[rg] = load_operand<MODE>(a, pcur[rg], gq & a.kc_mask);
        }
    }
    if (c_mine) cterm[threadIdx.x] = c_real ? c_bias - a.zxp * c_wsum + a.k * a.zxp * a.zwp : 0;
    if (lut_mine) reinterpret_cast<uint32_t *>(lutl)[threadIdx.x] = lut_word;
#pragma unroll
    for (int u = 0; u < 4; u++)
        if ((int)threadIdx.x + u * kThreads < n_first) reinterpret_cast<u32x4 *>(wlds)[threadIdx.x + u * kThreads] = w_first[u];
    if (nkc == 1) stage_weights(0, 4 * kThreads);
    __syncthreads();

#pragma clang loop unroll(disable)
    for (; mt < a.num_mtiles; mt += gridDim.x) {
        // The sums start from the per-channel constant of the zero-point identity, read from LDS for every tile
        // (the offset is hidden from the optimiser: kept in registers across tiles the constants would cost 4T of them).
        v4i acc[RG][T];
        v4i rs[RG];
        int ct_off = gq * (4 * T);
        asm volatile("" : "+v"(ct_off));
#pragma unroll
        for (int nt = 0; nt < T; nt++) {
            const v4i ct = *reinterpret_cast<const v4i *>(cterm + ct_off + nt * 4);
#pragma unroll
            for (int rg = 0; rg < RG; rg++) acc[rg][nt] = ct;
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) rs[rg] = v4i{0, 0, 0, 0};
        const int mt_next = mt + gridDim.x;
        // One pixel tile per block and a long reduction (the 7x7 layers, the classifier): the block is a chain of
        // k-steps, each as long as a memory round trip if only one slice is in flight.  Three register sets then
        // take the slices in turn (no copies between them: a copy would wait for the loads it copies).
        bool deep = false;
        constexpr bool kDeepBuilt = RG == 1 && T <= 6 && MODE == kRows16; // (wider chunks and the gathering loaders have no registers to spare)
        if constexpr (kDeepBuilt) deep = nkc == 1 && a.ksteps >= 4 && a.num_mtiles <= (int)gridDim.x;
        if (deep) {
            if constexpr (kDeepBuilt) {
                Act f1 = load_operand<MODE>(a, pcur[0], (4 + gq) & a.kc_mask), f2 = load_operand<MODE>(a, pcur[0], (8 + gq) & a.kc_mask);
                int ks = 0;
                auto step = [&](Act &f) __attribute__((always_inline)) {
                    const v4i xf = finish_operand(f);
                    const int nk = ks + 3 < a.ksteps ? ks + 3 : 0; // past the end: a valid slice, dropped
                    f = load_operand<MODE>(a, pcur[0], (nk * 4 + gq) & a.kc_mask);
                    rs[0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, xf, rs[0], 0, 0, 0);
                    const uint8_t *wstep = wlds + (size_t)ks * T * 1024 + lane * 16;
#pragma unroll
                    for (int nt = 0; nt < T; nt++) {
                        const v4i wf = *reinterpret_cast<const v4i *>(wstep + nt * 1024);
                        acc[0][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf, acc[0][nt], 0, 0, 0);
                    }
                    ks++;
                };
                for (;;) {
                    step(fcur[0]);
                    if (ks >= a.ksteps) break;
                    step(f1);
                    if (ks >= a.ksteps) break;
                    step(f2);
                    if (ks >= a.ksteps) break;
                }
            }
        } else
#pragma clang loop unroll(disable)
        for (int kci = 0; kci < nkc; kci++) {
            if (nkc > 1) {
                __syncthreads(); // previous stage fully consumed
                stage_weights(kci, 0);
                __syncthreads();
            }
            const int s0 = kci * a.kc_steps;
            const int s1 = min(a.ksteps, s0 + a.kc_steps);
#pragma clang loop unroll(disable)
            for (int ks = s0; ks < s1; ks++) {
                // Issue the loads of the next fragment before multiplying this one: the next k-step of this pixel
                // tile, or the first of the next tile.  The loads are issued on every trip (after the last tile
                // they re-read a valid address and the data is dropped): loads complete in order, and only a
                // compile-time count of younger loads lets the wait below spare the ones just issued.
                {
                    const bool same_tile = ks + 1 < a.ksteps;
                    if (!same_tile) {
                        const int mtn = mt_next < a.num_mtiles ? mt_next : mt;
#pragma unroll
                        for (int rg = 0; rg < RG; rg++) pnxt[rg] = pix_info<MODE>(a, mtn * pix_per_block + (wave * RG + rg) * 16 + j);
                    }
                    const int kc_next = (same_tile ? (ks + 1) * 4 + gq : gq) & a.kc_mask;
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) fnxt[rg] = load_operand<MODE>(a, select_pix(same_tile, pcur[rg], pnxt[rg]), kc_next);
                }
                v4i xf[RG]; // the slice loaded one step ago, now needed
#pragma unroll
                for (int rg = 0; rg < RG; rg++) xf[rg] = finish_operand(fcur[rg]);
                { // sum of x' per pixel (not needed where the weights carry the term it is for; a branch here costs more)
#pragma unroll
                    for (int rg = 0; rg < RG; rg++)
                        rs[rg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, xf[rg], rs[rg], 0, 0, 0);
                }
                const uint8_t *wstep = wlds + (size_t)(ks - s0) * T * 1024 + lane * 16;
#pragma unroll
                for (int nt = 0; nt < T; nt++) {
                    const v4i wf = *reinterpret_cast<const v4i *>(wstep + nt * 1024);
#pragma unroll
                    for (int rg = 0; rg < RG; rg++)
                        acc[rg][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf[rg], acc[rg][nt], 0, 0, 0);
                }
#pragma unroll
                for (int rg = 0; rg < RG; rg++) fcur[rg] = fnxt[rg];
            }
        }

        // ---- epilogue: the rest of the zero-point correction, requantisation, NHWC store ----
        // (written out for both cases: one epilogue behind a conditional correction would keep two copies of the sums)
        const int ch0 = ch_base + gq * (4 * T); // first of this lane's 4T channels
        if (a.zwp_rows != 0) {
            static_for<0, RG>([&](auto rg_c) __attribute__((always_inline)) {
                constexpr int rg = decltype(rg_c)::value;
                igemm_store_tile<T, kOwesRows, PLAIN, STAGED>(a, acc[rg], rs[rg][0], mt * pix_per_block + (wave * RG + rg) * 16 + j, ch0, gq, cterm, lutl, stage);
            });
        } else {
            static_for<0, RG>([&](auto rg_c) __attribute__((always_inline)) {
                constexpr int rg = decltype(rg_c)::value;
                igemm_store_tile<T, kOwesNothing, PLAIN, STAGED>(a, acc[rg], 0, mt * pix_per_block + (wave * RG + rg) * 16 + j, ch0, gq, cterm, lutl, stage);
            });
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++) pcur[rg] = pnxt[rg];
    }
}

// ---- 1x1 convolutions over a multiple of 16 channels whose epilogue needs none of the options ----
// The same implicit GEMM with everything that a pixel row does not need taken out of the loop: the activation
// operand of (pixel, k-step) is 16 bytes at pixel * ldx + k-step * 64 + quad * 16, fetched by a buffer load whose
// vector offset (the pixel's) is computed once per tile and whose scalar offset is the k-step; it is used as loaded
// (one xor per dword makes it s8): reduction indices past K meet zero weights, and the row sum the weight zero point
// multiplies comes from a ones operand that is zero past K, so nothing is masked; pixels past M are computed on a
// clamped address and not stored.  The first k-step of a tile starts the sums from the channel constants (the
// accumulator operand of the first product), so they are not copied.  One slice per pixel group is in flight ahead
// of the products.  ROWS: the epilogue still owes -zw' * (sum of x'); false where the weights carry that term
// (reductions of at most 32: the lanes of the upper half of the only k-step then re-read the pixel's bytes).
// MAGIC: the sums start from kMagicBias on top of the channel constants and the epilogue reads them as floats.
template <int T, int RG, bool ROWS, bool MAGIC> __global__ void __launch_bounds__(kThreads, 4) qconv_rows_kernel(const IgemmArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int32_t *cterm = reinterpret_cast<int32_t *>(smem); // [T * 16]
    uint8_t *wlds = smem + T * 16 * sizeof(int32_t);    // [ksteps][T][1024]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j = lane & 15, gq = lane >> 4;
    const int chunk = blockIdx.y;
    const int ch_base = chunk * (T * 16);
    const int KS = a.ksteps;
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);

    // constants and the chunk's weights -> LDS
    static_assert(T * 16 <= kThreads, "one constant per thread");
    if ((int)threadIdx.x < T * 16) {
        const int ch = ch_base + threadIdx.x;
        cterm[threadIdx.x] = (ch < a.n ? a.bias[ch] - a.zxp * a.wsum[ch] + a.k * a.zxp * a.zwp : 0) + (MAGIC ? kMagicBias : 0);
    }
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.wpk + (size_t)chunk * KS * T * 1024);
        u32x4 *dst = reinterpret_cast<u32x4 *>(wlds);
        const int n = KS * T * 64;
        for (int i = threadIdx.x; i < n; i += 4 * kThreads) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * kThreads < n) v[u] = src[i + u * kThreads];
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * kThreads < n) dst[i + u * kThreads] = v[u];
        }
    }

    // this lane's 16-byte slice of a pixel row: full k-steps take (k-step * 4 + quad), the last one may end before
    // the quad's slice (then the slice re-reads the row's first bytes and meets zero weights and a zero ones operand)
    const int last = KS - 1;
    const int tail_chunk = (last * 4 + gq) & a.kc_mask;
    const bool tail_in_k = tail_chunk * 16 < a.k;
    const uint32_t tail_off = tail_in_k ? (uint32_t)tail_chunk * 16u : 0u;
    const uint32_t quad_off = (uint32_t)gq * 16u;
    const int one = (ROWS && tail_in_k) ? 0x01010101 : 0;
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101}, ones_tail = {one, one, one, one};
    constexpr int pix_per_block = kWaves * RG * 16;

    auto pixel_off = [&](int mt, int rg) { // byte offset of the lane's pixel of tile mt (clamped into the tensor)
        const int p = min(mt * pix_per_block + (wave * RG + rg) * 16 + j, a.m - 1);
        return (uint32_t)p * (uint32_t)a.ldx + (uint32_t)a.x_coff;
    };
    auto load = [&](uint32_t poff, int ks) { // slice of k-step ks
        return ks == last ? __builtin_amdgcn_raw_buffer_load_b128(xres, poff + tail_off, 0, 0)
                          : __builtin_amdgcn_raw_buffer_load_b128(xres, poff + quad_off, ks * 64, 0);
    };

    int mt = blockIdx.x;
    uint32_t poff[RG];
    u32x4 cur[RG];
    if (mt < a.num_mtiles) {
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            poff[rg] = pixel_off(mt, rg);
            cur[rg] = load(poff[rg], 0);
        }
    }
    __syncthreads();

    const int ch0 = ch_base + gq * (4 * T);
#pragma clang loop unroll(disable)
    for (; mt < a.num_mtiles; mt += gridDim.x) {
        v4i acc[RG][T];
        v4i rs[RG];
        const int mt_next = mt + gridDim.x < a.num_mtiles ? mt + gridDim.x : mt; // past the end: re-read this tile, dropped
        uint32_t poff_next[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) poff_next[rg] = pixel_off(mt_next, rg);
#pragma clang loop unroll(disable)
        for (int ks = 0; ks < KS; ks++) {
            // the next slices: the next k-step of this tile, or the first of the next tile
            u32x4 nxt[RG];
            const bool same_tile = ks < last;
#pragma unroll
            for (int rg = 0; rg < RG; rg++) nxt[rg] = load(same_tile ? poff[rg] : poff_next[rg], same_tile ? ks + 1 : 0);
            v4i xf[RG];
#pragma unroll
            for (int rg = 0; rg < RG; rg++) xf[rg] = __builtin_bit_cast(v4i, cur[rg] ^ 0x80808080u);
            const uint8_t *wstep = wlds + (size_t)ks * T * 1024 + lane * 16;
            if (ks == 0) {
                int ct_off = gq * (4 * T);
                asm volatile("" : "+v"(ct_off)); // (read per tile: kept in registers the constants would cost 4T of them)
#pragma unroll
                for (int nt = 0; nt < T; nt++) {
                    const v4i ct = *reinterpret_cast<const v4i *>(cterm + ct_off + nt * 4);
                    const v4i wf = *reinterpret_cast<const v4i *>(wstep + nt * 1024);
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) acc[rg][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf[rg], ct, 0, 0, 0);
                }
                if (ROWS) {
                    const v4i zero = {0, 0, 0, 0};
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) rs[rg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ks == last ? ones_tail : ones, xf[rg], zero, 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int nt = 0; nt < T; nt++) {
                    const v4i wf = *reinterpret_cast<const v4i *>(wstep + nt * 1024);
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) acc[rg][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf[rg], acc[rg][nt], 0, 0, 0);
                }
                if (ROWS) {
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) rs[rg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ks == last ? ones_tail : ones, xf[rg], rs[rg], 0, 0, 0);
                }
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) cur[rg] = nxt[rg];
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
            igemm_store_tile<T, ROWS ? kOwesRows : kOwesNothing, true, false, MAGIC>(a, acc[rg], ROWS ? rs[rg][0] : 0,
                                                                        mt * pix_per_block + (wave * RG + rg) * 16 + j, ch0, gq, cterm, nullptr);
#pragma unroll
        for (int rg = 0; rg < RG; rg++) poff[rg] = poff_next[rg];
    }
}

// ---- windows over a multiple of 16 channels, the chunk's weights resident in LDS ---------------------------
// The loader of qconv_igemm_kernel finds a slice's tap by two divisions per slice and clamps its coordinates; for
// the stems that read 2 x 2 pixel blocks as 16-channel pixels (a few taps, 32 output channels, 10^6 pixels per
// launch) that address arithmetic is most of the kernel.  Where the 16-byte slice kc of the reduction lies relative
// to a pixel's window origin is the same for all pixels: a table in LDS, built once per block, holds per slice the
// byte offset, the tap's row and column, and what the slice holds when the tap lies in the padding (the zero point)
// or past the reduction (x' = 0).  A lane's slice then costs two additions and two comparisons: it is read
// through the range-checked buffer path either from its address or, through an offset outside the buffer, as
// zeros that the fill value is or-ed into.  The sums start from the channel constants; the row sums that the weight
// zero point multiplies come from a ones operand.
struct WindowSlice {
    u32x4 raw;
    uint32_t fill; // 0 where raw holds the data
};

template <int T, int RG, bool PLAIN, bool MAGIC = false> __global__ void __launch_bounds__(kThreads, 4) qconv_window_kernel(const IgemmArgs a) {
    static_assert(!MAGIC || PLAIN, "the magic-bias form exists for the option-free epilogue only");
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int32_t *cterm = reinterpret_cast<int32_t *>(smem);    // [T * 16]
    uint8_t *lutl = smem + T * 16 * sizeof(int32_t);       // [256]
    v4i *taps = reinterpret_cast<v4i *>(lutl + 256);       // [ksteps * 4]: byte offset, row, column, fill
    const int KS = a.ksteps;
    uint8_t *wlds = reinterpret_cast<uint8_t *>(taps + KS * 4); // [ksteps][T][1024]

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int j = lane & 15, gq = lane >> 4;
    const int chunk = blockIdx.y;
    const int ch_base = chunk * (T * 16);
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(a.x), 0, (int)a.x_bytes, 0x00020000);

    static_assert(T * 16 <= kThreads, "one constant per thread");
    if ((int)threadIdx.x < T * 16) {
        const int ch = ch_base + threadIdx.x;
        cterm[threadIdx.x] = (ch < a.n ? a.bias[ch] - a.zxp * a.wsum[ch] + a.k * a.zxp * a.zwp : 0) + (MAGIC ? kMagicBias : 0);
    }
    if (!PLAIN && a.lut && threadIdx.x < 64) reinterpret_cast<uint32_t *>(lutl)[threadIdx.x] = a.lut[threadIdx.x];
    for (int e = threadIdx.x; e < KS * 4; e += kThreads) {
        const int kk = e * 16;
        v4i t = {0, 0x40000000, 0, (int)0x80808080u}; // past the reduction: never inside the image, x' = 0
        if (kk < a.k) {
            const uint32_t tap = fastdiv((uint32_t)kk, a.d_gic);
            const int c = kk - (int)tap * a.g_ic;
            const uint32_t ky = fastdiv(tap, a.d_kw);
            const int dy = (int)ky * a.dil_h, dx = ((int)tap - (int)ky * a.kw) * a.dil_w;
            t = v4i{(dy * a.in_w + dx) * a.ldx + c, dy, dx, (int)a.zx_splat};
        }
        taps[e] = t;
    }
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.wpk + (size_t)chunk * KS * T * 1024);
        u32x4 *dst = reinterpret_cast<u32x4 *>(wlds);
        const int n = KS * T * 64;
        for (int i = threadIdx.x; i < n; i += 4 * kThreads) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * kThreads < n) v[u] = src[i + u * kThreads];
#pragma unroll
            for (int u = 0; u < 4; u++)
                if (i + u * kThreads < n) dst[i + u * kThreads] = v[u];
        }
    }
    __syncthreads();

    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    constexpr int pix_per_block = kWaves * RG * 16;
    struct Origin { // window origin of a lane's pixel: byte offset (may lie before the tensor), row, column
        uint32_t off;
        int iy0, ix0;
    };
    auto origin = [&](int mt, int rg) {
        const PixInfo pi = pix_info<kVec16>(a, mt * pix_per_block + (wave * RG + rg) * 16 + j);
        const bool ok = pi.base >= 0;
        Origin o;
        o.off = (uint32_t)(((ok ? pi.base : 0) + pi.iy0 * a.in_w + pi.ix0) * a.ldx + a.x_coff);
        o.iy0 = ok ? pi.iy0 : 0x40000000; // (a pixel past the end reads nothing)
        o.ix0 = pi.ix0;
        return o;
    };
    const v4i *const my_taps = taps + gq;
    auto load = [&](const Origin &o, int ks) {
        const v4i t = my_taps[ks * 4];
        const bool inside = (unsigned)(o.iy0 + t[1]) < (unsigned)a.in_h && (unsigned)(o.ix0 + t[2]) < (unsigned)a.in_w;
        WindowSlice f;
        f.raw = __builtin_amdgcn_raw_buffer_load_b128(xres, inside ? o.off + (uint32_t)t[0] : 0xffffffffu, 0, 0);
        f.fill = inside ? 0u : (uint32_t)t[3];
        return f;
    };

    // Tiles in the order of the tensor, a contiguous eighth of them per XCD (workgroups go to the 8 XCDs round-robin, each
    // XCD with an L2 of its own): the tiles that share input rows -- vertical neighbours -- then run on one XCD at about
    // the same time and the shared rows are fetched from memory once (with tiles dealt round-robin the 6x6 stem over
    // 640x640 images fetched 3.2 times its input).
    int mt = blockIdx.x, mt_step = gridDim.x, mt_end = a.num_mtiles;
    if (gridDim.y == 1 && (gridDim.x & 7u) == 0) {
        const int xcd = blockIdx.x & 7, per = (a.num_mtiles + 7) >> 3;
        mt = xcd * per + (int)(blockIdx.x >> 3);
        mt_step = gridDim.x >> 3;
        mt_end = min(a.num_mtiles, (xcd + 1) * per);
    }
    Origin org[RG];
    WindowSlice cur[RG];
    if (mt < mt_end) {
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            org[rg] = origin(mt, rg);
            cur[rg] = load(org[rg], 0);
        }
    }
    const int last = KS - 1;
    const int ch0 = ch_base + gq * (4 * T);
#pragma clang loop unroll(disable)
    for (; mt < mt_end; mt += mt_step) {
        v4i acc[RG][T];
        v4i rs[RG];
        const int mt_next = mt + mt_step < mt_end ? mt + mt_step : mt; // past the end: re-read this tile, dropped
        Origin org_next[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) org_next[rg] = origin(mt_next, rg);
#pragma clang loop unroll(disable)
        for (int ks = 0; ks < KS; ks++) {
            // the next slices: the next k-step of this tile, or the first of the next tile
            WindowSlice nxt[RG];
            const bool same_tile = ks < last;
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                Origin o;
                o.off = same_tile ? org[rg].off : org_next[rg].off;
                o.iy0 = same_tile ? org[rg].iy0 : org_next[rg].iy0;
                o.ix0 = same_tile ? org[rg].ix0 : org_next[rg].ix0;
                nxt[rg] = load(o, same_tile ? ks + 1 : 0);
            }
            v4i xf[RG];
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                u32x4 r;
#pragma unroll
                for (int d = 0; d < 4; d++) r[d] = (cur[rg].raw[d] | cur[rg].fill) ^ 0x80808080u;
                xf[rg] = __builtin_bit_cast(v4i, r);
            }
            const uint8_t *wstep = wlds + (size_t)ks * T * 1024 + lane * 16;
            if (ks == 0) {
                int ct_off = gq * (4 * T);
                asm volatile("" : "+v"(ct_off)); // (read per tile: kept in registers the constants would cost 4T of them)
                const v4i zero = {0, 0, 0, 0};
#pragma unroll
                for (int nt = 0; nt < T; nt++) {
                    const v4i ct = *reinterpret_cast<const v4i *>(cterm + ct_off + nt * 4);
                    const v4i wf = *reinterpret_cast<const v4i *>(wstep + nt * 1024);
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) acc[rg][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf[rg], ct, 0, 0, 0);
                }
#pragma unroll
                for (int rg = 0; rg < RG; rg++) rs[rg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, xf[rg], zero, 0, 0, 0);
            } else {
#pragma unroll
                for (int nt = 0; nt < T; nt++) {
                    const v4i wf = *reinterpret_cast<const v4i *>(wstep + nt * 1024);
#pragma unroll
                    for (int rg = 0; rg < RG; rg++) acc[rg][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf[rg], acc[rg][nt], 0, 0, 0);
                }
#pragma unroll
                for (int rg = 0; rg < RG; rg++) rs[rg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, xf[rg], rs[rg], 0, 0, 0);
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) cur[rg] = nxt[rg];
        }
#pragma unroll
        for (int rg = 0; rg < RG; rg++)
            igemm_store_tile<T, kOwesRows, PLAIN, false, MAGIC>(a, acc[rg], rs[rg][0], mt * pix_per_block + (wave * RG + rg) * 16 + j, ch0, gq, cterm, lutl);
#pragma unroll
        for (int rg = 0; rg < RG; rg++) org[rg] = org_next[rg];
    }
}

// Pixel groups per wave (RG) for a chunk width of T tiles.  The kernels are bound by the
// VALU work of the epilogue, and a dependent VALU instruction issues only every ~8 cycles
// from one wave, so what matters is having >= 4 waves per SIMD: RG is capped so that the
// kernel stays within 128 VGPRs, and lowered further while the grid would not give every
// compute unit a couple of blocks.
inline int choose_rg(const nncase_hip_ctx *ctx, int tiles, int nchunks, int m) {
    const long long target = 2LL * ctx->compute_units;
    const int cap = tiles == 1 ? 4 : (tiles <= 6 ? 2 : 1);
    for (int rg = cap; rg > 1; rg /= 2)
        if ((long long)ceil_div(m, kWaves * rg * 16) * nchunks >= target) return rg;
    return 1;
}

template <int T, int RG, int MODE> int launch_trg(nncase_hip_ctx *ctx, const IgemmArgs &a, int nchunks) {
    IgemmArgs args = a;
    constexpr int pix_per_block = kWaves * RG * 16;
    args.num_mtiles = ceil_div(a.m, pix_per_block);
    // persistent blocks: four per compute unit (a block's chain of load -> multiply -> store per pixel tile is
    // latency-bound, so more chains in flight beat longer ones)
    int gx = args.num_mtiles < ctx->compute_units * 4 ? args.num_mtiles : ctx->compute_units * 4;
    // Blocks are dealt to the 8 XCDs round-robin by linear id; with a multiple of 8
    // columns the blocks that share a pixel tile (same x, different chunk) land on
    // one XCD and find the activations in its L2.
    if (nchunks > 1) gx = ceil_div(gx, 8) * 8;
    size_t lds = (size_t)T * 16 * sizeof(int32_t) + 256 + (size_t)a.kc_steps * T * 1024;
    // dword outputs of chunks of 4, 8, 12 or 16 tiles go through a staging area per wave (store_dword_group)
    const bool stage_lds = staged_store_built(T) && (loads_rows(MODE) || MODE == kVec16) && (a.deq || a.ep.out_mode != kOutU8);
    if (stage_lds) lds += (size_t)kWaves * staged_store_bytes();
    // the 1x1 row loaders are also built without the epilogue's options (see igemm_store_tile)
    bool plain = false;
    if constexpr (loads_rows(MODE) || MODE == kVec16)
        plain = a.ep.out_mode == kOutU8 && !a.deq && a.ep.fast && a.ep.full && !a.lut && !a.rep.res && a.n % (4 * T) == 0 && ((a.ldy | a.y_coff) & 3) == 0;
    if constexpr (MODE == kVec16 && T <= 6) {
        // the whole chunk's weights resident and no folded reduction: the kernel with the tap table
        const size_t lds_win = (size_t)T * 16 * sizeof(int32_t) + 256 + (size_t)a.ksteps * 4 * sizeof(v4i) + (size_t)a.ksteps * T * 1024;
        if (a.kc_steps >= a.ksteps && a.kc_mask == -1 && lds_win <= 65536) {
            if (plain && a.magic_ok) hipLaunchKernelGGL((qconv_window_kernel<T, RG, true, true>), dim3(gx, nchunks, 1), dim3(kThreads), lds_win, ctx->stream, args);
            else if (plain) hipLaunchKernelGGL((qconv_window_kernel<T, RG, true>), dim3(gx, nchunks, 1), dim3(kThreads), lds_win, ctx->stream, args);
            else hipLaunchKernelGGL((qconv_window_kernel<T, RG, false>), dim3(gx, nchunks, 1), dim3(kThreads), lds_win, ctx->stream, args);
            NNHIP_LAUNCH_CHECK(ctx, "qconv_window_kernel");
            return 0;
        }
        plain = false;
    }
    if (plain) {
        if constexpr (MODE == kRows16) {
            // the whole chunk's weights resident, rows of at least 16 bytes: the lean kernel
            if (a.kc_steps >= a.ksteps) {
                const size_t lds_rows = (size_t)T * 16 * sizeof(int32_t) + (size_t)a.ksteps * T * 1024;
                if (a.magic_ok) {
                    if (a.zwp_rows != 0) hipLaunchKernelGGL((qconv_rows_kernel<T, RG, true, true>), dim3(gx, nchunks, 1), dim3(kThreads), lds_rows, ctx->stream, args);
                    else hipLaunchKernelGGL((qconv_rows_kernel<T, RG, false, true>), dim3(gx, nchunks, 1), dim3(kThreads), lds_rows, ctx->stream, args);
                } else {
                    if (a.zwp_rows != 0) hipLaunchKernelGGL((qconv_rows_kernel<T, RG, true, false>), dim3(gx, nchunks, 1), dim3(kThreads), lds_rows, ctx->stream, args);
                    else hipLaunchKernelGGL((qconv_rows_kernel<T, RG, false, false>), dim3(gx, nchunks, 1), dim3(kThreads), lds_rows, ctx->stream, args);
                }
                NNHIP_LAUNCH_CHECK(ctx, "qconv_rows_kernel");
                return 0;
            }
        }
        if constexpr (loads_rows(MODE))
            hipLaunchKernelGGL((qconv_igemm_kernel<T, RG, MODE, true>), dim3(gx, nchunks, 1), dim3(kThreads), lds, ctx->stream, args);
    } else if (stage_lds) {
        if constexpr (staged_store_built(T) && (loads_rows(MODE) || MODE == kVec16)) {
            if (lds > 65536) { // more than 64 KiB of dynamic LDS (full-depth weights and the staging areas) has to be asked for once per kernel and device
                static std::once_flag raised[16];
                hipError_t attr = hipSuccess;
                std::call_once(raised[ctx->device & 15], [&] {
                    attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&qconv_igemm_kernel<T, RG, MODE, false, true>), hipFuncAttributeMaxDynamicSharedMemorySize, 98304);
                });
                NNHIP_HIP(ctx, attr);
            }
            hipLaunchKernelGGL((qconv_igemm_kernel<T, RG, MODE, false, true>), dim3(gx, nchunks, 1), dim3(kThreads), lds, ctx->stream, args);
        }
    } else
        hipLaunchKernelGGL((qconv_igemm_kernel<T, RG, MODE>), dim3(gx, nchunks, 1), dim3(kThreads), lds, ctx->stream, args);
    NNHIP_LAUNCH_CHECK(ctx, "qconv_igemm_kernel");
    return 0;
}

template <int T, int MODE> int launch_t(nncase_hip_ctx *ctx, const IgemmArgs &a, int nchunks, int rg) {
    // only the combinations choose_rg can return are built: the others would need more registers than a wave has
    if (rg == 1) return launch_trg<T, 1, MODE>(ctx, a, nchunks);
    if constexpr (T <= 6) {
        if (rg == 2) return launch_trg<T, 2, MODE>(ctx, a, nchunks);
    }
    if constexpr (T == 1) {
        if (rg == 4) return launch_trg<T, 4, MODE>(ctx, a, nchunks);
    }
    return fail(ctx, -EINVAL, "igemm: no kernel for %d tiles x %d pixel groups", T, rg);
}

template <int MODE> int launch_mode(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    switch (tiles) {
    case 1: return launch_t<1, MODE>(ctx, a, nchunks, rg);
    case 2: return launch_t<2, MODE>(ctx, a, nchunks, rg);
    case 3: return launch_t<3, MODE>(ctx, a, nchunks, rg);
    case 4: return launch_t<4, MODE>(ctx, a, nchunks, rg);
    default: break;
    }
    if constexpr (MODE != kBytes) {
        switch (tiles) {
        case 5: return launch_t<5, MODE>(ctx, a, nchunks, rg);
        case 6: return launch_t<6, MODE>(ctx, a, nchunks, rg);
        case 8: return launch_t<8, MODE>(ctx, a, nchunks, rg);
        case 9: return launch_t<9, MODE>(ctx, a, nchunks, rg);
        case 10: return launch_t<10, MODE>(ctx, a, nchunks, rg);
        case 12: return launch_t<12, MODE>(ctx, a, nchunks, rg);
        case 16: return launch_t<16, MODE>(ctx, a, nchunks, rg);
        default: break;
        }
    }
    return fail(ctx, -EINVAL, "igemm: no kernel for %d tiles (load mode %d)", tiles, MODE);
}

int launch_igemm_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg);
int launch_igemm_vec16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg);
int launch_igemm_vec8(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg);
int launch_igemm_rows8(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg);
int launch_igemm_vec4(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg);
int launch_igemm_bytes(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg);

} // namespace nnhip
