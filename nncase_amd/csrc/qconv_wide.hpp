// u8/u8 convolution / matmul as an implicit GEMM with a wide register tile per wave, for the
// layers that are bound by the matrix cores: long reductions over many pixels and channels.
//
// The kernels of qconv_igemm.hpp give a wave 16 or 32 pixels, which suits reductions of one or
// two k-steps (most of MobileNetV2) where the epilogue is the work.  For a long reduction such a
// tile needs a 1 KiB operand fragment per matrix instruction or two, and the operand traffic, not
// the matrix cores, sets the pace.  Here a wave owns RG * 16 pixels x T * 16 output channels
// (64 x 128: 128 int32 accumulator registers), so a k-step of 64 needs RG activation fragments and
// T weight fragments for RG * T matrix instructions, and a block of WM x WN waves shares both
// operands through LDS:
//   * a ring of three LDS slots, each holding one k-step of the block's activations and weights;
//     global -> registers -> LDS two k-steps ahead of the multiply, one barrier per k-step;
//   * activations are fetched in row order (the four threads of a quad read the 64 contiguous
//     bytes of one pixel's k-step: full-width requests to the vector L1) and re-read from LDS in
//     matrix operand order; padding taps and the u8 -> s8 re-bias are applied on the way in;
//   * weights are pre-packed fragments in operand order (qconv_igemm.hpp, tiles = WN * T);
//   * a matrix instruction and an ordinary vector instruction of the same SIMD do not overlap
//     (measured: the vector work of a k-step adds to its matrix time), so the main loop is kept
//     almost free of vector instructions: buffer loads whose per-step offsets live in scalar
//     registers, LDS addresses that are a per-thread constant plus the slot's scalar offset plus an
//     immediate, tap geometry on the scalar
//     unit when a k-step lies within one tap, and the per-pixel sum of x' (which the weight zero
//     point multiplies) from v_dot4 on the registers being staged instead of further matrix work;
//   * blocks are numbered so that the channel chunks of one pixel tile run back to back on one
//     XCD: the activations are fetched from HBM once and found in that XCD's L2 by the other chunks.
// Arithmetic, weight packing and epilogue are those of qconv_igemm.hpp: the bytes are the same
// whichever kernel runs a layer.
#pragma once

#include "qconv_igemm.hpp"

#include <mutex>
#include <type_traits>

namespace nnhip {

// Where the wide tiles pay: measured against the kernels of qconv_igemm.hpp layer by layer (YOLOv5s-style network at
// batch 16, batched matmul), they win for reductions of 512 and more when the launch has at least one 256-pixel
// block per compute unit; below that a launch has too few 64-pixel wave tiles to fill the device and the small tiles'
// larger wave count wins.
constexpr int kWideMinKsteps = 8;
constexpr int kSmallWideMinKsteps = 5; // (measured on MobileNetV2 at batch 64 and the YOLOv5s-style network at batch 16: flat from 4 to 8)
constexpr int kWideSlots = 3;

// How a thread finds its 16-byte pieces of a k-step:
//   kWideRowsFull  contiguous reduction rows (1x1 windows, matmul), reduction a multiple of 64
//   kWideRows      contiguous reduction rows, any multiple of 16
//   kWideTap       windows; channels per group a multiple of 64, so a k-step lies within one tap (scalar tap geometry)
//   kWideWindow    windows; channels per group a multiple of 16
enum WideLoad { kWideRowsFull = 0, kWideRows = 1, kWideTap = 2, kWideWindow = 3 };

typedef uint32_t wide_u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wide_rsrc(const void *base, uint32_t bytes) {
    // raw buffer (stride 0): offsets are range-checked against `bytes`, reads outside return 0
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

// T: 16-channel tiles per wave; RG: 16-pixel groups per wave; a block is WM x WN waves: WM * RG * 16 pixels by
// WN * T * 16 channels (the block's channel chunk, packed with tiles = WN * T).
//
// LDS: kWideSlots slots, each [activations: pixels x 64 bytes | weights: WN * T fragments].  The four 16-byte
// pieces of pixel p are rotated by (p >> 1) & 3: the LDS serves a 16-byte read of eight neighbouring lanes per 128 bytes of
// banks, so pixels p and p + 2 (128 bytes apart) must not present the same piece (measured: 241 bytes per clock and
// compute unit with this rotation, 128 with a rotation by (p >> 2) or none); the row-order writes cover whole
// 128-byte runs whatever the rotation.
template <int T, int RG, int WM, int WN, int LM>
__global__ __launch_bounds__(WM * WN * 64, 2) void qconv_wide_kernel(const IgemmArgs a, int nchunks) {
    constexpr int THREADS = WM * WN * 64;
    constexpr int PIX = WM * RG * 16;                   // pixels per block
    constexpr int TB = T * WN;                          // channel tiles per block
    constexpr int AV = PIX * 4, WV = TB * 64;           // 16-byte vectors of activations / weights per k-step
    constexpr int NA = AV / THREADS, NW = WV / THREADS; // ... per thread
    static_assert(AV % THREADS == 0 && WV % THREADS == 0, "every thread moves the same number of vectors");
    static_assert(T % 2 == 0, "channel tiles are multiplied in pairs");
    constexpr int G = T / 2;
    constexpr int SLOT = AV * 16 + WV * 16;             // bytes of a ring slot
    constexpr bool kRows = LM == kWideRowsFull || LM == kWideRows;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int32_t *cterm = reinterpret_cast<int32_t *>(smem);              // [TB * 16]
    uint8_t *lutl = smem + TB * 16 * sizeof(int32_t);                // [256]
    int32_t *rowsums = reinterpret_cast<int32_t *>(lutl + 256);      // [PIX]
    uint8_t *ring = lutl + 256 + PIX * sizeof(int32_t);              // [kWideSlots][SLOT]

    // channel chunks of a pixel tile are consecutive on one XCD (blocks go to the 8 XCDs round-robin)
    // ... and every XCD takes a contiguous eighth of the pixel tiles, in the order of the tensor: the tiles that share
    // input rows of a window (vertical neighbours) then run on one XCD at about the same time
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int chunk = seq % nchunks;
    const int per = (a.num_mtiles + 7) >> 3;
    const int mt = xcd * per + seq / nchunks;
    if (seq / nchunks >= per || mt >= a.num_mtiles) return;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int j = lane & 15, gq = lane >> 4; // matrix operand order: pixel j of a group, 16-byte piece gq of the k-step
    const int ch_base = chunk * (TB * 16);
    const int KS = a.ksteps;
    const __amdgpu_buffer_rsrc_t wres = wide_rsrc(a.wpk + (size_t)chunk * KS * TB * 1024, (uint32_t)KS * TB * 1024);
    const __amdgpu_buffer_rsrc_t xres = wide_rsrc(a.x, (uint32_t)a.x_bytes);

    // per-channel constant of the zero-point identity and the byte table: requested now, needed by the epilogue
    constexpr int NC = (TB * 16 + THREADS - 1) / THREADS;
    int32_t c_bias[NC], c_wsum[NC];
#pragma unroll
    for (int i = 0; i < NC; i++) {
        const int c = i * THREADS + threadIdx.x;
        const bool real = c < TB * 16 && ch_base + c < a.n;
        c_bias[i] = real ? a.bias[ch_base + c] : 0;
        c_wsum[i] = real ? a.wsum[ch_base + c] : 0;
    }
    uint32_t lut_word = 0;
    const bool lut_mine = a.lut && threadIdx.x < 64;
    if (lut_mine) lut_word = a.lut[threadIdx.x];

    // ---- weights: thread t moves vectors t + i * THREADS of every k-step ----
    const uint32_t w_voff = threadIdx.x * 16;
    auto load_w = [&](wide_u32x4 (&dst)[NW], int ks) {
        const int ksc = min(ks, KS - 1); // a k-step past the end re-reads the last one (its data is never multiplied)
#pragma unroll
        for (int i = 0; i < NW; i++) dst[i] = __builtin_amdgcn_raw_buffer_load_b128(wres, w_voff, (ksc * WV + i * THREADS) * 16, 0);
    };
    uint8_t *const w_dst = ring + AV * 16 + threadIdx.x * 16;
    auto store_w = [&](const wide_u32x4 (&src)[NW], int slot /* byte offset of the ring slot */) {
#pragma unroll
        for (int i = 0; i < NW; i++) *reinterpret_cast<wide_u32x4 *>(w_dst + slot + i * THREADS * 16) = src[i];
    };

    // ---- activations: the NA pieces this thread fetches per k-step (row order: the four threads of a quad read the
    // 64 bytes of one pixel's k-step): piece lq of pixel lp + i * (THREADS / 4) of the block ----
    const int lp = threadIdx.x >> 2, lq = threadIdx.x & 3;
    int32_t p_off[NA];          // byte offset of the pixel's first piece (windows: of the window origin, may be negative)
    int32_t p_iy0[NA], p_ix0[NA];
#pragma unroll
    for (int i = 0; i < NA; i++) {
        const PixInfo pi = pix_info<kRows ? kRows16 : kVec16>(a, mt * PIX + lp + i * (THREADS / 4));
        const bool ok = pi.base >= 0; // a pixel past the end takes pixel 0's place: any valid address, the result is not stored
        if (kRows) {
            p_off[i] = (ok ? pi.base : 0) * a.ldx + a.x_coff + lq * 16;
            p_iy0[i] = p_ix0[i] = 0;
        } else {
            p_iy0[i] = ok ? pi.iy0 : 0;
            p_ix0[i] = ok ? pi.ix0 : 0;
            p_off[i] = ((ok ? pi.base : 0) + p_iy0[i] * a.in_w + p_ix0[i]) * a.ldx + a.x_coff + (LM == kWideTap ? lq * 16 : 0);
        }
    }
    struct Acts {
        wide_u32x4 raw[NA];
        uint32_t fill;    // what a piece that is not taken holds: the zero point (padding tap) or x' = 0 (past the reduction)
        bool take[NA];
    };
    auto load_acts = [&](Acts &f, int ks) {
        const int ksc = min(ks, KS - 1); // as for the weights
        if (LM == kWideRowsFull) {
#pragma unroll
            for (int i = 0; i < NA; i++) {
                f.raw[i] = __builtin_amdgcn_raw_buffer_load_b128(xres, p_off[i], ksc * 64, 0);
                f.take[i] = true;
            }
            f.fill = 0;
        } else if (LM == kWideRows) {
            // the last k-step may end inside the row: the piece's offset goes through the range-checked operand
            const bool in_k = ksc * 64 + lq * 16 < a.k;
#pragma unroll
            for (int i = 0; i < NA; i++) {
                f.raw[i] = __builtin_amdgcn_raw_buffer_load_b128(xres, p_off[i] + ksc * 64, 0, 0);
                f.take[i] = in_k;
            }
            f.fill = 0x80808080u;
        } else if (LM == kWideTap) {
            // one tap per k-step: its geometry is the same for the whole block (scalar unit)
            const uint32_t kk = (uint32_t)ksc * 64;
            const uint32_t tap = fastdiv(kk, a.d_gic);
            const int c0 = (int)kk - (int)tap * a.g_ic;
            const uint32_t ky = fastdiv(tap, a.d_kw);
            const int dy = (int)ky * a.dil_h, dx = ((int)tap - (int)ky * a.kw) * a.dil_w;
            const int shift = (dy * a.in_w + dx) * a.ldx + c0;
#pragma unroll
            for (int i = 0; i < NA; i++) {
                // no clamping: an address outside the tensor reads 0, one inside but outside the image is replaced below
                f.raw[i] = __builtin_amdgcn_raw_buffer_load_b128(xres, p_off[i] + shift, 0, 0);
                f.take[i] = (unsigned)(p_iy0[i] + dy) < (unsigned)a.in_h && (unsigned)(p_ix0[i] + dx) < (unsigned)a.in_w;
            }
            f.fill = a.zx_splat;
        } else {
            const int kk = ksc * 64 + lq * 16;
            const bool in_k = kk < a.k;
            const uint32_t tap = fastdiv((uint32_t)(in_k ? kk : 0), a.d_gic);
            const int c = (in_k ? kk : 0) - (int)tap * a.g_ic;
            const uint32_t ky = fastdiv(tap, a.d_kw);
            const int dy = (int)ky * a.dil_h, dx = ((int)tap - (int)ky * a.kw) * a.dil_w;
            const int shift = (dy * a.in_w + dx) * a.ldx + c;
#pragma unroll
            for (int i = 0; i < NA; i++) {
                f.raw[i] = __builtin_amdgcn_raw_buffer_load_b128(xres, p_off[i] + shift, 0, 0);
                f.take[i] = in_k && (unsigned)(p_iy0[i] + dy) < (unsigned)a.in_h && (unsigned)(p_ix0[i] + dx) < (unsigned)a.in_w;
            }
            f.fill = in_k ? a.zx_splat : 0x80808080u;
        }
    };
    // (THREADS / 4 is a multiple of 8, so the rotation of a thread's pieces is the same for all its pixels)
    uint8_t *const a_dst = ring + lp * 64 + ((lq + (lp >> 1)) & 3) * 16;
    uint32_t rsum[NA]; // sum of x (the bytes as staged, before the re-bias) over this thread's pieces of its i-th pixel
#pragma unroll
    for (int i = 0; i < NA; i++) rsum[i] = 0;
    // Padding and re-biasing happen on the way into the ring: x' = (piece taken ? x : fill) ^ 0x80; the sums of x are
    // taken from the same registers (every staged k-step adds 64 bytes per pixel, positions past the reduction as 128:
    // the sum of x' is the sum of x less 128 * 64 * k-steps).  A k-step past the end of the reduction is not staged (ks < KS is uniform).
    auto store_acts = [&](const Acts &f, int slot, int ks) {
        if (ks >= KS) return;
#pragma unroll
        for (int i = 0; i < NA; i++) {
            wide_u32x4 r;
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const uint32_t x = LM == kWideRowsFull ? f.raw[i][d] : (f.take[i] ? f.raw[i][d] : f.fill);
                rsum[i] = __builtin_amdgcn_sad_u8(x, 0u, rsum[i]); // (a dot product against ones costs the matrix unit seven cycles, this next to none)
                r[d] = x ^ 0x80808080u;
            }
            *reinterpret_cast<wide_u32x4 *>(a_dst + slot + i * (THREADS / 4) * 64) = r;
        }
    };

    v4i acc[RG][T];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int nt = 0; nt < T; nt++) acc[rg][nt] = v4i{0, 0, 0, 0};

    // ---- fill the pipeline ----
    // Loads are issued unconditionally (past the end of the reduction they re-read the last k-step): loads complete
    // in order, and only a compile-time count of younger loads lets a wait for one k-step's operands leave the later
    // ones in flight.
    wide_u32x4 wreg[2][NW];
    Acts af[2];
    {
        wide_u32x4 w0[NW];
        Acts a0;
        load_w(w0, 0);
        load_acts(a0, 0);
        load_w(wreg[1], 1);
        load_acts(af[1], 1);
        load_w(wreg[0], 2);
        load_acts(af[0], 2);
        store_w(w0, 0);
        store_acts(a0, 0, 0);
        __syncthreads(); // ring slot 0 is written
    }
    const uint8_t *const x_src = ring + (wm * RG * 16 + j) * 64 + ((gq + (j >> 1)) & 3) * 16; // + rg * 16 * 64
    const uint8_t *const w_src = ring + AV * 16 + (wn * T) * 1024 + lane * 16;                 // + nt * 1024
    // One k-step s (parity P) multiplies the ring slot at byte offset `cur`: operand reads of the next pair of channel
    // tiles are issued before the matrix instructions of the current pair (the order is pinned by scheduling
    // barriers).  Between the pairs data moves: the operands of k-step s + 1 (in wreg[1 - P] / af[1 - P], requested
    // two k-steps ago) go into the next slot and those of k-step s + 3 are requested.  The slot offsets are scalars:
    // four vector additions per k-step turn the per-thread constants into this k-step's LDS addresses, everything
    // else is an immediate.
    int cur = 0;
    auto kstep = [&](int s, auto parity) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        const int next = cur == (kWideSlots - 1) * SLOT ? 0 : cur + SLOT;
        const uint8_t *const xs = x_src + cur, *const ws = w_src + cur;
        v4i xf[RG];
#pragma unroll
        for (int rg = 0; rg < RG; rg++) xf[rg] = *reinterpret_cast<const v4i *>(xs + rg * 16 * 64);
        v4i wf[2][2];
        wf[0][0] = *reinterpret_cast<const v4i *>(ws);
        wf[0][1] = *reinterpret_cast<const v4i *>(ws + 1024);
#pragma unroll
        for (int g = 0; g < G; g++) {
            __builtin_amdgcn_sched_barrier(0);
            if (g + 1 < G) {
                wf[(g + 1) & 1][0] = *reinterpret_cast<const v4i *>(ws + (2 * g + 2) * 1024);
                wf[(g + 1) & 1][1] = *reinterpret_cast<const v4i *>(ws + (2 * g + 3) * 1024);
            }
#pragma unroll
            for (int e = 0; e < 2; e++)
#pragma unroll
                for (int rg = 0; rg < RG; rg++)
                    acc[rg][2 * g + e] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[g & 1][e], xf[rg], acc[rg][2 * g + e], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (g == 0) {
                store_w(wreg[1 - P], next);
                load_w(wreg[1 - P], s + 3);
            }
            if (g == (G > 2 ? 1 : 0)) {
                store_acts(af[1 - P], next, s + 1);
                load_acts(af[1 - P], s + 3);
            }
        }
        cur = next;
        __syncthreads();
    };
    int s = 0;
#pragma clang loop unroll(disable)
    for (; s + 1 < KS; s += 2) {
        kstep(s, std::integral_constant<int, 0>());
        kstep(s + 1, std::integral_constant<int, 1>());
    }
    if (s < KS) kstep(s, std::integral_constant<int, 0>()); // an odd number of k-steps

    // ---- epilogue ----
#pragma unroll
    for (int i = 0; i < NC; i++) {
        const int c = i * THREADS + threadIdx.x;
        if (c < TB * 16) cterm[c] = ch_base + c < a.n ? c_bias[i] - a.zxp * c_wsum[i] + a.k * a.zxp * a.zwp : 0;
    }
    if (lut_mine) reinterpret_cast<uint32_t *>(lutl)[threadIdx.x] = lut_word;
    // the sums of x' sit with the threads that loaded the pieces: add the four pieces of a pixel, pass them through LDS
#pragma unroll
    for (int i = 0; i < NA; i++) {
        int32_t r = (int32_t)rsum[i];
        r += __shfl_xor(r, 1);
        r += __shfl_xor(r, 2);
        if (lq == 0) rowsums[lp + i * (THREADS / 4)] = r - 128 * 64 * KS;
    }
    __syncthreads();
    // dword outputs are written through a staging area per wave (store_dword_rows): the ring is free now
    static_assert(!staged_store_built(T) || WM * WN * staged_store_bytes() <= kWideSlots * SLOT, "the staging areas fit the ring");
    uint8_t *const stage = staged_store_built(T) ? ring + wave * staged_store_bytes() : nullptr;
    // lane (j, gq) of wave (wm, wn) holds channels ch_base + gq * 4 TB + wn * 4 T + [0, 4 T) of its pixels
    const int ch0 = ch_base + gq * (4 * TB) + wn * (4 * T);
    const int32_t *ct = cterm + gq * (4 * TB) + wn * (4 * T) - gq * (4 * T); // igemm_store_tile adds gq * 4 T
    static_for<0, RG>([&](auto rg_c) __attribute__((always_inline)) {
        constexpr int rg = decltype(rg_c)::value;
        const int pl = (wm * RG + rg) * 16 + j;
        igemm_store_tile<T, kOwesAll, false, staged_store_built(T)>(a, acc[rg], rowsums[pl], mt * PIX + pl, ch0, gq, ct, lutl, stage, 4 * TB);
    });
}



// ---- the 256-pixel x 256-channel block ------------------------------------------------------------------------
// What a compute unit can take from its L2 bounds the matrix rate of a long reduction: a k-step of a P x C block moves
// (P + C) * 64 bytes for P * C / 64 cycles of the four matrix units, and the vector memory path delivers 55-62 bytes
// per cycle when a wave's load covers whole 128-byte lines (1 KiB runs of packed weights; 128 bytes per pixel) but
// 35-40 when it takes 64 bytes out of each line (measured on an L2-resident set).  The accumulators of 256 x 256
// outputs are half of the unit's registers, so that block is the largest there is: eight waves of 64 x 128, one block
// per unit, 32 bytes per cycle at the full matrix rate.  It therefore
//   * fetches activations for two k-steps at a time: eight threads read the 128 contiguous bytes of a pixel
//     (window modes: two 64-byte halves, each at its own tap), requested two k-steps before they are staged;
//   * keeps a ring of four k-step slots, so that a slot is free for two k-steps before its first read: the weights'
//     DMA is requested at the top of k-step s - 3 and waited for at the end of k-step s - 2;
// The rest (operand reads ahead of the products, rotation of a pixel's pieces, sums of x', epilogue) is the kernel above.
template <int T, int RG, int WM, int WN, int LM>
__global__ __launch_bounds__(WM * WN * 64, 2) void qconv_wide4_kernel(const IgemmArgs a, int nchunks) {
    constexpr int NS = 4;
    constexpr int THREADS = WM * WN * 64;
    constexpr int PIX = WM * RG * 16;
    constexpr int TB = T * WN;
    constexpr int AV = PIX * 4, WV = TB * 64;           // 16-byte vectors of activations / weights per k-step
    constexpr int NA2 = 2 * AV / THREADS;               // activation vectors per thread per pair of k-steps
    constexpr int NW = WV / THREADS;                    // weight runs per wave per k-step
    constexpr int PSTEP = THREADS / 8;                  // pixels between a thread's vectors
    static_assert((2 * AV) % THREADS == 0 && WV % THREADS == 0 && PSTEP % 8 == 0, "every thread moves the same number of vectors");
    static_assert(T % 4 == 0, "at least two pairs of channel tiles per k-step");
    constexpr int G = T / 2;
    constexpr int SLOT = AV * 16 + WV * 16;
    constexpr bool kRows = LM == kWideRowsFull || LM == kWideRows;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int32_t *cterm = reinterpret_cast<int32_t *>(smem);              // [TB * 16]
    uint8_t *lutl = smem + TB * 16 * sizeof(int32_t);                // [256]
    int32_t *rowsums = reinterpret_cast<int32_t *>(lutl + 256);      // [PIX]
    uint8_t *ring = lutl + 256 + PIX * sizeof(int32_t);              // [NS][SLOT]

    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int chunk = seq % nchunks;
    const int per = (a.num_mtiles + 7) >> 3;
    const int mt = xcd * per + seq / nchunks;
    if (seq / nchunks >= per || mt >= a.num_mtiles) return;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int j = lane & 15, gq = lane >> 4;
    const int ch_base = chunk * (TB * 16);
    const int KS = a.ksteps;
    const __amdgpu_buffer_rsrc_t wres = wide_rsrc(a.wpk + (size_t)chunk * KS * TB * 1024, (uint32_t)KS * TB * 1024);
    const __amdgpu_buffer_rsrc_t xres = wide_rsrc(a.x, (uint32_t)a.x_bytes);

    constexpr int NC = (TB * 16 + THREADS - 1) / THREADS;
    int32_t c_bias[NC], c_wsum[NC];
#pragma unroll
    for (int i = 0; i < NC; i++) {
        const int c = i * THREADS + threadIdx.x;
        const bool real = c < TB * 16 && ch_base + c < a.n;
        c_bias[i] = real ? a.bias[ch_base + c] : 0;
        c_wsum[i] = real ? a.wsum[ch_base + c] : 0;
    }
    uint32_t lut_word = 0;
    const bool lut_mine = a.lut && threadIdx.x < 64;
    if (lut_mine) lut_word = a.lut[threadIdx.x];

    // ---- weights: DMA, wave w moves the 1 KiB runs w + i * WAVES of a k-step ----
    const uint32_t w_voff = threadIdx.x * 16;
    auto dma_w = [&](int slot, int ks) __attribute__((always_inline)) {
        const int ksc = min(ks, KS - 1); // a k-step past the end re-reads the last one (its data is never multiplied)
#pragma unroll
        for (int i = 0; i < NW; i++) {
            __attribute__((address_space(3))) uint8_t *dst =
                (__attribute__((address_space(3))) uint8_t *)(ring + AV * 16 + slot + (i * THREADS + wave * 64) * 16);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wres, dst, 16, w_voff, (ksc * WV + i * THREADS) * 16, 0, 0);
        }
    };

    // ---- activations: thread t fetches piece lq4 of k-step 2 * pair + half of pixels lp + i * PSTEP ----
    const int lp = threadIdx.x >> 3, half = (threadIdx.x >> 2) & 1, lq4 = threadIdx.x & 3;
    int32_t p_off[NA2], p_iy0[NA2], p_ix0[NA2];
#pragma unroll
    for (int i = 0; i < NA2; i++) {
        const PixInfo pi = pix_info<kRows ? kRows16 : kVec16>(a, mt * PIX + lp + i * PSTEP);
        const bool ok = pi.base >= 0; // a pixel past the end takes pixel 0's place: any valid address, the result is not stored
        if (kRows) {
            p_off[i] = (ok ? pi.base : 0) * a.ldx + a.x_coff + lq4 * 16;
            p_iy0[i] = p_ix0[i] = 0;
        } else {
            p_iy0[i] = ok ? pi.iy0 : 0;
            p_ix0[i] = ok ? pi.ix0 : 0;
            p_off[i] = ((ok ? pi.base : 0) + p_iy0[i] * a.in_w + p_ix0[i]) * a.ldx + a.x_coff + (LM == kWideTap ? lq4 * 16 : 0);
        }
    }
    struct Acts {
        wide_u32x4 raw[NA2];
        uint32_t fill;
        bool take[NA2];
    };
    // What the loads of a pair of k-steps have in common: where this thread's pieces lie relative to a pixel's origin.
    struct Geom {
        int shift;    // byte offset added to the pixel's
        int dy, dx;   // window modes: the tap
        bool in_k;
        bool phantom; // a k-step past the end (the second half of the last pair of an odd number): read as zeros from outside the tensor
    };
    auto geometry = [&](int pair) {
        const int ksc = min(2 * pair + half, KS - 1);
        Geom g;
        g.phantom = 2 * pair + half >= KS;
        g.dy = g.dx = 0;
        if (kRows) {
            g.shift = ksc * 64;
            g.in_k = LM == kWideRowsFull || ksc * 64 + lq4 * 16 < a.k;
        } else {
            const int kk = ksc * 64 + (LM == kWideTap ? 0 : lq4 * 16);
            g.in_k = LM == kWideTap || kk < a.k;
            const uint32_t tap = fastdiv((uint32_t)(g.in_k ? kk : 0), a.d_gic);
            const int c = (g.in_k ? kk : 0) - (int)tap * a.g_ic;
            const uint32_t ky = fastdiv(tap, a.d_kw);
            g.dy = (int)ky * a.dil_h, g.dx = ((int)tap - (int)ky * a.kw) * a.dil_w;
            g.shift = (g.dy * a.in_w + g.dx) * a.ldx + c;
        }
        return g;
    };
    // piece i of the pair (no clamping: an address outside the tensor reads 0, one inside but outside the image is replaced when staged)
    auto load_piece = [&](Acts &f, const Geom &g, auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        f.raw[i] = __builtin_amdgcn_raw_buffer_load_b128(xres, g.phantom ? (int)0xfffffff0u : p_off[i] + g.shift, 0, 0);
        f.take[i] = g.phantom || (kRows ? g.in_k : (g.in_k && (unsigned)(p_iy0[i] + g.dy) < (unsigned)a.in_h && (unsigned)(p_ix0[i] + g.dx) < (unsigned)a.in_w));
        if (i == 0) f.fill = kRows ? 0x80808080u : (g.in_k ? a.zx_splat : 0x80808080u);
    };
    auto load_acts = [&](Acts &f, int pair) {
        const Geom g = geometry(pair);
        static_for<0, NA2>([&](auto i_c) __attribute__((always_inline)) { load_piece(f, g, i_c); });
    };
    uint8_t *const a_dst = ring + lp * 64 + ((lq4 + (lp >> 1)) & 3) * 16;
    uint32_t rsum[NA2]; // sum of x (the bytes as staged, before the re-bias) over this thread's pieces of its i-th pixel
#pragma unroll
    for (int i = 0; i < NA2; i++) rsum[i] = 0;
    // slot_even / slot_odd: ring slots of the pair's two k-steps (byte offsets)
    auto store_piece = [&](const Acts &f, int slot_even, int slot_odd, int pair, auto i_c) __attribute__((always_inline)) {
        constexpr int i = decltype(i_c)::value;
        // (the second half of the last pair of an odd number of k-steps is staged like any other: zeros, into a slot that no product reads)
        uint8_t *const dst = a_dst + (half ? slot_odd : slot_even);
        wide_u32x4 r;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t x = LM == kWideRowsFull ? f.raw[i][d] : (f.take[i] ? f.raw[i][d] : f.fill);
            rsum[i] = __builtin_amdgcn_sad_u8(x, 0u, rsum[i]); // (a dot product against ones costs the matrix unit seven cycles, this next to none)
            r[d] = x ^ 0x80808080u;
        }
        *reinterpret_cast<wide_u32x4 *>(dst + i * PSTEP * 64) = r;
    };
    auto store_acts = [&](const Acts &f, int slot_even, int slot_odd, int pair) {
        static_for<0, NA2>([&](auto i_c) __attribute__((always_inline)) { store_piece(f, slot_even, slot_odd, pair, i_c); });
    };

    v4i acc[RG][T];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int nt = 0; nt < T; nt++) acc[rg][nt] = v4i{0, 0, 0, 0};

    // s_waitcnt immediates (gfx9 encoding): vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8]
    constexpr auto waitcnt_imm = [](int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8); };
    // ---- fill: slots 0 and 1 complete, slot 2's weights and the activations of pair 1 on their way ----
    // (one register set for the activations in flight: with a second one, requested four k-steps ahead, the kernel
    // no longer fits 256 registers)
    Acts af;
    {
        dma_w(0, 0);
        dma_w(SLOT, 1);
        __builtin_amdgcn_sched_barrier(0);
        load_acts(af, 0);
        __builtin_amdgcn_sched_barrier(0);
        dma_w(2 * SLOT, 2);
        __builtin_amdgcn_sched_barrier(0);
        store_acts(af, 0, SLOT, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_acts(af, 1);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(NA2, 0)); // the first three k-steps' weights and the first pair's activations are in
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    }
    const uint8_t *const x_src = ring + (wm * RG * 16 + j) * 64 + ((gq + (j >> 1)) & 3) * 16; // + rg * 16 * 64
    const uint8_t *const w_src = ring + AV * 16 + (wn * T) * 1024 + lane * 16;                 // + nt * 1024
    v4i xf[2][RG], wf[2][2];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) xf[0][rg] = *reinterpret_cast<const v4i *>(x_src + rg * 16 * 64);
    wf[0][0] = *reinterpret_cast<const v4i *>(w_src);
    wf[0][1] = *reinterpret_cast<const v4i *>(w_src + 1024);
    // The slot offsets are scalars (a ring of 128 KiB is beyond the 64 KiB an LDS instruction's immediate offset
    // reaches, and as compile-time constants every slot's addresses would be held in registers of their own): a few
    // vector additions per k-step turn the per-thread constants into this k-step's addresses.
    int cur = 0;
    Geom geom = geometry(2);
    wide_u32x4 staged_piece = {0, 0, 0, 0};
    auto kstep = [&](int s, auto parity) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        asm volatile("" : "+s"(cur));
        const int nxt = (cur + SLOT) & (NS * SLOT - 1), nxt2 = (cur + 2 * SLOT) & (NS * SLOT - 1), nxt3 = (cur + 3 * SLOT) & (NS * SLOT - 1);
        static_assert((SLOT & (SLOT - 1)) == 0, "the ring wraps by a mask");
        const uint8_t *const ws = w_src + cur;
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int wb = g & 1; // (G is even)
            __builtin_amdgcn_sched_barrier(0);
            if (g + 1 < G) {
                wf[1 - wb][0] = *reinterpret_cast<const v4i *>(ws + (2 * g + 2) * 1024);
                wf[1 - wb][1] = *reinterpret_cast<const v4i *>(ws + (2 * g + 3) * 1024);
            }
            if (g == G - 2) {
                const uint8_t *const xn = x_src + nxt;
#pragma unroll
                for (int rg = 0; rg < RG; rg++) xf[1 - P][rg] = *reinterpret_cast<const v4i *>(xn + rg * 16 * 64);
            }
            if (g + 1 == G) {
                const uint8_t *const wn_ = w_src + nxt;
                wf[1 - wb][0] = *reinterpret_cast<const v4i *>(wn_);
                wf[1 - wb][1] = *reinterpret_cast<const v4i *>(wn_ + 1024);
            }
            __builtin_amdgcn_sched_barrier(0);
            // The products of this pair of tiles, and under them this group's share of the data movement: the DMA request
            // of the weights three k-steps on (first group), and in the even k-steps pieces of the pair of k-steps that
            // is staged next: re-bias, sums, the LDS write, and the request for the same pieces of the pair after it
            // into the registers just freed.  An ordinary vector instruction next to every matrix instruction costs
            // (measured) next to nothing; a run of them stops the matrix unit, so the scheduler is told to alternate.
            if (g == 0) dma_w(nxt3, s + 3);
            if (P == 0 && g == 0) geom = geometry((s >> 1) + 2);
            uint8_t *const dst = a_dst + (half ? nxt3 : nxt2);
            static_for<0, 2 * RG>([&](auto m_c) __attribute__((always_inline)) {
                constexpr int m = decltype(m_c)::value, e = m / RG, rg = m % RG;
                acc[rg][2 * g + e] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[wb][e], xf[P][rg], acc[rg][2 * g + e], 0, 0, 0);
                if (P == 0) {
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, NA2>([&](auto i_c) __attribute__((always_inline)) {
                        constexpr int i = decltype(i_c)::value;
                        if (i % G != g) return;
                        if (m < 4) { // dword m of the piece: padding / re-bias / sums
                            const uint32_t x = LM == kWideRowsFull ? af.raw[i][m] : (af.take[i] ? af.raw[i][m] : af.fill);
                            rsum[i] = __builtin_amdgcn_sad_u8(x, 0u, rsum[i]); // (a dot product against ones costs the matrix unit seven cycles, this next to none)
                            staged_piece[m] = x ^ 0x80808080u;
                        } else if (m == 4) {
                            *reinterpret_cast<wide_u32x4 *>(dst + i * PSTEP * 64) = staged_piece;
                        } else if (m == 5) {
                            load_piece(af, geom, i_c);
                        }
                    });
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
        }
        cur = nxt;
        __builtin_amdgcn_sched_barrier(0);
        // the DMA of k-step s + 2, requested during k-step s - 1, has landed: behind it came NW runs of this k-step's
        // DMA and, in one of the two k-steps, NA2 register loads; this wave's LDS writes are done (LDS operations
        // complete in order: only the two reads of the next weights may still be out)
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(NW + NA2, 2));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    int s = 0;
#pragma clang loop unroll(disable)
    for (; s + 1 < KS; s += 2) {
        kstep(s, std::integral_constant<int, 0>());
        kstep(s + 1, std::integral_constant<int, 1>());
    }
    if (s < KS) kstep(s, std::integral_constant<int, 0>()); // an odd number of k-steps

    // ---- epilogue ----
#pragma unroll
    for (int i = 0; i < NC; i++) {
        const int c = i * THREADS + threadIdx.x;
        if (c < TB * 16) cterm[c] = ch_base + c < a.n ? c_bias[i] - a.zxp * c_wsum[i] + a.k * a.zxp * a.zwp : 0;
    }
    if (lut_mine) reinterpret_cast<uint32_t *>(lutl)[threadIdx.x] = lut_word;
    // a pixel's sum of x' is spread over the eight threads that loaded its pieces
#pragma unroll
    for (int i = 0; i < NA2; i++) {
        int32_t r = (int32_t)rsum[i];
        r += __shfl_xor(r, 1);
        r += __shfl_xor(r, 2);
        r += __shfl_xor(r, 4);
        if ((threadIdx.x & 7) == 0) rowsums[lp + i * PSTEP] = r - 128 * 64 * KS;
    }
    __syncthreads(); // (also: every wave's reads of the ring are done before the staging areas below are written, every DMA has landed)
    static_assert(!staged_store_built(T) || WM * WN * staged_store_bytes() <= NS * SLOT, "the staging areas fit the ring");
    uint8_t *const stage = staged_store_built(T) ? ring + wave * staged_store_bytes() : nullptr;
    const int ch0 = ch_base + gq * (4 * TB) + wn * (4 * T);
    const int32_t *ct = cterm + gq * (4 * TB) + wn * (4 * T) - gq * (4 * T); // igemm_store_tile adds gq * 4 T
    static_for<0, RG>([&](auto rg_c) __attribute__((always_inline)) {
        constexpr int rg = decltype(rg_c)::value;
        const int pl = (wm * RG + rg) * 16 + j;
        igemm_store_tile<T, kOwesAll, false, staged_store_built(T)>(a, acc[rg], rowsums[pl], mt * PIX + pl, ch0, gq, ct, lutl, stage, 4 * TB);
    });
}

template <int T, int RG, int WM, int WN, int LM> int launch_wide4_t(nncase_hip_ctx *ctx, const IgemmArgs &a, int nchunks) {
    IgemmArgs args = a;
    constexpr int PIX = WM * RG * 16, TB = T * WN;
    args.num_mtiles = ceil_div(a.m, PIX);
    const int blocks = ceil_div(args.num_mtiles, 8) * 8 * nchunks;
    const size_t lds = (size_t)TB * 16 * sizeof(int32_t) + 256 + PIX * sizeof(int32_t) + (size_t)4 * (PIX * 64 + TB * 1024);
    static std::once_flag raised[16]; // more than 64 KiB of dynamic LDS has to be asked for once per kernel and device
    hipError_t attr = hipSuccess;
    std::call_once(raised[ctx->device & 15], [&] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&qconv_wide4_kernel<T, RG, WM, WN, LM>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    NNHIP_HIP(ctx, attr);
    hipLaunchKernelGGL((qconv_wide4_kernel<T, RG, WM, WN, LM>), dim3(blocks), dim3(WM * WN * 64), lds, ctx->stream, args, nchunks);
    NNHIP_LAUNCH_CHECK(ctx, "qconv_wide4_kernel");
    return 0;
}



// ---- the same block for contiguous reduction rows (1x1 windows, matmul), fed by DMA alone ------------------------
// With nothing to substitute on the way in (no padding taps), the activations can take the DMA path as well: no
// staging registers, no LDS writes by the waves, no wait on loaded registers inside the loop.  The re-bias to s8 and
// the sums of x move to the consuming side: a wave reads its operand of the NEXT k-step at the top of a k-step and,
// one instruction next to each matrix instruction of the k-step, adds the bytes of every register (v_sad_u8) and
// xors it; a lane ends up with the sum of its own 16-byte pieces, and the four lanes of a pixel add them in the
// epilogue (they are the lanes that need the sum).
//   LDS = 160 KiB: weights, four k-step slots of TB KiB (requested three k-steps ahead, two to land);
//   activations, three stages of PIX pixels x 128 bytes (a pair of k-steps; requested five k-steps ahead, four to
//   land: the trip to HBM).  A pixel's eight 16-byte pieces sit rotated by the pixel index, so that the eight
//   lanes an LDS read serves together -- same piece, eight consecutive pixels -- meet eight different bank groups;
//   the lanes of a DMA request (a 1 KiB run: eight pixels) fetch the pieces in the rotated order.
// The per-channel constants, the byte table and the staging areas of dword outputs take over the ring's memory once
// the last k-step is done.
// Float32 (or int32) results of a wave's 16 pixels x 16 T channels, T = 8, written as whole 128-byte lines.  A lane holds
// 4 T = 32 consecutive channels of one pixel, 128 bytes of the output row; all of them go into the wave's staging area
// (a run per lane, padded against bank conflicts) and come back with eight lanes per run, so that a store instruction
// covers eight complete lines -- the staged stores of four tiles at a time write half lines, and the memory side
// pays for the other half.  LDS operations of a wave execute in order: no barrier, one wait in front of the data read back.
constexpr int kLineRun = 128 + 16;
constexpr int line_store_bytes() { return 64 * kLineRun; } // per wave
template <int T>
__device__ __forceinline__ void wide_store_lines(const IgemmArgs &a, const v4i (&acc)[T], int32_t rowsum, int p, int ch0, int gq, const int32_t *ct,
                                                 uint8_t *stage, int quarter_stride) {
    static_assert(T == 8, "a lane's run is one 128-byte line");
    const int lane = threadIdx.x & 63, j = lane & 15;
    const int32_t nrsz = -a.zwp * rowsum;
    const bool as_int = a.ep.out_mode == kOutI32;
#pragma unroll
    for (int nt = 0; nt < T; nt++) {
        const v4i c = *reinterpret_cast<const v4i *>(ct + gq * (4 * T) + nt * 4);
        u32x4 o;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int32_t v = add3(acc[nt][r], c[r], nrsz);
            o[r] = as_int ? (uint32_t)v : __float_as_uint(clamp_ref((float)v * a.ep.mult, a.ep.lo, a.ep.hi));
        }
        *reinterpret_cast<u32x4 *>(stage + (j * 4 + gq) * kLineRun + nt * 16) = o;
    }
    const int p_first = p - j, ch_first = ch0 - gq * quarter_stride;
    const int u = lane & 7, sub = lane >> 3;
    uint32_t *yo = reinterpret_cast<uint32_t *>(a.y);
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int run = it * 8 + sub; // (pixel of the group, channel quarter)
        const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + run * kLineRun + u * 16);
        const int pp = p_first + (run >> 2), ch = ch_first + (run & 3) * quarter_stride + u * 4;
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

template <int T, int RG, int WM, int WN, int LM>
__global__ __launch_bounds__(WM * WN * 64, WM * WN >= 8 ? 2 : 1) void qconv_wide_dma_kernel(const IgemmArgs a, int nchunks) {
    static_assert(LM == kWideRowsFull || LM == kWideRows, "contiguous reduction rows only");
    constexpr int NSW = 4, NSA = 3;
    constexpr int THREADS = WM * WN * 64, WAVES = WM * WN;
    constexpr int PIX = WM * RG * 16;
    constexpr int TB = T * WN;
    constexpr int WSLOT = TB * 1024;                    // bytes of a weight slot (one k-step)
    constexpr int ASTAGE = PIX * 128;                   // bytes of an activation stage (two k-steps)
    constexpr int NW = TB / WAVES;                      // weight runs (1 KiB) per wave per k-step
    constexpr int NA = PIX / 8 / WAVES;                 // activation runs per wave per pair of k-steps
    static_assert(TB % WAVES == 0 && (PIX / 8) % WAVES == 0 && NA % 4 == 0, "every wave moves the same number of runs");
    static_assert(T % 4 == 0, "at least two pairs of channel tiles per k-step");
    static_assert((WSLOT & (WSLOT - 1)) == 0, "the weight ring wraps by a mask");
    constexpr int G = T / 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t *const wring = smem;                        // [NSW][WSLOT]
    uint8_t *const aring = smem + NSW * WSLOT;          // [NSA][ASTAGE]
    // after the main loop
    int32_t *cterm = reinterpret_cast<int32_t *>(smem);              // [TB * 16]
    uint8_t *lutl = smem + TB * 16 * sizeof(int32_t);                // [256]
    uint8_t *stage_base = lutl + 256;

    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int chunk = seq % nchunks;
    const int per = (a.num_mtiles + 7) >> 3;
    const int mt = xcd * per + seq / nchunks;
    if (seq / nchunks >= per || mt >= a.num_mtiles) return;

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int j = lane & 15, gq = lane >> 4;
    const int ch_base = chunk * (TB * 16);
    const int KS = a.ksteps;
    const __amdgpu_buffer_rsrc_t wres = wide_rsrc(a.wpk + (size_t)chunk * KS * TB * 1024, (uint32_t)KS * TB * 1024);
    const __amdgpu_buffer_rsrc_t xres = wide_rsrc(a.x, (uint32_t)a.x_bytes);

    // ---- weights: wave w moves the runs w + i * WAVES of a k-step ----
    const uint32_t w_voff = threadIdx.x * 16;
    auto dma_w = [&](int slot /* byte offset in the weight ring */, int ks, auto first, auto count) __attribute__((always_inline)) {
        const int ksc = min(ks, KS - 1); // a k-step past the end re-reads the last one (its data is never multiplied)
        static_for<decltype(first)::value, decltype(first)::value + decltype(count)::value>([&](auto i_c) __attribute__((always_inline)) {
            constexpr int i = decltype(i_c)::value;
            __attribute__((address_space(3))) uint8_t *dst = (__attribute__((address_space(3))) uint8_t *)(wring + slot + (i * WAVES + wave) * 1024);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wres, dst, 16, (int)w_voff, (ksc * TB + i * WAVES) * 1024, 0, 0);
        });
    };
    // ---- activations: wave w moves the runs w * NA + i of a pair; lane l of run r fetches, for pixel 8 r + (l >> 3),
    // the piece that belongs at position l & 7 of the pixel's 128 bytes ----
    uint32_t a_voff[NA];
#pragma unroll
    for (int i = 0; i < NA; i++) {
        const int pl = (wave * NA + i) * 8 + (lane >> 3);                 // pixel of the block
        const int p = min(mt * PIX + pl, a.m - 1);                         // (a pixel past the end repeats the last one: not stored)
        const int piece = ((lane & 7) - pl) & 7;
        a_voff[i] = (uint32_t)p * (uint32_t)a.ldx + (uint32_t)a.x_coff + piece * 16;
    }
    auto dma_a = [&](int stage /* byte offset in the activation ring */, int pair, auto first, auto count) __attribute__((always_inline)) {
        const int pc = min(pair, (KS - 1) >> 1);
        static_for<decltype(first)::value, decltype(first)::value + decltype(count)::value>([&](auto i_c) __attribute__((always_inline)) {
            constexpr int i = decltype(i_c)::value;
            __attribute__((address_space(3))) uint8_t *dst = (__attribute__((address_space(3))) uint8_t *)(aring + stage + (wave * NA + i) * 1024);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(xres, dst, 16, (int)a_voff[i], pc * 128, 0, 0);
        });
    };

    v4i acc[RG][T];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int nt = 0; nt < T; nt++) acc[rg][nt] = v4i{0, 0, 0, 0};
    // sums of x over this lane's pieces of its RG pixels: rs runs one k-step ahead of the products (it is taken from the
    // operand read ahead), so what the epilogue uses is its value at the start of the last k-step
    uint32_t rs[RG], rs_final[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) rs[rg] = rs_final[rg] = 0;

    // s_waitcnt immediates (gfx9 encoding): vmcnt in bits [3:0] and [15:14], expcnt [6:4], lgkmcnt [11:8]
    constexpr auto waitcnt_imm = [](int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 15) << 8); };
    // ---- fill (the order is what the waits count) ----
    constexpr std::integral_constant<int, 0> c0;
    constexpr std::integral_constant<int, NW> cNW;
    constexpr std::integral_constant<int, NA> cNA;
    constexpr std::integral_constant<int, NW / 2> cNWh;
    constexpr std::integral_constant<int, NA / 2> cNAh;
    static_assert(NW % 2 == 0 && NA % 2 == 0, "requests are issued in halves");
    dma_w(0, 0, c0, cNW);
    dma_w(WSLOT, 1, c0, cNW);
    __builtin_amdgcn_sched_barrier(0);
    dma_a(0, 0, c0, cNA);
    __builtin_amdgcn_sched_barrier(0);
    dma_a(ASTAGE, 1, c0, cNA);
    __builtin_amdgcn_sched_barrier(0);
    dma_w(2 * WSLOT, 2, c0, cNW);
    __builtin_amdgcn_sched_barrier(0);
    dma_a(2 * ASTAGE, 2, c0, cNA);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(NA + NW + NA, 15)); // the first two k-steps' weights and the first pair's activations are in
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);

    // operand addresses: pixel (wm RG + rg) * 16 + j, piece (h * 4 + gq) of the stage, rotated by the pixel index
    const uint8_t *const x_src0 = aring + (wm * RG * 16 + j) * 128 + ((gq + j) & 7) * 16;     // first k-step of a pair, + rg * 2048
    const uint8_t *const x_src1 = aring + (wm * RG * 16 + j) * 128 + ((4 + gq + j) & 7) * 16; // second
    const uint8_t *const w_src = wring + (wn * T) * 1024 + lane * 16;                           // + nt * 1024
    // the last k-step may end inside the row: pieces past K meet zero weights, and are masked out of the sums of x
    const uint32_t tail_mask = (LM == kWideRows && (KS - 1) * 64 + gq * 16 >= a.k) ? 0u : 0xffffffffu;
    // weight operands are read two pairs of tiles ahead of their products (an LDS read under this load takes longer
    // than the eight matrix instructions of one pair): one register buffer per pair of a k-step
    static_assert(G == 4, "four pairs of channel tiles per k-step");
    v4i xf[2][RG], wf[G][2];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        xf[0][rg] = *reinterpret_cast<const v4i *>(x_src0 + rg * 2048);
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const uint32_t x = (uint32_t)xf[0][rg][d] & (LM == kWideRows && KS == 1 ? tail_mask : 0xffffffffu);
            rs[rg] = __builtin_amdgcn_sad_u8(x, 0u, rs[rg]);
            xf[0][rg][d] = (int)((uint32_t)xf[0][rg][d] ^ 0x80808080u);
        }
    }
    wf[0][0] = *reinterpret_cast<const v4i *>(w_src);
    wf[0][1] = *reinterpret_cast<const v4i *>(w_src + 1024);
    wf[1][0] = *reinterpret_cast<const v4i *>(w_src + 2048);
    wf[1][1] = *reinterpret_cast<const v4i *>(w_src + 3072);
    int wcur = 0, acur = 0; // ring offsets of k-step s: weight slot, activation stage (the latter moves every other k-step)
    auto kstep = [&](int s, auto parity) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value; // s & 1: operand buffer, and which half of the stage
        asm volatile("" : "+s"(wcur), "+s"(acur));
        const int wnxt = (wcur + WSLOT) & (NSW * WSLOT - 1), wnxt3 = (wcur + 3 * WSLOT) & (NSW * WSLOT - 1);
        // stage of k-step s + 1: the same for an even s, the next one for an odd s
        const int anext = acur + ASTAGE >= NSA * ASTAGE ? 0 : acur + ASTAGE;
        const int a_of_next = P == 0 ? acur : anext;
        const uint8_t *const ws = w_src + wcur;
        // the mask of the next k-step's sums (all ones but for the lanes past K of the last k-step)
        const uint32_t mask = (LM == kWideRows && s + 1 == KS - 1) ? tail_mask : 0xffffffffu;
        constexpr int NM = 2 * RG; // matrix instructions per group
        {
            const bool last = s == KS - 1;
#pragma unroll
            for (int rg = 0; rg < RG; rg++) rs_final[rg] = last ? rs[rg] : rs_final[rg];
        }
        static_for<0, G>([&](auto g_c) __attribute__((always_inline)) {
            constexpr int g = decltype(g_c)::value;
            constexpr int wb = g; // this pair's buffer
            __builtin_amdgcn_sched_barrier(0);
            {
                // the pair two on: of this k-step, or the first two of the next (whose slot is complete since the last barrier)
                constexpr int gn = (g + 2) % G;
                const uint8_t *const wsrc = (g + 2 < G ? ws : w_src + wnxt) + (2 * gn) * 1024;
                wf[gn][0] = *reinterpret_cast<const v4i *>(wsrc);
                wf[gn][1] = *reinterpret_cast<const v4i *>(wsrc + 1024);
            }
            if (g == 0) {
                // the next k-step's operand (its slot is complete since the last barrier): re-biased and summed under this k-step's products
                const uint8_t *const xn = (P == 0 ? x_src1 : x_src0) + a_of_next;
#pragma unroll
                for (int rg = 0; rg < RG; rg++) xf[1 - P][rg] = *reinterpret_cast<const v4i *>(xn + rg * 2048);
            }
            __builtin_amdgcn_sched_barrier(0);
            // Requests, a few per group so that the address unit's queue never fills and holds a wave at a load with its
            // matrix instructions behind it (in this order in the instruction stream: the wait below counts what
            // follows a k-step's weights): the weights of k-step s + 3 in halves (groups 0 and 2); activations in
            // quarters, pair (s + 5) / 2 in the odd k-step that frees its stage -- this k-step's own pair, whose last
            // operands were read in the first group of the previous k-step, by every wave before the barrier that
            // ended it -- and in the even one behind it (groups 1 and 3)
            if (g == 0) dma_w(wnxt3, s + 3, c0, cNWh);
            if (g == 2) dma_w(wnxt3, s + 3, cNWh, cNWh);
            if (P == 1) {
                if (g == 1) dma_a(acur, (s + 5) >> 1, c0, std::integral_constant<int, NA / 4>());
                if (g == 3) dma_a(acur, (s + 5) >> 1, std::integral_constant<int, NA / 4>(), std::integral_constant<int, NA / 4>());
            } else {
                // (an even k-step: the stage before this one's, pair (s + 4) / 2)
                const int aprev = acur == 0 ? (NSA - 1) * ASTAGE : acur - ASTAGE;
                if (g == 1) dma_a(aprev, (s + 4) >> 1, cNAh, std::integral_constant<int, NA / 4>());
                if (g == 3) dma_a(aprev, (s + 4) >> 1, std::integral_constant<int, 3 * NA / 4>(), std::integral_constant<int, NA / 4>());
            }
            static_for<0, NM>([&](auto m_c) __attribute__((always_inline)) {
                constexpr int m = decltype(m_c)::value, e = m / RG, rg = m % RG;
                acc[rg][2 * g + e] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[wb][e], xf[P][rg], acc[rg][2 * g + e], 0, 0, 0);
                // groups 1 .. G - 1 carry the 4 RG registers of the next operand, spread evenly: sum, then re-bias
                if constexpr (g >= 1) {
                    constexpr int slots = (G - 1) * NM;              // matrix instructions to spread over
                    constexpr int idx = (g - 1) * NM + m;            // this one's index
                    constexpr int lo = idx * (4 * RG) / slots, hi = (idx + 1) * (4 * RG) / slots;
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<lo, hi>([&](auto r_c) __attribute__((always_inline)) {
                        constexpr int r = decltype(r_c)::value, xr = r / 4, d = r % 4;
                        const uint32_t x = (uint32_t)xf[1 - P][xr][d];
                        rs[xr] = __builtin_amdgcn_sad_u8(LM == kWideRows ? (x & mask) : x, 0u, rs[xr]);
                        xf[1 - P][xr][d] = (int)(x ^ 0x80808080u);
                    });
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        wcur = wnxt;
        acur = a_of_next;
        __builtin_amdgcn_sched_barrier(0);
        // the weights of k-step s + 2 (requested during k-step s - 1) and the activations requested two and three
        // k-steps ago have landed: behind them came the last quarter of that k-step's activation runs, this k-step's
        // NW weight runs and its NA / 2 activation runs; of this wave's operand reads only the four of the next weights
        // may still be out
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(NA / 4 + NW + NA / 2, 4));
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    int s = 0;
#pragma clang loop unroll(disable)
    for (; s + 1 < KS; s += 2) {
        kstep(s, std::integral_constant<int, 0>());
        kstep(s + 1, std::integral_constant<int, 1>());
    }
    if (s < KS) kstep(s, std::integral_constant<int, 0>()); // an odd number of k-steps

    // ---- epilogue ----
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0)); // every DMA of this wave has landed, every operand read is back
    __syncthreads();                               // ... of every wave: the rings are free
    constexpr int NC = (TB * 16 + THREADS - 1) / THREADS;
#pragma unroll
    for (int i = 0; i < NC; i++) {
        const int c = i * THREADS + threadIdx.x;
        if (c < TB * 16) cterm[c] = ch_base + c < a.n ? a.bias[ch_base + c] - a.zxp * a.wsum[ch_base + c] + a.k * a.zxp * a.zwp : 0;
    }
    if (a.lut && threadIdx.x < 64) reinterpret_cast<uint32_t *>(lutl)[threadIdx.x] = a.lut[threadIdx.x];
    __syncthreads();
    // dword results (float32, int32) of eight channel tiles leave as whole lines; everything else through the shared epilogue
    const bool lines = T == 8 && a.ep.out_mode != kOutU8 && !a.deq;
    uint8_t *const stage = stage_base + wave * (lines ? line_store_bytes() : staged_store_bytes());
    const int ch0 = ch_base + gq * (4 * TB) + wn * (4 * T);
    const int32_t *ct = cterm + gq * (4 * TB) + wn * (4 * T) - gq * (4 * T); // the epilogues add gq * 4 T
    static_for<0, RG>([&](auto rg_c) __attribute__((always_inline)) {
        constexpr int rg = decltype(rg_c)::value;
        const int pl = (wm * RG + rg) * 16 + j;
        // the pixel's sum of x, spread over the lanes of its four pieces; x' = x - 128 over the K real positions
        int32_t sx = (int32_t)rs_final[rg];
        sx += __shfl_xor(sx, 16);
        sx += __shfl_xor(sx, 32);
        if constexpr (T == 8) {
            if (lines) {
                wide_store_lines<T>(a, acc[rg], sx - 128 * a.k, mt * PIX + pl, ch0, gq, ct, stage, 4 * TB);
                return;
            }
        }
        igemm_store_tile<T, kOwesAll, false, staged_store_built(T)>(a, acc[rg], sx - 128 * a.k, mt * PIX + pl, ch0, gq, ct, lutl, stage, 4 * TB);
    });
}

template <int T, int RG, int WM, int WN, int LM> int launch_wide_dma_t(nncase_hip_ctx *ctx, const IgemmArgs &a, int nchunks) {
    IgemmArgs args = a;
    constexpr int PIX = WM * RG * 16, TB = T * WN;
    args.num_mtiles = ceil_div(a.m, PIX);
    const int blocks = ceil_div(args.num_mtiles, 8) * 8 * nchunks;
    const size_t lds = (size_t)4 * TB * 1024 + (size_t)3 * PIX * 128;
    static std::once_flag raised[16]; // more than 64 KiB of dynamic LDS has to be asked for once per kernel and device
    hipError_t attr = hipSuccess;
    std::call_once(raised[ctx->device & 15], [&] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&qconv_wide_dma_kernel<T, RG, WM, WN, LM>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    });
    NNHIP_HIP(ctx, attr);
    hipLaunchKernelGGL((qconv_wide_dma_kernel<T, RG, WM, WN, LM>), dim3(blocks), dim3(WM * WN * 64), lds, ctx->stream, args, nchunks);
    NNHIP_LAUNCH_CHECK(ctx, "qconv_wide_dma_kernel");
    return 0;
}

template <int T, int RG, int WM, int WN, int LM> int launch_wide_t(nncase_hip_ctx *ctx, const IgemmArgs &a, int nchunks) {
    IgemmArgs args = a;
    constexpr int PIX = WM * RG * 16, TB = T * WN;
    args.num_mtiles = ceil_div(a.m, PIX);
    const int blocks = ceil_div(args.num_mtiles, 8) * 8 * nchunks;
    const size_t lds = (size_t)TB * 16 * sizeof(int32_t) + 256 + PIX * sizeof(int32_t) + (size_t)kWideSlots * (PIX * 64 + TB * 1024);
    if (lds > 65536) { // more than 64 KiB of dynamic LDS has to be asked for once per kernel and device
        static std::once_flag raised[16];
        hipError_t attr = hipSuccess;
        std::call_once(raised[ctx->device & 15], [&] {
            attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&qconv_wide_kernel<T, RG, WM, WN, LM>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        });
        NNHIP_HIP(ctx, attr);
    }
    hipLaunchKernelGGL((qconv_wide_kernel<T, RG, WM, WN, LM>), dim3(blocks), dim3(WM * WN * 64), lds, ctx->stream, args, nchunks);
    NNHIP_LAUNCH_CHECK(ctx, "qconv_wide_kernel");
    return 0;
}

// Pixel tiles of 256 while that gives every compute unit a block, else 128.
inline int wide_waves(const nncase_hip_ctx *ctx, int m, int nchunks) {
    return (long long)ceil_div(m, 256) * nchunks >= (long long)ctx->compute_units ? 4 : 2;
}

// Block shapes: tiles = 16 -> 256 pixels x 256 channels (4 x 2 waves); tiles = 8 -> 256 or 128 pixels x 128 channels;
// tiles = 4 -> 256 or 128 pixels x 64 channels.
template <int LM> int launch_wide_lm(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks) {
    if (tiles == 16) {
        if constexpr (LM == kWideRowsFull || LM == kWideRows) {
            if (a.x_bytes < ((size_t)1 << 31)) return launch_wide_dma_t<8, 4, 4, 2, LM>(ctx, a, nchunks);
        }
        return launch_wide4_t<8, 4, 4, 2, LM>(ctx, a, nchunks);
    }
    const int wmv = wide_waves(ctx, a.m, nchunks);
    if (tiles == 8) return wmv == 4 ? launch_wide_t<8, 4, 4, 1, LM>(ctx, a, nchunks) : launch_wide_t<8, 4, 2, 1, LM>(ctx, a, nchunks);
    if (tiles == 4) return wmv == 4 ? launch_wide_t<4, 4, 4, 1, LM>(ctx, a, nchunks) : launch_wide_t<4, 4, 2, 1, LM>(ctx, a, nchunks);
    return fail(ctx, -EINVAL, "qconv2d: no wide kernel for %d channel tiles", tiles);
}

template <int LM> int launch_wide_small_lm(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks) {
    if (tiles == 4) return launch_wide_t<4, 2, 4, 1, LM>(ctx, a, nchunks);
    if (tiles == 2) return launch_wide_t<2, 2, 2, 1, LM>(ctx, a, nchunks);
    return fail(ctx, -EINVAL, "qconv2d: no small wide kernel for %d channel tiles", tiles);
}
int launch_wide_small_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int variant, int nchunks);
int launch_wide_small_vec16(nncase_hip_ctx *ctx, const IgemmArgs &a, int variant, int nchunks);
int launch_wide_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks);
int launch_wide_vec16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks);

} // namespace nnhip
