// The rest of an LLM decode step around paged attention (fp16 activations, W8A16 weights):
// RMSNorm, the small-M weight-streaming GEMM, rotary embedding + KV append into the block-paged
// cache, arg-max, embedding gather and the per-step advance of the context lengths.
//
// A decode step multiplies a handful of token rows (M = batch, <= 64) with every weight matrix, so
// each int8 weight byte is read from HBM exactly once and the step is bound by that stream
// (~0.5 GB for a Qwen2-0.5B-shaped model).  The GEMM is organised around it: weights are
// pre-packed so that a wave's load of one k-step is a contiguous 1 KiB fragment (16 bytes per
// lane), converted int8 -> fp16 in registers (exactly: (w ^ 0x80) | 0x6400 is the fp16 1024 + w + 128)
// and fed to v_mfma_f32_16x16x32_f16 as the A operand (16 output channels), the token rows being
// the B operand; a lane ends up with 4 consecutive output channels of one token.  The four waves
// of a block split the reduction and combine through LDS.  Per-output-channel scales, bias, the
// residual add and the SwiGLU gate are applied in the epilogue.
#include "common.hpp"

#include <hip/hip_fp16.h>

#include <cmath>
#include <mutex>
#include <new>
#include <vector>

namespace nnhip {

typedef _Float16 h16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef uint32_t lu32x4 __attribute__((ext_vector_type(4)));

constexpr int kLlmThreads = 256;
constexpr int kMaxRows = 64; // token rows per GEMM call (4 MFMA column tiles)

} // namespace nnhip

// Pre-packed W8A16 matrix: out[m, n] = scale[n] * sum_k a[m, k] * w[n, k] (+ bias[n]).
struct nncase_hip_w8a16 {
    int k = 0, n = 0;      // reduction length (multiple of 64), output channels (multiple of 16)
    int ntiles = 0, ksteps = 0;
    void *d_packed = nullptr; // [ntiles][ksteps][64 lanes][16 B]: lane (i = l % 16, kg = l / 16) holds
                              // w[tile * 16 + i][ks * 64 + kg * 16 .. + 15]
    float *d_scale = nullptr; // [n]
    float *d_bias = nullptr;  // [n] or null
};

namespace nnhip {

struct RopeArgs {
    const __half *qkv; // [batch][(hq + 2 * hkv) * d]: q heads, then k heads, then v heads
    __half *q_out;     // [batch][hq][d]
    __half *k_cache;   // [blocks][hkv][block][d]
    __half *v_cache;   // [blocks][hkv][d][block]
    const int32_t *block_table, *ctx_lens; // the new token of sequence b goes to position ctx_lens[b]
    int batch, hq, hkv, d, block_size, max_blocks, num_blocks;
    float theta;
};

struct GemmArgs {
    const uint16_t *a; // [m][k] fp16
    const lu32x4 *w;
    const float *scale, *bias;
    const uint16_t *residual; // [m][n_out] fp16 or null
    void *out;                // [m][n_out] fp16 or fp32
    int m, k, n_out, ksteps, mode, out_f32;
    int up_tile_offset; // SwiGLU: tile t of the gate pairs with tile t + up_tile_offset of the up projection
    // RMS normalisation of the token rows in front of the product (null: none): the block computes every row's
    // 1 / sqrt(mean(x^2) + eps) the way rmsnorm_f16_kernel does, and a token slice becomes
    // fp16(x * r * weight) as it is loaded, so the result is what the two kernels give one after the other
    const uint16_t *ln_w; // [k] fp16
    float ln_eps;
    // ROPE kernels: the product is a q / k / v projection whose rows do not go to `out` but, rotated, to the query buffer
    // and the paged cache (rope.qkv unused)
    RopeArgs rope;
};

// 1 / sqrt(mean(x^2) + eps) of a row, the way every kernel here forms it.  A lane owns the 8 consecutive elements
// 8 * lane .. 8 * lane + 7 of every 512-element piece of the row (one 16-byte load per piece); it adds their squares
// in index order, piece after piece, and a butterfly adds the 64 lanes.  The order is part of the definition: the
// product kernel that normalises its own rows must arrive at the same bits as rmsnorm_f16_kernel.
__device__ __forceinline__ void add_squares8(const lu32x4 &v, float &ss) {
    __half h[8];
    __builtin_memcpy(h, &v, 16);
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const float f = __half2float(h[e]);
        ss += f * f;
    }
}
__device__ __forceinline__ float rstd_from_sum(float ss, int hidden, float eps) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    return 1.0f / sqrtf(ss / (float)hidden + eps);
}
// R rows at once (row r0 + i * stride for i < R, those below `rows`): the loads of one piece of all of them are in
// flight together.  hidden is a multiple of 8 and the rows are 16-byte aligned.
template <int R>
__device__ __forceinline__ void rms_rstd_rows(const __half *x, int hidden, int rows, int r0, int stride, int lane, float eps,
                                              float (&out)[R]) {
    float ss[R];
#pragma unroll
    for (int i = 0; i < R; i++) ss[i] = 0.f;
    for (int e0 = lane * 8; e0 < ((hidden + 511) & ~511); e0 += 512) {
        lu32x4 v[R];
#pragma unroll
        for (int i = 0; i < R; i++) {
            const int r = r0 + i * stride;
            v[i] = lu32x4{0, 0, 0, 0}; // (+0 squares leave a sum as it is)
            if (r < rows && e0 < hidden) v[i] = *reinterpret_cast<const lu32x4 *>(x + (size_t)r * hidden + e0);
        }
#pragma unroll
        for (int i = 0; i < R; i++) add_squares8(v[i], ss[i]);
    }
#pragma unroll
    for (int i = 0; i < R; i++) out[i] = rstd_from_sum(ss[i], hidden, eps);
}
// any row length and alignment: the same order with one element per load
__device__ __forceinline__ float rms_rstd_scalar(const __half *xr, int hidden, float eps, int lane) {
    float ss = 0.f;
    for (int e0 = lane * 8; e0 < ((hidden + 511) & ~511); e0 += 512)
        for (int e = 0; e < 8; e++)
            if (e0 + e < hidden) {
                const float f = __half2float(xr[e0 + e]);
                ss += f * f;
            }
    return rstd_from_sum(ss, hidden, eps);
}

// One rotate-half pair of the new token of sequence b: elements i and i + d/2 of head h (q heads, then k heads, then
// v heads), given as the fp16 values the projection stores.  q goes rotated to the query buffer, k rotated and v as it
// is to position ctx_lens[b] of the paged cache.  The one definition of that arithmetic: the rope kernel and the
// projection that rotates in its own epilogue both call it.
__device__ __forceinline__ void rope_store_pair(const RopeArgs &a, int b, int h, int i, float x0, float x1) {
    const int half = a.d / 2;
    const int pos = a.ctx_lens[b];
    const int lb = pos / a.block_size, in_block = pos - lb * a.block_size;
    const bool fits = pos >= 0 && lb < a.max_blocks; // a negative length appends nothing (it would index before the block)
    const int pb = fits ? min(max(a.block_table[(size_t)b * a.max_blocks + lb], 0), a.num_blocks - 1) : 0;
    if (h < a.hq + a.hkv) {
        const float inv = powf(a.theta, -2.0f * (float)i / (float)a.d);
        const float ang = (float)pos * inv;
        const float c = cosf(ang), s = sinf(ang);
        const __half y0 = __float2half_rn(x0 * c - x1 * s), y1 = __float2half_rn(x1 * c + x0 * s);
        if (h < a.hq) {
            __half *dst = a.q_out + ((size_t)b * a.hq + h) * a.d;
            dst[i] = y0, dst[i + half] = y1;
        } else if (fits) {
            __half *dst = a.k_cache + ((((size_t)pb * a.hkv + (h - a.hq)) * a.block_size) + in_block) * a.d;
            dst[i] = y0, dst[i + half] = y1;
        }
    } else if (fits) {
        __half *dst = a.v_cache + ((size_t)pb * a.hkv + (h - a.hq - a.hkv)) * a.d * a.block_size + in_block;
        dst[(size_t)i * a.block_size] = __float2half_rn(x0);
        dst[(size_t)(i + half) * a.block_size] = __float2half_rn(x1);
    }
}

// 8 int8 weights (two dwords' low / high halves handled by the caller) -> 8 fp16, exact.
__device__ __forceinline__ h16x8 w8_to_f16(uint32_t lo, uint32_t hi) {
    const uint32_t x0 = lo ^ 0x80808080u, x1 = hi ^ 0x80808080u;
    uint32_t h[4];
    h[0] = __builtin_amdgcn_perm(0x64646464u, x0, 0x07010700u); // [b0, 0x64, b1, 0x64] -> halves 1024 + b0, 1024 + b1
    h[1] = __builtin_amdgcn_perm(0x64646464u, x0, 0x07030702u);
    h[2] = __builtin_amdgcn_perm(0x64646464u, x1, 0x07010700u);
    h[3] = __builtin_amdgcn_perm(0x64646464u, x1, 0x07030702u);
    h16x8 v;
    __builtin_memcpy(&v, h, 16);
    return v - (_Float16)1152.0f; // 1024 + (w + 128) - 1152 = w, exact in fp16
}

// Epilogue of 4 consecutive output channels of one token: SwiGLU gate, residual, conversion, store.  `res`: the four
// residual halves where the caller has loaded them already (have_res), else they are read here.
template <int G> __device__ __forceinline__ void store_gemm_row(const GemmArgs &a, const float (&v)[G][4], size_t o, uint2 res = uint2{0u, 0u},
                                                               bool have_res = false) {
    float y[4];
    if (a.residual && !have_res) res = *reinterpret_cast<const uint2 *>(a.residual + o);
    __half rh[4];
    __builtin_memcpy(rh, &res, 8);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (G == 2) y[r] = v[0][r] / (1.f + __expf(-v[0][r])) * v[G - 1][r]; // silu(gate) * up
        else y[r] = v[0][r];
        if (a.residual) y[r] += __half2float(rh[r]);
    }
    if (a.out_f32) {
        *reinterpret_cast<float4 *>(reinterpret_cast<float *>(a.out) + o) = float4{y[0], y[1], y[2], y[3]};
    } else {
        __half h[4];
#pragma unroll
        for (int r = 0; r < 4; r++) h[r] = __float2half_rn(y[r]);
        uint2 pk;
        __builtin_memcpy(&pk, h, 8);
        *reinterpret_cast<uint2 *>(reinterpret_cast<__half *>(a.out) + o) = pk;
    }
}

// MT = 16-token column tiles (m <= 16 * MT); G = matrices multiplied at once (2: SwiGLU gate and up).
// grid.x = output tiles of 16 channels.  The eight waves of a block split the reduction; a wave
// requests the weights and token slices of four k-steps before it multiplies any of them, so a
// whole share of a short reduction (896 / 8 waves = 2 k-steps) is a single memory round trip.
constexpr int kGemmWaves = 8;
constexpr int kGemmThreads = kGemmWaves * 64;
constexpr int kGemmBatch = 4; // k-steps a wave requests before it multiplies any (5 where that halves a long share's trips to memory)

// SPLIT: the block's waves share one output tile and split its reduction (few tiles, long reductions);
// otherwise every wave owns a tile of its own and the whole reduction (many tiles: the vocabulary head).
template <int MT, int G, bool SPLIT, int B = kGemmBatch> __global__ __launch_bounds__(kGemmThreads) void w8a16_gemm_kernel(const GemmArgs a) {
    __shared__ float red[SPLIT ? kGemmWaves : 1][G][MT][64][4];
    __shared__ float rstd[MT * 16];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i16 = lane & 15, kg = lane >> 4;
    if (a.ln_w) { // (uniform; before any wave leaves the block)
        constexpr int R = MT * 16 / kGemmWaves; // rows per wave
        float rs[R];
        rms_rstd_rows<R>(reinterpret_cast<const __half *>(a.a), a.k, a.m, wave, kGemmWaves, lane, a.ln_eps, rs);
        if (lane == 0) {
#pragma unroll
            for (int i = 0; i < R; i++)
                if (wave + i * kGemmWaves < a.m) rstd[wave + i * kGemmWaves] = rs[i];
        }
        __syncthreads();
    }
    const int per = SPLIT ? (a.ksteps + kGemmWaves - 1) / kGemmWaves : a.ksteps;
    const int ks0 = SPLIT ? wave * per : 0, ks1 = min(a.ksteps, ks0 + per);
    const int out_tile = SPLIT ? (int)blockIdx.x : (int)blockIdx.x * kGemmWaves + wave;
    if (out_tile >= a.up_tile_offset) return; // SPLIT: never; otherwise the last block's spare waves (uniform per wave)
    f32x4v acc[G][MT];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[g][t] = f32x4v{0.f, 0.f, 0.f, 0.f};

    const int tile[2] = {out_tile, out_tile + a.up_tile_offset};
    // token rows of this lane (clamped: rows past m read row m - 1 and are never stored)
    const uint16_t *arow[MT];
    float rrow[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) {
        arow[t] = a.a + (size_t)min(t * 16 + i16, a.m - 1) * a.k + kg * 16;
        rrow[t] = a.ln_w ? rstd[min(t * 16 + i16, a.m - 1)] : 1.f;
    }

    // The epilogue's operands (SPLIT: of the token tile this wave finishes) are asked for before the products: the
    // launch is a chain of memory round trips, and this takes the last one out of it.
    // (not with four token tiles: their slices leave no registers for it)
    constexpr bool kPre = SPLIT && MT <= 2;
    float4 sc[G], bs[G];
    uint2 res_pre = uint2{0u, 0u};
    if (kPre) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            sc[g] = *reinterpret_cast<const float4 *>(a.scale + tile[g] * 16 + kg * 4);
            bs[g] = float4{0.f, 0.f, 0.f, 0.f};
            if (a.bias) bs[g] = *reinterpret_cast<const float4 *>(a.bias + tile[g] * 16 + kg * 4);
        }
        const int m_pre = min(min(wave, MT - 1) * 16 + i16, a.m - 1);
        if (a.residual) res_pre = *reinterpret_cast<const uint2 *>(a.residual + (size_t)m_pre * a.n_out + out_tile * 16 + kg * 4);
    }
    for (int kb = ks0; kb < ks1; kb += B) {
        lu32x4 wv[B][G];
        lu32x4 av[B][MT][2];
        lu32x4 lw[B][2]; // the normalisation weights of the lane's 16 reduction indices
#pragma unroll
        for (int u = 0; u < B; u++) {
            const int ks = min(kb + u, ks1 - 1); // steps past the share re-read the last one and are not multiplied
#pragma unroll
            for (int g = 0; g < G; g++) wv[u][g] = a.w[((size_t)tile[g] * a.ksteps + ks) * 64 + lane];
#pragma unroll
            for (int t = 0; t < MT; t++) {
                av[u][t][0] = *reinterpret_cast<const lu32x4 *>(arow[t] + ks * 64);
                av[u][t][1] = *reinterpret_cast<const lu32x4 *>(arow[t] + ks * 64 + 8);
            }
            if (a.ln_w) {
                lw[u][0] = *reinterpret_cast<const lu32x4 *>(a.ln_w + ks * 64 + kg * 16);
                lw[u][1] = *reinterpret_cast<const lu32x4 *>(a.ln_w + ks * 64 + kg * 16 + 8);
            }
        }
        if (a.ln_w) {
#pragma unroll
            for (int u = 0; u < B; u++)
                if (MT > 2 || kb + u < ks1) // (uniform for the wave: the slices past its share are not multiplied; four token tiles have no registers to spare for the branch)
#pragma unroll
                for (int t = 0; t < MT; t++)
#pragma unroll
                    for (int hlf = 0; hlf < 2; hlf++) {
                        __half xh[8], wh[8];
                        __builtin_memcpy(xh, &av[u][t][hlf], 16);
                        __builtin_memcpy(wh, &lw[u][hlf], 16);
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            // the fp32 product is rounded before it is converted, as in rmsnorm_f16_kernel (see there)
                            float pr = __half2float(xh[e]) * rrow[t] * __half2float(wh[e]);
                            asm volatile("" : "+v"(pr));
                            xh[e] = __float2half_rn(pr);
                        }
                        __builtin_memcpy(&av[u][t][hlf], xh, 16);
                    }
        }
#pragma unroll
        for (int u = 0; u < B; u++) {
            if (kb + u < ks1) { // uniform for the wave
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const h16x8 w0 = w8_to_f16(wv[u][g][0], wv[u][g][1]), w1 = w8_to_f16(wv[u][g][2], wv[u][g][3]);
#pragma unroll
                    for (int t = 0; t < MT; t++) {
                        h16x8 x0, x1;
                        __builtin_memcpy(&x0, &av[u][t][0], 16);
                        __builtin_memcpy(&x1, &av[u][t][1], 16);
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, x0, acc[g][t], 0, 0, 0);
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, x1, acc[g][t], 0, 0, 0);
                    }
                }
            }
        }
    }
    // ---- combine the waves' partial sums ------------------------------------------------------------
    if (SPLIT) {
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) red[wave][g][t][lane][r] = acc[g][t][r];
        __syncthreads();
        if (wave >= MT) return; // wave w finishes token tile w
    }
    // lane (i16 = token within the tile, kg): channels tile * 16 + kg * 4 + r
#pragma unroll
    for (int tt = 0; tt < (SPLIT ? 1 : MT); tt++) {
        const int t = SPLIT ? wave : tt;
        const int m = t * 16 + i16;
        float v[G][4];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float scv[4] = {sc[g].x, sc[g].y, sc[g].z, sc[g].w}, bsv[4] = {bs[g].x, bs[g].y, bs[g].z, bs[g].w};
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float s = 0.f;
                if (SPLIT) {
#pragma unroll
                    for (int w = 0; w < kGemmWaves; w++) s += red[w][g][t][lane][r]; // fixed order: deterministic
                } else {
                    s = acc[g][tt][r];
                }
                if (kPre) {
                    s *= scv[r];
                    if (a.bias) s += bsv[r];
                } else {
                    const int ch = tile[g] * 16 + kg * 4 + r;
                    s *= a.scale[ch];
                    if (a.bias) s += a.bias[ch];
                }
                v[g][r] = s;
            }
        }
        if (m >= a.m) continue;
        store_gemm_row<G>(a, v, (size_t)m * a.n_out + out_tile * 16 + kg * 4, res_pre, kPre);
    }
}

// Many output tiles and a reduction short enough for the token rows to fit in LDS (the vocabulary head, the gate / up
// projection): a wave owns a tile (G = 2: the gate tile and its up tile) and the whole reduction, as in the kernel
// above without SPLIT, but the block's waves share the token rows through LDS.  A wave brings in whole rows (row
// wave, wave + WAVES, ...): it adds their squares in rms_rstd_rows' order as they arrive, parks them in LDS as loaded,
// and, knowing 1 / sqrt(mean + eps) of its own rows without asking another wave, normalises them in place -- one trip
// to memory and one barrier in front of the products, and every element normalised once per block instead of once per
// wave.  A wave has the weights of KB k-steps in flight, the first KB from the start of the kernel.  The arithmetic per element and the order of the
// multiply-adds are those of the kernel above.
constexpr int kRowsBatch = 8;
constexpr int kGluSplitWaves = 4;             // waves that split the reduction of one gate / up tile pair
constexpr int kRowsPieces = 4;                 // 512-element pieces of a row: k <= 2048
constexpr int kRowsMaxK = kRowsPieces * 512;
inline int rows_in_lds_pitch(int k) { return k * 2 + 16; } // bytes per token row: the padding spreads the rows over the banks

// SPLIT: the block's waves share ONE output tile and split its reduction (few tiles: the q / k / v projection), combined
// through LDS in the fixed order of the kernel above.
// ROPE (with SPLIT and G = 2): a q / k / v projection whose block owns the two tiles that hold the halves of eight
// rotate-half pairs -- tile j of a head and tile j + up_tile_offset (= head_dim / 32) -- so that a lane ends up with
// both elements of its four pairs; the epilogue rounds them to fp16 as the projection's output would be stored and
// hands them to rope_store_pair.
template <int MT, int G, int WAVES, bool SPLIT = false, int KB = kRowsBatch, int PIECES = kRowsPieces, bool ROPE = false>
__global__ __launch_bounds__(WAVES * 64) void w8a16_gemm_rows_in_lds_kernel(const GemmArgs a) {
    static_assert(!ROPE || (SPLIT && G == 2), "the rotating epilogue pairs two tiles of one block");
    extern __shared__ __attribute__((aligned(16))) uint8_t xs[]; // [MT * 16][k halves + padding]
    __shared__ float red[SPLIT ? WAVES : 1][G][SPLIT ? MT : 1][64][4];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i16 = lane & 15, kg = lane >> 4;
    const int pitch = a.k * 2 + 16;
    // The weights do not depend on the rows: the first KB k-steps of this wave's share are requested before anything
    // else, so that their trip to memory runs beside the one that brings the rows in (a spare wave of the last block
    // reads the last tile's and multiplies nothing).
    // Without SPLIT a block walks the groups of WAVES tiles blockIdx.x, blockIdx.x + gridDim.x, ...: a launch with fewer
    // blocks than groups (the vocabulary head) brings the rows in and normalises them once per block, not once per group.
    int group = (int)blockIdx.x;
    int out_tile = ROPE    ? ((int)blockIdx.x / a.up_tile_offset) * (2 * a.up_tile_offset) + (int)blockIdx.x % a.up_tile_offset
                   : SPLIT ? (int)blockIdx.x
                           : group * WAVES + wave;
    const int per = SPLIT ? (a.ksteps + WAVES - 1) / WAVES : a.ksteps;
    const int ks0 = SPLIT ? wave * per : 0, ks1 = min(a.ksteps, ks0 + per);
    int first = ROPE ? out_tile : min(out_tile, a.up_tile_offset - 1);
    int tile[2] = {first, first + a.up_tile_offset};
    lu32x4 wv[KB][G];
    auto request_first = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < KB; u++) {
            const int ks = max(min(ks0 + u, ks1 - 1), 0); // steps past the share re-read its last one (an empty share: step 0) and are not multiplied
#pragma unroll
            for (int g = 0; g < G; g++) wv[u][g] = a.w[((size_t)tile[g] * a.ksteps + ks) * 64 + lane];
        }
    };
    request_first();
    {
        constexpr int R = MT * 16 / WAVES; // rows per wave
        // The wave's rows stay in registers from the load to the one LDS write: their sums of squares, the butterflies
        // and the normalisation run for all R rows side by side (independent chains), element by element in the order
        // rms_rstd_rows and rmsnorm_f16_kernel use.
        lu32x4 v[R][PIECES], lwp[PIECES];
#pragma unroll
        for (int p = 0; p < PIECES; p++) {
            const int e0 = lane * 8 + p * 512;
            lwp[p] = lu32x4{0, 0, 0, 0};
            if (a.ln_w && e0 < a.k) lwp[p] = *reinterpret_cast<const lu32x4 *>(a.ln_w + e0);
#pragma unroll
            for (int i = 0; i < R; i++) {
                const int r = wave + i * WAVES;
                v[i][p] = lu32x4{0, 0, 0, 0}; // rows past m: zeros (their products are never stored)
                if (r < a.m && e0 < a.k) v[i][p] = *reinterpret_cast<const lu32x4 *>(a.a + (size_t)r * a.k + e0);
            }
        }
            if (a.ln_w) {
            float ss[R];
#pragma unroll
            for (int i = 0; i < R; i++) ss[i] = 0.f;
#pragma unroll
            for (int p = 0; p < PIECES; p++)
#pragma unroll
                for (int i = 0; i < R; i++) add_squares8(v[i][p], ss[i]); // (pieces past the row are zeros: +0 leaves a sum as it is)
#pragma unroll
            for (int o = 32; o > 0; o >>= 1)
#pragma unroll
                for (int i = 0; i < R; i++) ss[i] += __shfl_xor(ss[i], o);
            float rr[R];
#pragma unroll
            for (int i = 0; i < R; i++) rr[i] = 1.0f / sqrtf(ss[i] / (float)a.k + a.ln_eps); // rstd_from_sum's formula
#pragma unroll
            for (int p = 0; p < PIECES; p++) {
                __half wh[8];
                __builtin_memcpy(wh, &lwp[p], 16);
                __half xh[R][8];
#pragma unroll
                for (int i = 0; i < R; i++) __builtin_memcpy(xh[i], &v[i][p], 16);
#pragma unroll
                for (int e = 0; e < 8; e++)
#pragma unroll
                    for (int i = 0; i < R; i++) {
                        // the fp32 product is rounded before it is converted, as in rmsnorm_f16_kernel (see there)
                        float pr = __half2float(xh[i][e]) * rr[i] * __half2float(wh[e]);
                        asm volatile("" : "+v"(pr));
                        xh[i][e] = __float2half_rn(pr);
                    }
#pragma unroll
                for (int i = 0; i < R; i++) __builtin_memcpy(&v[i][p], xh[i], 16);
            }
        }
#pragma unroll
        for (int p = 0; p < PIECES; p++) {
            const int e0 = lane * 8 + p * 512;
            if (e0 < a.k) {
#pragma unroll
                for (int i = 0; i < R; i++) *reinterpret_cast<lu32x4 *>(xs + (size_t)(wave + i * WAVES) * pitch + e0 * 2) = v[i][p];
            }
        }
    }
    __syncthreads();
    const int groups = SPLIT ? 0 : (a.up_tile_offset + WAVES - 1) / WAVES;
    for (;;) { // (one pass with SPLIT)
    if (!ROPE && out_tile >= a.up_tile_offset) return; // SPLIT: never; otherwise the last group's spare waves (uniform per wave; no group follows it)
    f32x4v acc[G][MT];
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
        for (int t = 0; t < MT; t++) acc[g][t] = f32x4v{0.f, 0.f, 0.f, 0.f};
    const uint8_t *xl = xs + (size_t)i16 * pitch + kg * 32; // the lane's 16 reduction indices of a k-step
    float4 sc[G], bs[G]; // the epilogue's operands, asked for before the products
#pragma unroll
    for (int g = 0; g < G; g++) {
        sc[g] = *reinterpret_cast<const float4 *>(a.scale + tile[g] * 16 + kg * 4);
        bs[g] = float4{0.f, 0.f, 0.f, 0.f};
        if (a.bias) bs[g] = *reinterpret_cast<const float4 *>(a.bias + tile[g] * 16 + kg * 4);
    }
    uint2 res_pre = uint2{0u, 0u};
    if (SPLIT && a.residual) // (the token tile this wave finishes)
        res_pre = *reinterpret_cast<const uint2 *>(a.residual + (size_t)min(min(wave, MT - 1) * 16 + i16, a.m - 1) * a.n_out + out_tile * 16 + kg * 4);
    for (int kb = ks0; kb < ks1; kb += KB) {
        if (kb != ks0) { // (the first batch is on its way since the start)
#pragma unroll
            for (int u = 0; u < KB; u++) {
                const int ks = min(kb + u, ks1 - 1); // steps past the end re-read the last one and are not multiplied
#pragma unroll
                for (int g = 0; g < G; g++) wv[u][g] = a.w[((size_t)tile[g] * a.ksteps + ks) * 64 + lane];
            }
        }
#pragma unroll
        for (int u = 0; u < KB; u++) {
            if (kb + u < ks1) { // uniform
                h16x8 x0[MT], x1[MT];
#pragma unroll
                for (int t = 0; t < MT; t++) {
                    const uint8_t *xp = xl + (size_t)t * 16 * pitch + (size_t)(kb + u) * 128;
                    x0[t] = *reinterpret_cast<const h16x8 *>(xp), x1[t] = *reinterpret_cast<const h16x8 *>(xp + 16);
                }
#pragma unroll
                for (int g = 0; g < G; g++) {
                    const h16x8 w0 = w8_to_f16(wv[u][g][0], wv[u][g][1]), w1 = w8_to_f16(wv[u][g][2], wv[u][g][3]);
#pragma unroll
                    for (int t = 0; t < MT; t++) {
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w0, x0[t], acc[g][t], 0, 0, 0);
                        acc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w1, x1[t], acc[g][t], 0, 0, 0);
                    }
                }
            }
        }
    }
    // the next group's first weights are requested as soon as this one's are multiplied: they travel under the epilogue
    group += (int)gridDim.x;
    const bool more = !SPLIT && group < groups;
    const int next_tile = group * WAVES + wave;
    if (more) {
        first = min(next_tile, a.up_tile_offset - 1);
        tile[0] = first, tile[1] = first + a.up_tile_offset;
        request_first();
    }
    if (SPLIT) {
#pragma unroll
        for (int g = 0; g < G; g++)
#pragma unroll
            for (int t = 0; t < MT; t++)
#pragma unroll
                for (int r = 0; r < 4; r++) red[wave][g][t][lane][r] = acc[g][t][r];
        __syncthreads();
        if constexpr (ROPE) {
            // The rotation costs a few hundred instructions per pair (the angle's power, sine and cosine), so the
            // pairs are spread over all the waves: wave w takes channel w % 4 of each lane's four, token tile w / 4.
            static_assert(WAVES == 8, "channel w % 4, token tile w / 4");
            const int t = wave >> 2, r = wave & 3;
            const int m = t * 16 + i16;
            if (t >= MT || m >= a.m) return;
            float v2[2];
#pragma unroll
            for (int g = 0; g < 2; g++) {
                const float scv[4] = {sc[g].x, sc[g].y, sc[g].z, sc[g].w}, bsv[4] = {bs[g].x, bs[g].y, bs[g].z, bs[g].w};
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; w++) s += red[w][g][t][lane][r]; // fixed order, as below
                float sv = scv[0], bv = bsv[0];
#pragma unroll
                for (int q = 1; q < 4; q++) sv = r == q ? scv[q] : sv, bv = r == q ? bsv[q] : bv;
                s *= sv;
                if (a.bias) s += bv;
                v2[g] = s;
            }
            // (rounded to fp16 as the projection's output would be stored; the partner is d / 2 channels further)
            const int c = out_tile * 16 + kg * 4 + r;
            rope_store_pair(a.rope, m, c / a.rope.d, c % a.rope.d, __half2float(__float2half_rn(v2[0])), __half2float(__float2half_rn(v2[1])));
            return;
        }
        if (wave >= MT) return; // wave w finishes token tile w
    }
    // lane (i16 = token within the tile, kg): channels tile * 16 + kg * 4 + r
#pragma unroll
    for (int tt = 0; tt < (SPLIT ? 1 : MT); tt++) {
        const int t = SPLIT ? wave : tt;
        const int m = t * 16 + i16;
        float v[G][4];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float scv[4] = {sc[g].x, sc[g].y, sc[g].z, sc[g].w}, bsv[4] = {bs[g].x, bs[g].y, bs[g].z, bs[g].w};
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float s = 0.f;
                if (SPLIT) {
#pragma unroll
                    for (int w = 0; w < WAVES; w++) s += red[w][g][t][lane][r]; // fixed order: deterministic
                } else {
                    s = acc[g][tt][r];
                }
                s *= scv[r];
                if (a.bias) s += bsv[r];
                v[g][r] = s;
            }
        }
        if (m >= a.m) continue;
        store_gemm_row<G>(a, v, (size_t)m * a.n_out + out_tile * 16 + kg * 4, res_pre, SPLIT);
    }
    if (!more) return;
    out_tile = next_tile;
    }
}

// out[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * weight, fp32 arithmetic; one wave per row.
__global__ __launch_bounds__(kLlmThreads) void rmsnorm_f16_kernel(const __half *__restrict__ x, const __half *__restrict__ w,
                                                                 __half *__restrict__ out, int rows, int hidden, float eps) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= rows) return;
    const __half *xr = x + (size_t)row * hidden;
    float r;
    if ((hidden & 7) == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
        float rs[1];
        rms_rstd_rows<1>(x, hidden, rows, row, 1, lane, eps, rs);
        r = rs[0];
    } else {
        r = rms_rstd_scalar(xr, hidden, eps, lane);
    }
    for (int i = lane; i < hidden; i += 64) {
        // The fp32 product is rounded before it is converted to fp16.  Left to itself the compiler turns multiply and
        // conversion into one mixed-precision instruction (a single rounding) in some copies of this loop's body
        // and not in others, so the same input could round either way depending on where it sits in the row.
        float pr = __half2float(xr[i]) * r * __half2float(w[i]);
        asm volatile("" : "+v"(pr));
        out[(size_t)row * hidden + i] = __float2half_rn(pr);
    }
}

// Rotary embedding (rotate-half pairing: element i with i + d/2, angle pos * theta^(-2i/d)) of the q
// and k heads of the new token, and the append of the rotated k and of v at position ctx_lens[b]
// of the paged cache.  One thread per (sequence, head, pair).
__global__ __launch_bounds__(kLlmThreads) void rope_append_kernel(const RopeArgs a) {
    const int half = a.d / 2;
    const int heads = a.hq + 2 * a.hkv;
    const int gid = blockIdx.x * kLlmThreads + threadIdx.x;
    if (gid >= a.batch * heads * half) return;
    const int i = gid % half, h = (gid / half) % heads, b = gid / (half * heads);
    const __half *src = a.qkv + ((size_t)b * heads + h) * a.d;
    rope_store_pair(a, b, h, i, __half2float(src[i]), __half2float(src[i + half]));
}

// Index of the largest element of every row (the lowest index among equals); one block of 1024
// threads per row, 16-byte loads, so that a 152 K-entry vocabulary row is a few dozen independent
// loads per thread.
constexpr int kArgmaxThreads = 1024;
__device__ __forceinline__ void argmax_take(float v, int i, float &best, int &bi) {
    if (v > best || (v == best && i < bi)) best = v, bi = i;
}
__global__ __launch_bounds__(kArgmaxThreads) void argmax_f32_kernel(const float *__restrict__ x, int32_t *__restrict__ out, int cols) {
    __shared__ float sv[kArgmaxThreads / 64];
    __shared__ int si[kArgmaxThreads / 64];
    const float *row = x + (size_t)blockIdx.x * cols;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    // rows start 16-byte aligned when cols is a multiple of 4 (x itself is aligned by the allocator)
    const int nvec = ((cols & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) ? cols / 4 : 0;
    // eight 16-byte loads per thread are requested before any of them is compared: a row of the vocabulary is five
    // memory round trips, not one per load
    constexpr int U = 8;
    for (int i0 = threadIdx.x; i0 < nvec; i0 += U * kArgmaxThreads) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = reinterpret_cast<const float4 *>(row)[min(i0 + u * kArgmaxThreads, nvec - 1)];
        // the batch's maximum first (one instruction per element); only a batch that beats the running maximum -- a
        // handful per thread -- is searched for where (its first such element: indices grow with u and i0)
        float m = -INFINITY;
#pragma unroll
        for (int u = 0; u < U; u++)
            if (i0 + u * kArgmaxThreads < nvec) m = fmaxf(m, fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w)));
        if (m > best) {
            best = m;
            bi = 0x7fffffff;
#pragma unroll
            for (int u = U - 1; u >= 0; u--) {
                const int i = i0 + u * kArgmaxThreads;
                if (i < nvec) {
                    bi = v[u].w == m ? 4 * i + 3 : bi;
                    bi = v[u].z == m ? 4 * i + 2 : bi;
                    bi = v[u].y == m ? 4 * i + 1 : bi;
                    bi = v[u].x == m ? 4 * i : bi;
                }
            }
        }
    }
    for (int i = nvec * 4 + threadIdx.x; i < cols; i += kArgmaxThreads) argmax_take(row[i], i, best, bi);
    // the wave's winner by exchanges between lanes, the block's through LDS
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) argmax_take(__shfl_xor(best, d), __shfl_xor(bi, d), best, bi);
    if ((threadIdx.x & 63) == 0) sv[threadIdx.x >> 6] = best, si[threadIdx.x >> 6] = bi;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kArgmaxThreads / 64; w++) argmax_take(sv[w], si[w], best, bi);
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

__global__ __launch_bounds__(kLlmThreads) void embed_f16_kernel(const __half *__restrict__ table, const int32_t *__restrict__ ids,
                                                               __half *__restrict__ out, int rows, int hidden, int vocab) {
    const int gid = blockIdx.x * kLlmThreads + threadIdx.x;
    if (gid >= rows * hidden) return;
    const int r = gid / hidden, c = gid - r * hidden;
    const int id = min(max(ids[r], 0), vocab - 1);
    out[gid] = table[(size_t)id * hidden + c];
}

__global__ void add_i32_kernel(int32_t *x, int n, int32_t delta) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += delta;
}

} // namespace nnhip

using namespace nnhip;

extern "C" int nncase_hip_w8a16_destroy(nncase_hip_ctx_t *ctx, nncase_hip_w8a16_t *w) {
    NNHIP_CHECK_CTX(ctx);
    if (!w) return 0;
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (w->d_packed) (void)hipFree(w->d_packed);
    if (w->d_scale) (void)hipFree(w->d_scale);
    if (w->d_bias) (void)hipFree(w->d_bias);
    delete w;
    return 0;
}

extern "C" int nncase_hip_w8a16_prepack(nncase_hip_ctx_t *ctx, const int8_t *w_host, const float *scale_host,
                                        const float *bias_host, int32_t k, int32_t n, nncase_hip_w8a16_t **out) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, w_host && scale_host && out, -EINVAL, "w8a16_prepack: null argument");
    *out = nullptr;
    NNHIP_REQUIRE(ctx, k > 0 && n > 0 && k % 64 == 0 && n % 16 == 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "w8a16_prepack: k = %d must be a multiple of 64 and n = %d a multiple of 16", k, n);
    nncase_hip_w8a16 *w = new (std::nothrow) nncase_hip_w8a16();
    NNHIP_REQUIRE(ctx, w, -ENOMEM, "w8a16_prepack: out of host memory");
    w->k = k, w->n = n, w->ntiles = n / 16, w->ksteps = k / 64;
    const size_t bytes = (size_t)n * k;
    std::vector<int8_t> packed(bytes);
    for (int t = 0; t < w->ntiles; t++)
        for (int ks = 0; ks < w->ksteps; ks++)
            for (int l = 0; l < 64; l++) {
                const int i = l & 15, kg = l >> 4;
                memcpy(&packed[(((size_t)t * w->ksteps + ks) * 64 + l) * 16], w_host + (size_t)(t * 16 + i) * k + ks * 64 + kg * 16, 16);
            }
    auto cleanup = [&](int rc) {
        (void)nncase_hip_w8a16_destroy(ctx, w);
        return rc;
    };
    if (hipMalloc(&w->d_packed, bytes) != hipSuccess || hipMalloc((void **)&w->d_scale, sizeof(float) * n) != hipSuccess)
        return cleanup(fail(ctx, -ENOMEM, "w8a16_prepack: out of device memory"));
    if (bias_host && hipMalloc((void **)&w->d_bias, sizeof(float) * n) != hipSuccess)
        return cleanup(fail(ctx, -ENOMEM, "w8a16_prepack: out of device memory"));
    if (hipMemcpy(w->d_packed, packed.data(), bytes, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(w->d_scale, scale_host, sizeof(float) * n, hipMemcpyHostToDevice) != hipSuccess ||
        (bias_host && hipMemcpy(w->d_bias, bias_host, sizeof(float) * n, hipMemcpyHostToDevice) != hipSuccess))
        return cleanup(fail(ctx, -EFAULT, "w8a16_prepack: upload failed"));
    *out = w;
    return 0;
}

// A launch whose LDS (the dynamic part plus the kernel's own static arrays: `total`) passes 48 KiB asks, once per kernel
// and device, for a dynamic limit of `limit` bytes.
template <typename KernelT> static hipError_t raise_dynamic_lds(KernelT kernel, int device, size_t total, int limit) {
    if (total <= 48 * 1024) return hipSuccess;
    static std::once_flag raised[16];
    hipError_t e = hipSuccess;
    std::call_once(raised[device & 15], [&] { e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, limit); });
    return e;
}

// Whether the q / k / v projection of this geometry can rotate and append in its own epilogue (else the caller runs
// the projection and the rope kernel one after the other).
static bool rope_epilogue_fits(const nncase_hip_w8a16_t *w, int m, const RopeArgs &r) {
    const int mt_built = m <= 16 ? 1 : 2;
    return m <= 32 && r.d % 32 == 0 && w->n == (r.hq + 2 * r.hkv) * r.d && w->k <= kRowsMaxK &&
           (size_t)mt_built * 16 * rows_in_lds_pitch(w->k) <= 64 * 1024 && (w->ksteps + kGemmWaves - 1) / kGemmWaves <= 2;
}

static int launch_w8a16_gemm(nncase_hip_ctx_t *ctx, const void *a_dev, const nncase_hip_w8a16_t *w, void *out_dev, int32_t m,
                             int32_t mode, const void *residual_dev, int32_t out_dtype, const void *ln_weight_dev, float ln_eps,
                             const RopeArgs *rope = nullptr) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, a_dev && w && out_dev, -EINVAL, "w8a16_gemm: null argument");
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(ln_weight_dev) & 15u) == 0, -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION,
                  "w8a16_gemm: normalisation weights must be 16-byte aligned");
    NNHIP_REQUIRE(ctx, m > 0 && m <= kMaxRows, -NNCASE_HIP_ERR_SHAPE_MISMATCH, "w8a16_gemm: %d token rows (1..%d supported)", m, kMaxRows);
    NNHIP_REQUIRE(ctx, mode == NNCASE_HIP_GEMM_PLAIN || mode == NNCASE_HIP_GEMM_SWIGLU, -EINVAL, "w8a16_gemm: unknown mode %d", mode);
    NNHIP_REQUIRE(ctx, out_dtype == NNCASE_HIP_DT_F16 || out_dtype == NNCASE_HIP_DT_F32, -NNCASE_HIP_ERR_DATATYPE_MISMATCH,
                  "w8a16_gemm: output type 0x%x", out_dtype);
    NNHIP_REQUIRE(ctx, mode != NNCASE_HIP_GEMM_SWIGLU || w->ntiles % 2 == 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "w8a16_gemm: SwiGLU needs gate and up halves of equal size");
    NNHIP_REQUIRE(ctx, ((reinterpret_cast<uintptr_t>(a_dev) | reinterpret_cast<uintptr_t>(out_dev)) & 15u) == 0,
                  -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION, "w8a16_gemm: buffers must be 16-byte aligned");
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(residual_dev) & 7u) == 0, -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION,
                  "w8a16_gemm: the residual must be 8-byte aligned");
    GemmArgs a;
    memset(&a, 0, sizeof(a));
    a.a = (const uint16_t *)a_dev;
    a.w = (const lu32x4 *)w->d_packed;
    a.scale = w->d_scale, a.bias = w->d_bias;
    a.residual = (const uint16_t *)residual_dev;
    a.ln_w = (const uint16_t *)ln_weight_dev;
    a.ln_eps = ln_eps;
    a.out = out_dev;
    a.m = m, a.k = w->k, a.ksteps = w->ksteps, a.mode = mode, a.out_f32 = out_dtype == NNCASE_HIP_DT_F32;
    const int out_tiles = mode == NNCASE_HIP_GEMM_SWIGLU ? w->ntiles / 2 : w->ntiles;
    a.up_tile_offset = out_tiles;
    a.n_out = out_tiles * 16;
    // few output tiles: the block's waves split the reduction of one tile; many: a tile per wave
    const bool split = out_tiles < 4 * ctx->compute_units;
    const dim3 grid(split ? out_tiles : (out_tiles + kGemmWaves - 1) / kGemmWaves), block(kGemmThreads);
    const int mt = (m + 15) / 16;
    const bool glu = mode == NNCASE_HIP_GEMM_SWIGLU;
    // a tile per wave with the token rows shared through LDS: where the rows fit and the launch has a tile for every
    // compute unit (measured on the decode step: the 72- and 56-tile products are quicker with the reduction split
    // over a block's waves, 9.7 against 11.2 us; the 304 gate / up tile pairs take 11.4 us in 38 blocks of eight waves
    // with a pair per wave, 10.7 us in 304 blocks of four waves that split a pair's reduction, 12.8 us in blocks of
    // eight.  What the launches cost is not the weights' trip to memory but what every block repeats: the rows' trip,
    // 1.2 us, their normalisation, 0.3 us of vector issue per row and SIMD, and, with a pair per wave, 0.24 us of
    // conversions and matrix instructions per k-step on a SIMD that two waves share)
    const int mt_built = mt <= 1 ? 1 : (mt == 2 ? 2 : 4);
    const size_t rows_lds = (size_t)mt_built * 16 * rows_in_lds_pitch(w->k);
    if (rope) {
        // (the caller has checked rope_epilogue_fits) a block per pair of tiles d / 2 channels apart
        a.rope = *rope;
        a.up_tile_offset = rope->d / 32;
        const dim3 pgrid(w->ntiles / 2), pblock(kGemmThreads);
        const bool two_pieces = w->k <= 1024;
#define NNHIP_ROPE_LAUNCH(MTV, PV)                                                                                             \
    do {                                                                                                                       \
        NNHIP_HIP(ctx, raise_dynamic_lds(w8a16_gemm_rows_in_lds_kernel<MTV, 2, kGemmWaves, true, 2, PV, true>, ctx->device,   \
                                         rows_lds + MTV * 16 * 1024, 96 * 1024));                                              \
        hipLaunchKernelGGL((w8a16_gemm_rows_in_lds_kernel<MTV, 2, kGemmWaves, true, 2, PV, true>), pgrid, pblock, rows_lds, ctx->stream, a); \
    } while (0)
        if (mt_built == 1 && two_pieces) NNHIP_ROPE_LAUNCH(1, 2);
        else if (mt_built == 1) NNHIP_ROPE_LAUNCH(1, kRowsPieces);
        else if (two_pieces) NNHIP_ROPE_LAUNCH(2, 2);
        else NNHIP_ROPE_LAUNCH(2, kRowsPieces);
#undef NNHIP_ROPE_LAUNCH
        NNHIP_LAUNCH_CHECK(ctx, "w8a16_gemm_rows_in_lds_kernel");
        return 0;
    }
    const bool short_rows = w->k <= 1024; // rows of two 512-element pieces (a lane keeps a row's pieces in registers)
    if (split && glu && w->k <= kRowsMaxK && rows_lds <= 64 * 1024 && mt_built <= 2 && // (with or without rows to normalise: one summation order)
        (w->ksteps + kGluSplitWaves - 1) / kGluSplitWaves <= 4) {
        // the gate / up projection of a decode step (a few hundred tile pairs over a short reduction): a block per tile
        // pair, its waves splitting the reduction, so that every compute unit takes part.  Four waves for 32 rows (eight
        // took 12.8 against 10.7 us); eight for 16 rows, where a wave then brings in and normalises two rows instead of
        // four (the decode step of two lanes: 1.097 against 1.114 ms)
#define NNHIP_GLU_SPLIT_LAUNCH(MTV, PV, GWV, KBV)                                                                              \
    do {                                                                                                                       \
        NNHIP_HIP(ctx, raise_dynamic_lds(w8a16_gemm_rows_in_lds_kernel<MTV, 2, GWV, true, KBV, PV>, ctx->device,              \
                                         rows_lds + GWV * 2 * MTV * 1024, 96 * 1024));                                         \
        hipLaunchKernelGGL((w8a16_gemm_rows_in_lds_kernel<MTV, 2, GWV, true, KBV, PV>), grid, dim3(GWV * 64), rows_lds, ctx->stream, a); \
    } while (0)
        const bool two_steps = (w->ksteps + 7) / 8 <= 2; // a wave's share of the reduction with eight waves
        if (mt_built == 1 && short_rows && two_steps) NNHIP_GLU_SPLIT_LAUNCH(1, 2, 8, 2);
        else if (mt_built == 1 && short_rows) NNHIP_GLU_SPLIT_LAUNCH(1, 2, 8, 4);
        else if (mt_built == 1) NNHIP_GLU_SPLIT_LAUNCH(1, kRowsPieces, 8, 4);
        else if (short_rows) NNHIP_GLU_SPLIT_LAUNCH(2, 2, kGluSplitWaves, 4);
        else NNHIP_GLU_SPLIT_LAUNCH(2, kRowsPieces, kGluSplitWaves, 4);
#undef NNHIP_GLU_SPLIT_LAUNCH
        NNHIP_LAUNCH_CHECK(ctx, "w8a16_gemm_rows_in_lds_kernel");
        return 0;
    }
    if (split && !glu && ln_weight_dev && w->k <= kRowsMaxK && rows_lds <= 64 * 1024 && mt_built <= 2) {
        // few tiles and rows to normalise (the q / k / v projection): the reduction split over the block's waves, the
        // rows parked and normalised in LDS in one trip to memory
        // (the kernel's static reduction area comes on top of the rows: past 48 KiB in all, the limit is raised like below)
        // (a wave's share of the reduction is requested at once where it is at most two k-steps, the decode step's case)
        const bool short_share = (w->ksteps + kGemmWaves - 1) / kGemmWaves <= 2;
#define NNHIP_SPLIT_ROWS_LAUNCH_P(MTV, KBV, PV)                                                                                \
    do {                                                                                                                       \
        NNHIP_HIP(ctx, raise_dynamic_lds(w8a16_gemm_rows_in_lds_kernel<MTV, 1, kGemmWaves, true, KBV, PV>, ctx->device,       \
                                         rows_lds + MTV * 8 * 1024, 64 * 1024));                                               \
        hipLaunchKernelGGL((w8a16_gemm_rows_in_lds_kernel<MTV, 1, kGemmWaves, true, KBV, PV>), grid, block, rows_lds, ctx->stream, a); \
    } while (0)
#define NNHIP_SPLIT_ROWS_LAUNCH(MTV, KBV)                                                                                      \
    do {                                                                                                                       \
        if (short_rows) NNHIP_SPLIT_ROWS_LAUNCH_P(MTV, KBV, 2);                                                                \
        else NNHIP_SPLIT_ROWS_LAUNCH_P(MTV, KBV, kRowsPieces);                                                                 \
    } while (0)
        if (mt_built == 1) {
            if (short_share) NNHIP_SPLIT_ROWS_LAUNCH(1, 2);
            else NNHIP_SPLIT_ROWS_LAUNCH(1, kRowsBatch);
        } else {
            if (short_share) NNHIP_SPLIT_ROWS_LAUNCH(2, 2);
            else NNHIP_SPLIT_ROWS_LAUNCH(2, kRowsBatch);
        }
#undef NNHIP_SPLIT_ROWS_LAUNCH
#undef NNHIP_SPLIT_ROWS_LAUNCH_P
        NNHIP_LAUNCH_CHECK(ctx, "w8a16_gemm_rows_in_lds_kernel");
        return 0;
    }
    if (w->k <= kRowsMaxK && rows_lds <= 128 * 1024 && out_tiles >= ctx->compute_units) {
        // (at most two blocks per compute unit, each walking several groups of eight tiles: what a block repeats -- the
        // rows' trip and their normalisation -- is then paid twice per compute unit, not once per group)
        const dim3 rgrid(std::min((out_tiles + kGemmWaves - 1) / kGemmWaves, 2 * ctx->compute_units)), rblock(kGemmThreads);
        // (eight k-steps of weights per request: asking for a whole 14-step reduction at once costs registers that the
        // vocabulary head needs for occupancy -- 50.7 against 43.9 us when it still ran as 1187 one-group blocks)
#define NNHIP_ROWS_LAUNCH_KB(MTV, GV, KBV, PV)                                                                                 \
    do {                                                                                                                       \
        NNHIP_HIP(ctx, raise_dynamic_lds(w8a16_gemm_rows_in_lds_kernel<MTV, GV, kGemmWaves, false, KBV, PV>, ctx->device, rows_lds + 1024, 128 * 1024)); \
        hipLaunchKernelGGL((w8a16_gemm_rows_in_lds_kernel<MTV, GV, kGemmWaves, false, KBV, PV>), rgrid, rblock, rows_lds, ctx->stream, a); \
    } while (0)
#define NNHIP_ROWS_LAUNCH(MTV, GV)                                                                                             \
    do {                                                                                                                       \
        if (short_rows) NNHIP_ROWS_LAUNCH_KB(MTV, GV, kRowsBatch, 2);                                                          \
        else NNHIP_ROWS_LAUNCH_KB(MTV, GV, kRowsBatch, kRowsPieces);                                                           \
    } while (0)
        if (glu) {
            if (mt_built == 1) NNHIP_ROWS_LAUNCH(1, 2);
            else if (mt_built == 2) NNHIP_ROWS_LAUNCH(2, 2);
            else NNHIP_ROWS_LAUNCH(4, 2);
        } else {
            if (mt_built == 1) NNHIP_ROWS_LAUNCH(1, 1);
            else if (mt_built == 2) NNHIP_ROWS_LAUNCH(2, 1);
            else NNHIP_ROWS_LAUNCH(4, 1);
        }
#undef NNHIP_ROWS_LAUNCH_KB
#undef NNHIP_ROWS_LAUNCH
        NNHIP_LAUNCH_CHECK(ctx, "w8a16_gemm_rows_in_lds_kernel");
        return 0;
    }
    // a share of 9 or 10 k-steps per wave (the 4864-deep down projection): one request of all ten for up to 16 token rows,
    // two of five for up to 32 (whose slices of ten k-steps do not fit the registers), instead of 4 + 4 + 2
    const int share = (w->ksteps + kGemmWaves - 1) / kGemmWaves;
    const bool long_share = !ln_weight_dev && mt <= 2 && (share == 9 || share == 10);
#define NNHIP_GEMM_LAUNCH(MTV)                                                                                                 \
    do {                                                                                                                       \
        if (glu && split) hipLaunchKernelGGL((w8a16_gemm_kernel<MTV, 2, true>), grid, block, 0, ctx->stream, a);              \
        else if (glu) hipLaunchKernelGGL((w8a16_gemm_kernel<MTV, 2, false>), grid, block, 0, ctx->stream, a);                 \
        else if (split && long_share) hipLaunchKernelGGL((w8a16_gemm_kernel<(MTV <= 2 ? MTV : 2), 1, true, (MTV == 1 ? 10 : 5)>), grid, block, 0, ctx->stream, a); \
        else if (split) hipLaunchKernelGGL((w8a16_gemm_kernel<MTV, 1, true>), grid, block, 0, ctx->stream, a);                \
        else hipLaunchKernelGGL((w8a16_gemm_kernel<MTV, 1, false>), grid, block, 0, ctx->stream, a);                          \
    } while (0)
    if (mt == 1) NNHIP_GEMM_LAUNCH(1);
    else if (mt == 2) NNHIP_GEMM_LAUNCH(2);
    else NNHIP_GEMM_LAUNCH(4);
#undef NNHIP_GEMM_LAUNCH
    NNHIP_LAUNCH_CHECK(ctx, "w8a16_gemm_kernel");
    return 0;
}

extern "C" int nncase_hip_w8a16_gemm(nncase_hip_ctx_t *ctx, const void *a_dev, const nncase_hip_w8a16_t *w, void *out_dev,
                                     int32_t m, int32_t mode, const void *residual_dev, int32_t out_dtype) {
    return launch_w8a16_gemm(ctx, a_dev, w, out_dev, m, mode, residual_dev, out_dtype, nullptr, 0.f);
}

extern "C" int nncase_hip_rmsnorm_w8a16_gemm(nncase_hip_ctx_t *ctx, const void *x_dev, const void *ln_weight_dev, float eps,
                                             const nncase_hip_w8a16_t *w, void *out_dev, int32_t m, int32_t mode,
                                             const void *residual_dev, int32_t out_dtype) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, ln_weight_dev, -EINVAL, "rmsnorm_w8a16_gemm: null normalisation weights");
    return launch_w8a16_gemm(ctx, x_dev, w, out_dev, m, mode, residual_dev, out_dtype, ln_weight_dev, eps);
}

extern "C" int nncase_hip_rmsnorm_f16(nncase_hip_ctx_t *ctx, const void *x_dev, const void *weight_dev, void *out_dev, int32_t rows,
                                      int32_t hidden, float eps) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && weight_dev && out_dev && rows > 0 && hidden > 0, -EINVAL, "rmsnorm_f16: bad argument");
    hipLaunchKernelGGL(rmsnorm_f16_kernel, dim3((rows + 3) / 4), dim3(kLlmThreads), 0, ctx->stream, (const __half *)x_dev,
                       (const __half *)weight_dev, (__half *)out_dev, rows, hidden, eps);
    NNHIP_LAUNCH_CHECK(ctx, "rmsnorm_f16_kernel");
    return 0;
}

static int make_rope_args(nncase_hip_ctx_t *ctx, const void *qkv_dev, void *q_out_dev, void *k_cache_dev, void *v_cache_dev,
                          const int32_t *block_table_dev, const int32_t *ctx_lens_dev, const nncase_hip_paged_attn_args_t *p,
                          float rope_theta, RopeArgs *out) {
    NNHIP_REQUIRE(ctx, q_out_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && p, -EINVAL,
                  "rope_kv_append: null argument");
    NNHIP_REQUIRE(ctx, p->batch > 0 && p->num_q_heads > 0 && p->num_kv_heads > 0 && p->head_dim > 0 && p->head_dim % 2 == 0 &&
                           p->block_size > 0 && p->max_blocks_per_seq > 0 && p->num_blocks > 0 && rope_theta > 0.f,
                  -EINVAL, "rope_kv_append: bad geometry");
    RopeArgs &a = *out;
    a.qkv = (const __half *)qkv_dev, a.q_out = (__half *)q_out_dev, a.k_cache = (__half *)k_cache_dev, a.v_cache = (__half *)v_cache_dev;
    a.block_table = block_table_dev, a.ctx_lens = ctx_lens_dev;
    a.batch = p->batch, a.hq = p->num_q_heads, a.hkv = p->num_kv_heads, a.d = p->head_dim, a.block_size = p->block_size;
    a.max_blocks = p->max_blocks_per_seq, a.num_blocks = p->num_blocks, a.theta = rope_theta;
    return 0;
}

extern "C" int nncase_hip_rope_kv_append(nncase_hip_ctx_t *ctx, const void *qkv_dev, void *q_out_dev, void *k_cache_dev,
                                         void *v_cache_dev, const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                         const nncase_hip_paged_attn_args_t *p, float rope_theta) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, qkv_dev, -EINVAL, "rope_kv_append: null argument");
    RopeArgs a;
    const int rc = make_rope_args(ctx, qkv_dev, q_out_dev, k_cache_dev, v_cache_dev, block_table_dev, ctx_lens_dev, p, rope_theta, &a);
    if (rc) return rc;
    const int64_t total = (int64_t)a.batch * (a.hq + 2 * a.hkv) * (a.d / 2);
    NNHIP_REQUIRE(ctx, total < ((int64_t)1 << 31), -EINVAL, "rope_kv_append: too large");
    hipLaunchKernelGGL(rope_append_kernel, dim3((unsigned)((total + kLlmThreads - 1) / kLlmThreads)), dim3(kLlmThreads), 0, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "rope_append_kernel");
    return 0;
}

extern "C" int nncase_hip_w8a16_gemm_rope_kv_append(nncase_hip_ctx_t *ctx, const void *x_dev, const void *ln_weight_dev, float eps,
                                                    const nncase_hip_w8a16_t *w, void *qkv_dev, void *q_out_dev, void *k_cache_dev,
                                                    void *v_cache_dev, const int32_t *block_table_dev, const int32_t *ctx_lens_dev,
                                                    const nncase_hip_paged_attn_args_t *p, float rope_theta) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && w && qkv_dev, -EINVAL, "w8a16_gemm_rope_kv_append: null argument");
    RopeArgs r;
    int rc = make_rope_args(ctx, qkv_dev, q_out_dev, k_cache_dev, v_cache_dev, block_table_dev, ctx_lens_dev, p, rope_theta, &r);
    if (rc) return rc;
    NNHIP_REQUIRE(ctx, w->n == (r.hq + 2 * r.hkv) * r.d, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "w8a16_gemm_rope_kv_append: the matrix has %d output channels, the heads need %d", w->n, (r.hq + 2 * r.hkv) * r.d);
    if (rope_epilogue_fits(w, r.batch, r))
        return launch_w8a16_gemm(ctx, x_dev, w, qkv_dev, r.batch, NNCASE_HIP_GEMM_PLAIN, nullptr, NNCASE_HIP_DT_F16, ln_weight_dev, eps, &r);
    // other geometries: the projection into qkv_dev, then the rope kernel (the same values: the epilogue above rounds to
    // fp16 where this path stores fp16)
    rc = launch_w8a16_gemm(ctx, x_dev, w, qkv_dev, r.batch, NNCASE_HIP_GEMM_PLAIN, nullptr, NNCASE_HIP_DT_F16, ln_weight_dev, eps);
    if (rc) return rc;
    return nncase_hip_rope_kv_append(ctx, qkv_dev, q_out_dev, k_cache_dev, v_cache_dev, block_table_dev, ctx_lens_dev, p, rope_theta);
}

extern "C" int nncase_hip_argmax_f32(nncase_hip_ctx_t *ctx, const float *x_dev, int32_t *out_dev, int32_t rows, int32_t cols) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && out_dev && rows > 0 && cols > 0, -EINVAL, "argmax_f32: bad argument");
    hipLaunchKernelGGL(argmax_f32_kernel, dim3(rows), dim3(kArgmaxThreads), 0, ctx->stream, x_dev, out_dev, cols);
    NNHIP_LAUNCH_CHECK(ctx, "argmax_f32_kernel");
    return 0;
}

extern "C" int nncase_hip_embedding_f16(nncase_hip_ctx_t *ctx, const void *table_dev, const int32_t *ids_dev, void *out_dev,
                                        int32_t rows, int32_t hidden, int32_t vocab) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, table_dev && ids_dev && out_dev && rows > 0 && hidden > 0 && vocab > 0, -EINVAL, "embedding_f16: bad argument");
    const int64_t total = (int64_t)rows * hidden;
    NNHIP_REQUIRE(ctx, total < ((int64_t)1 << 31), -EINVAL, "embedding_f16: too large");
    hipLaunchKernelGGL(embed_f16_kernel, dim3((unsigned)((total + kLlmThreads - 1) / kLlmThreads)), dim3(kLlmThreads), 0, ctx->stream,
                       (const __half *)table_dev, ids_dev, (__half *)out_dev, rows, hidden, vocab);
    NNHIP_LAUNCH_CHECK(ctx, "embed_f16_kernel");
    return 0;
}

extern "C" int nncase_hip_add_i32(nncase_hip_ctx_t *ctx, int32_t *x_dev, int32_t count, int32_t delta) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && count > 0, -EINVAL, "add_i32: bad argument");
    hipLaunchKernelGGL(add_i32_kernel, dim3((count + 255) / 256), dim3(256), 0, ctx->stream, x_dev, count, delta);
    NNHIP_LAUNCH_CHECK(ctx, "add_i32_kernel");
    return 0;
}
