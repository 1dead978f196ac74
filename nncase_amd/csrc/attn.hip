// Paged-attention decode: one query token per sequence against a block-paged
// fp16 KV cache.  HBM-bound (every cached K and V element is read once per
// step, ~7 flop per byte), so the kernel is organised around the KV stream:
//
//   grid = (splits, kv heads, sequences).  A block owns one kv head of one
//   sequence and a contiguous range of `kSplitTokens` cached tokens, and
//   serves ALL query heads that share the kv head, so K and V cross the memory
//   system once however many query heads there are (GQA).
//   A wave reads a run of tokens as one contiguous, fully coalesced segment
//   (each lane 32 bytes = 16 fp16 of one token), i.e. physical KV blocks are
//   consumed whole in the order the block table lists them.
//   Pass 1 writes scaled logits to LDS, the block takes the max and the
//   exponentials there, pass 2 accumulates P.V in fp32 registers; partial
//   (max, sum, unnormalised output) triples go to a workspace and a second
//   kernel merges the splits.
#include "common.hpp"

#include <hip/hip_fp16.h>

namespace nnhip {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = 4;
constexpr int kSplitTokens = 512;
constexpr int kMaxGroup = 8; // query heads per kv head

struct AttnArgs {
    const uint16_t *q, *k_cache, *v_cache;
    const int32_t *block_table, *ctx_lens;
    float *part_o; // [batch][q heads][splits][D]
    float *part_ml; // [batch][q heads][splits][2]
    void *out;
    int batch, hq, hkv, group, d, block_size, max_blocks, num_blocks, splits;
    float scale;
    int out_f16;
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// D = head_dim (64 or 128).  LPT lanes share one token (16 fp16 each).
template <int D> __global__ __launch_bounds__(kAttnThreads) void paged_attn_split_kernel(const AttnArgs a) {
    constexpr int LPT = D / 16;   // lanes per token
    constexpr int TPW = 64 / LPT; // tokens per wave step
    __shared__ float sc[kMaxGroup][kSplitTokens]; // logits, then probabilities
    __shared__ float red[kAttnWaves][kMaxGroup][D];
    __shared__ float hmax[kMaxGroup], hsum[kMaxGroup];

    const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int ctx = min(a.ctx_lens[b], a.max_blocks * a.block_size);
    const int tok0 = split * kSplitTokens;
    if (tok0 >= ctx) return; // uniform for the block
    const int ntok = min(kSplitTokens, ctx - tok0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int lt = lane / LPT;  // token within the wave step
    const int dq = lane % LPT;  // which 16-element slice of the head
    const int G = a.group;

    // this lane's slice of every query head of the group
    half2_t qv[kMaxGroup][8];
#pragma unroll
    for (int h = 0; h < kMaxGroup; h++) {
        if (h < G) {
            const uint4 *src =
                reinterpret_cast<const uint4 *>(a.q + ((size_t)b * a.hq + kvh * G + h) * D + dq * 16);
            const uint4 lo = src[0], hi = src[1];
            __builtin_memcpy(&qv[h][0], &lo, 16);
            __builtin_memcpy(&qv[h][4], &hi, 16);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) qv[h][i] = half2_t{0, 0};
        }
    }
    const int32_t *table = a.block_table + (size_t)b * a.max_blocks;
    const int steps = (ntok + TPW - 1) / TPW;

    // ---- pass 1: logits ----------------------------------------------------
    for (int st = wave; st < steps; st += kAttnWaves) {
        const int tl = st * TPW + lt; // token within the split
        float s[kMaxGroup];
#pragma unroll
        for (int h = 0; h < kMaxGroup; h++) s[h] = 0.f;
        if (tl < ntok) {
            const int tok = tok0 + tl;
            // a block id outside the cache would fault; read block 0 instead (undefined result, no fault)
            const int pb = min(max(table[tok / a.block_size], 0), a.num_blocks - 1);
            const uint16_t *kp =
                a.k_cache + (((size_t)pb * a.hkv + kvh) * a.block_size + tok % a.block_size) * D + dq * 16;
            const uint4 lo = reinterpret_cast<const uint4 *>(kp)[0], hi = reinterpret_cast<const uint4 *>(kp)[1];
            half2_t kv[8];
            __builtin_memcpy(&kv[0], &lo, 16);
            __builtin_memcpy(&kv[4], &hi, 16);
#pragma unroll
            for (int h = 0; h < kMaxGroup; h++)
                if (h < G) {
#pragma unroll
                    for (int i = 0; i < 8; i++) s[h] = __builtin_amdgcn_fdot2(qv[h][i], kv[i], s[h], false);
                }
        }
#pragma unroll
        for (int h = 0; h < kMaxGroup; h++)
            if (h < G) {
                float v = s[h];
#pragma unroll
                for (int o = 1; o < LPT; o <<= 1) v += __shfl_xor(v, o);
                if (dq == 0) sc[h][st * TPW + lt] = (tl < ntok) ? v * a.scale : -INFINITY;
            }
    }
    __syncthreads();

    // ---- softmax statistics over the split ---------------------------------
    const int padded = steps * TPW;
    for (int h = wave; h < G; h += kAttnWaves) {
        float m = -INFINITY;
        for (int i = lane; i < padded; i += 64) m = fmaxf(m, sc[h][i]);
        m = wave_max(m);
        float l = 0.f;
        for (int i = lane; i < padded; i += 64) {
            const float p = __expf(sc[h][i] - m);
            sc[h][i] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) {
            hmax[h] = m;
            hsum[h] = l;
        }
    }
    __syncthreads();

    // ---- pass 2: P.V ----------------------------------------------------------
    float o[kMaxGroup][16];
#pragma unroll
    for (int h = 0; h < kMaxGroup; h++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[h][i] = 0.f;
    for (int st = wave; st < steps; st += kAttnWaves) {
        const int tl = st * TPW + lt;
        if (tl < ntok) {
            const int tok = tok0 + tl;
            const int pb = min(max(table[tok / a.block_size], 0), a.num_blocks - 1);
            const uint16_t *vp =
                a.v_cache + (((size_t)pb * a.hkv + kvh) * a.block_size + tok % a.block_size) * D + dq * 16;
            const uint4 lo = reinterpret_cast<const uint4 *>(vp)[0], hi = reinterpret_cast<const uint4 *>(vp)[1];
            _Float16 vv[16];
            __builtin_memcpy(&vv[0], &lo, 16);
            __builtin_memcpy(&vv[8], &hi, 16);
#pragma unroll
            for (int h = 0; h < kMaxGroup; h++)
                if (h < G) {
                    const float p = sc[h][tl];
#pragma unroll
                    for (int i = 0; i < 16; i++) o[h][i] += p * (float)vv[i];
                }
        }
    }
    // sum over the lanes that hold different tokens of the same slice, then over waves
#pragma unroll
    for (int h = 0; h < kMaxGroup; h++)
        if (h < G) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float v = o[h][i];
#pragma unroll
                for (int off = LPT; off < 64; off <<= 1) v += __shfl_xor(v, off);
                o[h][i] = v;
            }
            if (lt == 0) {
#pragma unroll
                for (int i = 0; i < 16; i++) red[wave][h][dq * 16 + i] = o[h][i];
            }
        }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * D; idx += kAttnThreads) {
        const int h = idx / D, e = idx % D;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) v += red[w][h][e];
        const size_t row = ((size_t)b * a.hq + kvh * G + h) * a.splits + split;
        a.part_o[row * D + e] = v;
        if (e == 0) {
            a.part_ml[row * 2 + 0] = hmax[h];
            a.part_ml[row * 2 + 1] = hsum[h];
        }
    }
}

// Merges the per-split partials of one (sequence, query head).
__global__ void paged_attn_merge_kernel(const AttnArgs a) {
    const int h = blockIdx.x, b = blockIdx.y, e = threadIdx.x; // blockDim.x == D
    const int ctx = min(a.ctx_lens[b], a.max_blocks * a.block_size);
    const int ns = (ctx + kSplitTokens - 1) / kSplitTokens;
    const size_t row0 = ((size_t)b * a.hq + h) * a.splits;
    float m = -INFINITY;
    for (int s = 0; s < ns; s++) m = fmaxf(m, a.part_ml[(row0 + s) * 2]);
    float num = 0.f, den = 0.f;
    for (int s = 0; s < ns; s++) {
        const float w = __expf(a.part_ml[(row0 + s) * 2] - m);
        num += w * a.part_o[(row0 + s) * a.d + e];
        den += w * a.part_ml[(row0 + s) * 2 + 1];
    }
    const float r = ns > 0 ? num / den : 0.f;
    const size_t oi = ((size_t)b * a.hq + h) * a.d + e;
    if (a.out_f16) reinterpret_cast<__half *>(a.out)[oi] = __float2half_rn(r);
    else reinterpret_cast<float *>(a.out)[oi] = r;
}

} // namespace nnhip

using namespace nnhip;

struct AttnWorkspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};
// One workspace per device, grown on demand and kept until the process ends.
static AttnWorkspace g_attn_ws[16];

extern "C" int nncase_hip_paged_attention_decode(nncase_hip_ctx_t *ctx, const void *q_dev, const void *k_cache_dev,
                                                 const void *v_cache_dev, const int32_t *block_table_dev,
                                                 const int32_t *ctx_lens_dev, void *out_dev,
                                                 const nncase_hip_paged_attn_args_t *p) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, q_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && out_dev && p, -EINVAL,
                  "paged_attention_decode: null argument");
    NNHIP_REQUIRE(ctx, p->batch > 0 && p->num_q_heads > 0 && p->num_kv_heads > 0 && p->max_blocks_per_seq > 0 &&
                           p->num_blocks > 0,
                  -EINVAL, "paged_attention_decode: non-positive dimension");
    NNHIP_REQUIRE(ctx, p->head_dim == 64 || p->head_dim == 128, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "paged_attention_decode: head_dim %d (64 or 128 supported)", p->head_dim);
    NNHIP_REQUIRE(ctx, p->num_q_heads % p->num_kv_heads == 0 && p->num_q_heads / p->num_kv_heads <= kMaxGroup,
                  -NNCASE_HIP_ERR_SHAPE_MISMATCH, "paged_attention_decode: %d query heads per kv head unsupported (max %d)",
                  p->num_q_heads / p->num_kv_heads, kMaxGroup);
    const int tpw = 64 / (p->head_dim / 16);
    NNHIP_REQUIRE(ctx, p->block_size > 0 && p->block_size % tpw == 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "paged_attention_decode: block_size %d must be a multiple of %d", p->block_size, tpw);
    NNHIP_REQUIRE(ctx, p->out_dtype == NNCASE_HIP_DT_F16 || p->out_dtype == NNCASE_HIP_DT_F32,
                  -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "paged_attention_decode: output type 0x%x", p->out_dtype);
    NNHIP_REQUIRE(ctx, p->batch <= 65535 && p->num_kv_heads <= 65535, -EINVAL, "paged_attention_decode: grid too large");
    NNHIP_REQUIRE(ctx, ctx->device >= 0 && ctx->device < 16, -EINVAL, "paged_attention_decode: device index");

    AttnArgs a;
    memset(&a, 0, sizeof(a));
    a.q = (const uint16_t *)q_dev;
    a.k_cache = (const uint16_t *)k_cache_dev;
    a.v_cache = (const uint16_t *)v_cache_dev;
    a.block_table = block_table_dev;
    a.ctx_lens = ctx_lens_dev;
    a.out = out_dev;
    a.batch = p->batch;
    a.hq = p->num_q_heads;
    a.hkv = p->num_kv_heads;
    a.group = p->num_q_heads / p->num_kv_heads;
    a.d = p->head_dim;
    a.block_size = p->block_size;
    a.max_blocks = p->max_blocks_per_seq;
    a.num_blocks = p->num_blocks;
    const int64_t max_tokens = (int64_t)p->max_blocks_per_seq * p->block_size;
    a.splits = (int)((max_tokens + kSplitTokens - 1) / kSplitTokens);
    a.scale = p->scale;
    a.out_f16 = p->out_dtype == NNCASE_HIP_DT_F16;

    const size_t rows = (size_t)a.batch * a.hq * a.splits;
    const size_t need = rows * (a.d + 2) * sizeof(float);
    AttnWorkspace &ws = g_attn_ws[ctx->device];
    if (ws.bytes < need) {
        NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
        if (ws.ptr) NNHIP_HIP(ctx, hipFree(ws.ptr));
        ws.ptr = nullptr;
        ws.bytes = 0;
        NNHIP_HIP(ctx, hipMalloc(&ws.ptr, need));
        ws.bytes = need;
    }
    a.part_o = reinterpret_cast<float *>(ws.ptr);
    a.part_ml = a.part_o + rows * a.d;

    const dim3 grid(a.splits, a.hkv, a.batch);
    if (a.d == 64) hipLaunchKernelGGL(paged_attn_split_kernel<64>, grid, dim3(kAttnThreads), 0, ctx->stream, a);
    else hipLaunchKernelGGL(paged_attn_split_kernel<128>, grid, dim3(kAttnThreads), 0, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "paged_attn_split_kernel");
    hipLaunchKernelGGL(paged_attn_merge_kernel, dim3(a.hq, a.batch), dim3(a.d), 0, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "paged_attn_merge_kernel");
    return 0;
}
