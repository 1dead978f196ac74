// Paged-attention decode: one query token per sequence against a block-paged
// fp16 KV cache.  HBM-bound (every cached K and V element is read once per
// step, ~7 flop per byte), so the kernel is organised around the KV stream and
// keeps the arithmetic on the matrix cores:
//
//   grid = (sequences x kv heads, splits).  A block owns one kv head of one
//   sequence and a contiguous range of cached tokens, and serves ALL query
//   heads that share the kv head, so K and V cross the memory system once
//   however many query heads there are (GQA).  Each of its eight waves owns a
//   contiguous run of 16-token tiles and issues the loads of ALL its K and V
//   tiles before any arithmetic (8 KiB of K + 8 KiB of V in flight per wave).
//
//   Logits: S^T[token, head] = K[token, :] . Q^T[:, head] with K rows as the
//   MFMA A operand (one 16-byte load per lane straight from the cache) and the
//   query heads, padded to 16, as B.  The accumulator layout of S^T (lane =
//   head, 4 consecutive tokens per lane) IS the A-operand layout of the 16x16x16
//   product P.V, so probabilities never move between lanes.  V is cached
//   d-major ([block][kv head][d][token]) so that a lane's B operand (4
//   consecutive tokens of one d) is one 8-byte load.  P is split into two fp16
//   terms (p = hi + lo), which keeps the P.V product at fp32-level accuracy.
//
//   Every wave keeps its own (max, sum, unnormalised output); the block merges
//   its waves through LDS and writes one partial per split.  The block
//   that finishes last for a (sequence, kv head) - found with one atomic
//   counter per pair, which it resets for the next call - merges the splits
//   and writes the output, so there is a single launch per call.
#include "common.hpp"

#include <hip/hip_fp16.h>

namespace nnhip {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t au32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t au32x2 __attribute__((ext_vector_type(2)));

constexpr int kAttnHeads = 16; // query heads per kv head, padded to the MFMA tile
constexpr float kLog2e = 1.4426950408889634f;

constexpr int kAttnMaxSplits = 1024; // splits of one sequence (bounds the merge loop and the workspace)

struct AttnArgs {
    const uint16_t *q, *k_cache, *v_cache;
    const int32_t *block_table, *ctx_lens;
    float *part_o;  // [batch][q heads][splits][D], unnormalised, relative to the split's max
    float *part_ml; // [batch][q heads][splits][2]: max of (logit * scale * log2 e), sum of 2^(. - max)
    uint32_t *done; // [batch][kv heads] blocks finished; zero between calls
    void *out;
    int batch, hq, hkv, group, d, block_size, max_blocks, num_blocks, splits, split_tokens, len_offset;
    FastDiv d_block;
    float scale_log2e;
    int out_f16;
};

__device__ __forceinline__ void coherent_store(float *p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// bytes of dynamic LDS of a block of W waves: the waves' unnormalised outputs, maxima and sums
constexpr size_t attn_lds_bytes(int d, int waves) { return (size_t)waves * kAttnHeads * (d + 2) * sizeof(float); }

// NT = 16-token tiles per wave (even); W = waves per block (a block owns W * NT * 16 tokens).
template <int D, int NT, int W> __global__ __launch_bounds__(W * 64, W <= 8 ? 2 : 1) void paged_attn_kernel(const AttnArgs a) {
    constexpr int kAttnWaves = W, kAttnThreads = W * 64;
    constexpr int KS = D / 32; // 32-deep steps of the logit product
    constexpr int DT = D / 16; // 16-wide column tiles of the output
    constexpr int WAVE_TOKENS = NT * 16;
    constexpr int SPLIT = kAttnWaves * WAVE_TOKENS;
    extern __shared__ __align__(16) float attn_smem[];
    float(*red)[kAttnHeads][D] = reinterpret_cast<float(*)[kAttnHeads][D]>(attn_smem);                            // [W][heads][D]
    float(*smax)[kAttnHeads] = reinterpret_cast<float(*)[kAttnHeads]>(attn_smem + (size_t)W * kAttnHeads * D);    // [W][heads]
    float(*ssum)[kAttnHeads] = smax + W;                                                                            // [W][heads]
    __shared__ uint32_t s_last;

    // kv head fastest, then sequence, then split: consecutive workgroups go to different XCDs, so
    // every XCD gets the same mix of early (always present) and late (long contexts only) splits
    const int kvh = blockIdx.x % a.hkv, b = blockIdx.x / a.hkv, split = blockIdx.y;
    const int tok0 = split * SPLIT;
    const int G = a.group;
    const int lane = threadIdx.x & 63;
    // the wave index as a scalar, so that everything derived from it (tile positions, block-table
    // lookups, cache base addresses) stays on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 15, g = lane >> 4;
    const int wave_tok0 = tok0 + wave * WAVE_TOKENS;
    // The block-table entries of this wave's tiles do not depend on the context length, so they
    // are fetched together with it (one scalar-memory round trip instead of two).  A tile past
    // the end of the context may get any entry of the table; its block id is clamped into the
    // cache, its logits are masked and its V operand is zeroed.
    const int32_t *table = a.block_table + (size_t)b * a.max_blocks;
    int pbs[NT], inb[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int tt = wave_tok0 + t * 16;
        const uint32_t lb = fastdiv((uint32_t)tt, a.d_block);
        inb[t] = tt - (int)lb * a.block_size;
        pbs[t] = table[min((int)lb, a.max_blocks - 1)];
    }
    const int ctx = min(a.ctx_lens[b] + a.len_offset, a.max_blocks * a.block_size);
    if (ctx <= 0) { // empty context: zeros, written by the first block of the pair
        if (split == 0)
            for (int idx = threadIdx.x; idx < G * D; idx += kAttnThreads) {
                const size_t oi = ((size_t)b * a.hq + kvh * G) * D + idx;
                if (a.out_f16) reinterpret_cast<__half *>(a.out)[oi] = __float2half_rn(0.f);
                else reinterpret_cast<float *>(a.out)[oi] = 0.f;
            }
        return;
    }
    if (tok0 >= ctx) return; // uniform for the block
    const int ns = (ctx + SPLIT - 1) / SPLIT; // blocks of this (sequence, kv head) that get here

    float m_w = -INFINITY, l_w = 0.f;
    f32x4 o[DT];
#pragma unroll
    for (int dt = 0; dt < DT; dt++) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (wave_tok0 < ctx) { // uniform for the wave
        // ---- issue every load of this wave ----------------------------------------------
        // Every K and V load back to back (the block-table entries are already here: a lookup
        // between two tiles' loads would wait for the earlier tile's data as well).
        au32x4 kf[NT][KS];
        au32x2 vf[NT][DT];
        const uint32_t koff = (uint32_t)(j * D + g * 8) * 2u;            // bytes, the same for every tile
        const uint32_t voff = (uint32_t)(j * a.block_size + g * 4) * 2u;
        const size_t vstep = (size_t)a.block_size * 32;                  // 16 rows of d
#pragma unroll
        for (int t = 0; t < NT; t++) {
            // a block id outside the cache would fault; read block 0 instead (undefined result, no fault)
            const int pb = min(max(pbs[t], 0), a.num_blocks - 1);
            const size_t head_base = ((size_t)pb * a.hkv + kvh) * (size_t)a.block_size * D;
            const char *kb = reinterpret_cast<const char *>(a.k_cache) + (head_base + (size_t)inb[t] * D) * 2;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) kf[t][ks] = *reinterpret_cast<const au32x4 *>(kb + ks * 64 + koff);
            const char *vb = reinterpret_cast<const char *>(a.v_cache) + (head_base + (size_t)inb[t]) * 2;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) vf[t][dt] = *reinterpret_cast<const au32x2 *>(vb + dt * vstep + voff);
        }
        // query heads of the group as the B operand (columns past the group are zero)
        f16x8 qf[KS];
        {
            const uint16_t *qp = a.q + ((size_t)b * a.hq + kvh * G + min(j, G - 1)) * D + g * 8;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                au32x4 raw = *reinterpret_cast<const au32x4 *>(qp + ks * 32);
                if (j >= G) raw = au32x4{0u, 0u, 0u, 0u};
                __builtin_memcpy(&qf[ks], &raw, 16);
            }
        }

        // keep every load above the arithmetic (the scheduler would otherwise sink the V loads
        // below the logit products to save registers, exposing a second memory round trip)
        __builtin_amdgcn_sched_barrier(0);

        // ---- logits, scaled to base-2 exponents -------------------------------------------
        float s[NT][4];
        float m_lane = -INFINITY;
#pragma unroll
        for (int t = 0; t < NT; t++) {
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                f16x8 kk;
                __builtin_memcpy(&kk, &kf[t][ks], 16);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kk, qf[ks], acc, 0, 0, 0);
            }
            const int left = ctx - (wave_tok0 + t * 16 + g * 4); // valid tokens among this lane's four
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float v = acc[r] * a.scale_log2e;
                s[t][r] = r < left ? v : -INFINITY;
                m_lane = fmaxf(m_lane, s[t][r]);
            }
        }
        m_w = fmaxf(m_lane, __shfl_xor(m_lane, 16));
        m_w = fmaxf(m_w, __shfl_xor(m_w, 32)); // finite: the wave's first token is valid for every head

        // ---- probabilities and P.V, two token tiles per 16x16x32 product ----------------------
        float l_lane = 0.f;
#pragma unroll
        for (int t = 0; t < NT; t += 2) {
            f16x8 ph, pl;
            uint32_t keep[2][2];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int left = ctx - (wave_tok0 + (t + u) * 16 + g * 4);
                keep[u][0] = (left > 0 ? 0x0000ffffu : 0u) | (left > 1 ? 0xffff0000u : 0u);
                keep[u][1] = (left > 2 ? 0x0000ffffu : 0u) | (left > 3 ? 0xffff0000u : 0u);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float p = __builtin_amdgcn_exp2f(s[t + u][r] - m_w);
                    l_lane += p;
                    const _Float16 hi = (_Float16)p;
                    ph[u * 4 + r] = hi;
                    pl[u * 4 + r] = (_Float16)(p - (float)hi);
                }
            }
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                // k slot (g, e): token 4g + e of tile t for e < 4, of tile t+1 otherwise - the same in both operands
                const au32x4 raw = au32x4{vf[t][dt].x & keep[0][0], vf[t][dt].y & keep[0][1],
                                          vf[t + 1][dt].x & keep[1][0], vf[t + 1][dt].y & keep[1][1]};
                f16x8 vv;
                __builtin_memcpy(&vv, &raw, 16);
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ph, vv, o[dt], 0, 0, 0);
                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pl, vv, o[dt], 0, 0, 0);
            }
        }
        l_w = l_lane + __shfl_xor(l_lane, 16);
        l_w += __shfl_xor(l_w, 32);
    }

    // ---- merge the waves ----------------------------------------------------------------
    if (g == 0) {
        smax[wave][j] = m_w;
        ssum[wave][j] = l_w;
    }
    __syncthreads();
    // o[dt][r] belongs to head 4g + r, column dt*16 + j
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int h = g * 4 + r;
        float m = smax[0][h];
#pragma unroll
        for (int w = 1; w < kAttnWaves; w++) m = fmaxf(m, smax[w][h]);
        const float f = __builtin_amdgcn_exp2f(smax[wave][h] - m); // 0 for a wave without tokens
#pragma unroll
        for (int dt = 0; dt < DT; dt++) red[wave][h][dt * 16 + j] = o[dt][r] * f;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < G * D; idx += kAttnThreads) {
        const int h = idx / D, e = idx % D;
        float v = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) v += red[w][h][e];
        float m = smax[0][h];
#pragma unroll
        for (int w = 1; w < kAttnWaves; w++) m = fmaxf(m, smax[w][h]);
        float l = 0.f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; w++) l += ssum[w][h] * __builtin_amdgcn_exp2f(smax[w][h] - m);
        if (ns == 1) { // the whole context was in this block
            const float r = v / l;
            const size_t oi = ((size_t)b * a.hq + kvh * G + h) * D + e;
            if (a.out_f16) reinterpret_cast<__half *>(a.out)[oi] = __float2half_rn(r);
            else reinterpret_cast<float *>(a.out)[oi] = r;
        } else {
            const size_t row = ((size_t)b * a.hq + kvh * G + h) * a.splits + split;
            coherent_store(a.part_o + row * D + e, v);
            if (e == 0) {
                coherent_store(a.part_ml + row * 2 + 0, m);
                coherent_store(a.part_ml + row * 2 + 1, l);
            }
        }
    }
    if (ns == 1) return;

    // ---- the last block of the (sequence, kv head) to finish merges the splits -------------------
    // The partials are written and read with device-scope accesses, which go through to the
    // memory side instead of staying in the L2 of the XCD that issued them; waiting for this
    // thread's stores and then for the block makes them globally visible before the count.
    // (A device-scope fence would do the same by writing back and invalidating the whole L2,
    // once per block - an order of magnitude slower here.)
    uint32_t *done = a.done + (size_t)b * a.hkv + kvh;
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0)
        s_last = __hip_atomic_fetch_add(done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (uint32_t)(ns - 1);
    __syncthreads();
    if (!s_last) return;
    // Each thread merges one output element: the (max, sum, value) triples of eight splits are
    // requested together (one memory round trip per eight splits), and groups of eight are
    // combined with a running maximum.
    for (int idx = threadIdx.x; idx < G * D; idx += kAttnThreads) {
        const int h = idx / D, e = idx % D;
        const size_t row0 = ((size_t)b * a.hq + kvh * G + h) * a.splits;
        float m = -INFINITY, num = 0.f, den = 0.f;
        for (int sp0 = 0; sp0 < ns; sp0 += 8) {
            float pm[8], pl[8], pv[8];
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const size_t row = row0 + min(sp0 + k, ns - 1);
                pm[k] = coherent_load(a.part_ml + row * 2);
                pl[k] = coherent_load(a.part_ml + row * 2 + 1);
                pv[k] = coherent_load(a.part_o + row * D + e);
            }
            float mc = m;
#pragma unroll
            for (int k = 0; k < 8; k++) mc = fmaxf(mc, pm[k]); // a repeated last split does not change the max
            const float f = __builtin_amdgcn_exp2f(m - mc);      // 0 on the first group (m = -inf)
            num *= f;
            den *= f;
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (sp0 + k < ns) {
                    const float w = __builtin_amdgcn_exp2f(pm[k] - mc);
                    num += w * pv[k];
                    den += w * pl[k];
                }
            m = mc;
        }
        const float r = num / den;
        const size_t oi = ((size_t)b * a.hq + kvh * G + h) * D + e;
        if (a.out_f16) reinterpret_cast<__half *>(a.out)[oi] = __float2half_rn(r);
        else reinterpret_cast<float *>(a.out)[oi] = r;
    }
    if (threadIdx.x == 0) // ready for the next call on this stream
        __hip_atomic_store(done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}



// Sets `count` 32-bit words to zero (counter areas are cleared with a kernel, not a memset node, so
// the call may sit inside a captured graph).
__global__ void attn_zero_u32_kernel(uint32_t *p, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) p[i] = 0u;
}

// ---- static device scratch of the entry point that allocates nothing -------------------------
// One copy per GPU, held until the process ends: completion counters first, split partials after.
constexpr size_t kScratchCounterBytes = 64u << 10;  // 16384 (sequence, kv head) pairs
constexpr size_t kScratchPartialBytes = 8u << 20;   // batch * query heads * splits * (head_dim + 2) floats
static __device__ __align__(256) unsigned char scratch[kScratchCounterBytes + kScratchPartialBytes];

// Every GPU holds its own copy of the array at its own address: a context takes the address of its device's copy when
// it is created (ctx.hip) and the entry point uses that pointer, never the array's name.
hipError_t attn_static_scratch_address(void **ptr) { return hipGetSymbolAddress(ptr, HIP_SYMBOL(scratch)); }

// Everything a launch needs except the buffers: checked geometry, split plan, sizes of the scratch areas.
struct AttnPlan {
    AttnArgs a;
    int nt = 2, waves = 8;
    size_t partial_bytes = 0, counter_bytes = 0;
};

static int attn_plan(nncase_hip_ctx *ctx, const nncase_hip_paged_attn_args_t *p, AttnPlan *plan) {
    NNHIP_REQUIRE(ctx, p->batch > 0 && p->num_q_heads > 0 && p->num_kv_heads > 0 && p->max_blocks_per_seq > 0 &&
                           p->num_blocks > 0,
                  -EINVAL, "paged_attention_decode: non-positive dimension");
    NNHIP_REQUIRE(ctx, p->head_dim == 64 || p->head_dim == 128, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "paged_attention_decode: head_dim %d (64 or 128 supported)", p->head_dim);
    NNHIP_REQUIRE(ctx, p->num_q_heads % p->num_kv_heads == 0 && p->num_q_heads / p->num_kv_heads <= kAttnHeads,
                  -NNCASE_HIP_ERR_SHAPE_MISMATCH, "paged_attention_decode: %d query heads per kv head unsupported (max %d)",
                  p->num_q_heads / p->num_kv_heads, kAttnHeads);
    NNHIP_REQUIRE(ctx, p->block_size > 0 && p->block_size % 16 == 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "paged_attention_decode: block_size %d must be a multiple of 16", p->block_size);
    NNHIP_REQUIRE(ctx, (int64_t)p->max_blocks_per_seq * p->block_size < (int64_t(1) << 31), -EINVAL,
                  "paged_attention_decode: context capacity exceeds 2^31 tokens");
    NNHIP_REQUIRE(ctx, p->out_dtype == NNCASE_HIP_DT_F16 || p->out_dtype == NNCASE_HIP_DT_F32,
                  -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "paged_attention_decode: output type 0x%x", p->out_dtype);
    NNHIP_REQUIRE(ctx, (int64_t)p->batch * p->num_kv_heads < (int64_t(1) << 31), -EINVAL, "paged_attention_decode: grid too large");

    AttnArgs &a = plan->a;
    memset(&a, 0, sizeof(a));
    a.batch = p->batch;
    a.hq = p->num_q_heads;
    a.hkv = p->num_kv_heads;
    a.group = p->num_q_heads / p->num_kv_heads;
    a.d = p->head_dim;
    a.block_size = p->block_size;
    a.max_blocks = p->max_blocks_per_seq;
    a.num_blocks = p->num_blocks;
    a.len_offset = p->ctx_len_offset;
    const int64_t max_tokens = (int64_t)p->max_blocks_per_seq * p->block_size;
    // Eight waves per block, and tiles per wave: the largest run that still leaves about two blocks per compute unit
    // when every sequence is at full length (the kernel cannot know the real lengths on the host).  Measured at batch
    // 32, 2 kv heads, contexts of 512-4096 tokens, microseconds for 2 / 4 / 8 tiles per wave: four waves 17.7 / 14.2 /
    // 13.2, eight waves 13.3 / 12.2 / 12.9, sixteen waves 13.7 / 13.6 / 22.3 -- the same tokens per block are quicker as
    // more waves with shorter runs (more loads in flight per block, a shorter chain per wave), up to the point where a
    // block's merge through LDS outweighs it.  The rule picks 4 tiles there and 2 for the 16 sequences of a decode lane.
    const int nt_max = 512 / p->head_dim; // 8 KiB of K per wave
    const int waves = 8;
    auto splits_at = [&](int tiles) { return (max_tokens + waves * tiles * 16 - 1) / (waves * tiles * 16); };
    int nt = 2;
    while (nt < nt_max && (splits_at(nt) > kAttnMaxSplits ||
                           (int64_t)p->batch * p->num_kv_heads * splits_at(nt * 2) >= (int64_t)2 * ctx->compute_units))
        nt *= 2;
    plan->nt = nt;
    plan->waves = waves;
    a.split_tokens = waves * nt * 16;
    a.splits = (int)((max_tokens + a.split_tokens - 1) / a.split_tokens);
    NNHIP_REQUIRE(ctx, a.splits <= kAttnMaxSplits, -EINVAL,
                  "paged_attention_decode: context capacity of %lld tokens exceeds %d (head_dim %d)", (long long)max_tokens,
                  kAttnMaxSplits * a.split_tokens, p->head_dim);
    a.d_block = make_fastdiv((uint32_t)p->block_size);
    a.scale_log2e = p->scale * kLog2e;
    a.out_f16 = p->out_dtype == NNCASE_HIP_DT_F16;
    plan->partial_bytes = (size_t)a.batch * a.hq * a.splits * (a.d + 2) * sizeof(float);
    plan->counter_bytes = (size_t)a.batch * a.hkv * sizeof(uint32_t);
    return 0;
}

static int attn_launch(nncase_hip_ctx *ctx, AttnPlan &plan, const void *q_dev, const void *k_cache_dev, const void *v_cache_dev,
                       const int32_t *block_table_dev, const int32_t *ctx_lens_dev, void *out_dev, void *partials, void *counters) {
    AttnArgs &a = plan.a;
    a.q = (const uint16_t *)q_dev;
    a.k_cache = (const uint16_t *)k_cache_dev;
    a.v_cache = (const uint16_t *)v_cache_dev;
    a.block_table = block_table_dev;
    a.ctx_lens = ctx_lens_dev;
    a.out = out_dev;
    a.done = reinterpret_cast<uint32_t *>(counters);
    a.part_o = reinterpret_cast<float *>(partials);
    a.part_ml = a.part_o + (size_t)a.batch * a.hq * a.splits * a.d;
    const dim3 grid(a.hkv * a.batch, a.splits);
    const int nt = plan.nt, waves = plan.waves;
    const dim3 block(waves * 64);
    const size_t lds = attn_lds_bytes(a.d, waves);
    bool launched = false;
    auto go = [&](auto kernel) {
        if (lds > 65536) { // more than 64 KiB of dynamic LDS has to be asked for (cheap: a field of the function's record)
            if (hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) return;
        }
        hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, a);
        launched = true;
    };
#define NNHIP_ATTN_CASE(DV, NTV, WV) \
    if (!launched && a.d == DV && nt == NTV && waves == WV) go(paged_attn_kernel<DV, NTV, WV>);
    NNHIP_ATTN_CASE(64, 8, 8) NNHIP_ATTN_CASE(64, 4, 8) NNHIP_ATTN_CASE(64, 2, 8)
    NNHIP_ATTN_CASE(128, 4, 8) NNHIP_ATTN_CASE(128, 2, 8)
#undef NNHIP_ATTN_CASE
    NNHIP_REQUIRE(ctx, launched, -EINVAL, "paged_attention_decode: no kernel for head_dim %d, %d tiles per wave, %d waves", a.d, nt, waves);
    NNHIP_LAUNCH_CHECK(ctx, "paged_attn_kernel");
    return 0;
}

// Makes the context's split workspace and counters large enough for this geometry.  Growth frees the
// old areas, so it is refused while a captured graph holds their addresses (-EBUSY) and while the
// context's stream is capturing (an allocation and a synchronisation would invalidate the capture):
// resident functions reserve when the operator is recorded, before any capture.
int attn_reserve(nncase_hip_ctx *ctx, const nncase_hip_paged_attn_args_t *p) {
    AttnPlan plan;
    const int rc = attn_plan(ctx, p, &plan);
    if (rc) return rc;
    if (ctx->attn_ws_bytes >= plan.partial_bytes && ctx->attn_done_bytes >= plan.counter_bytes) return 0;
    NNHIP_REQUIRE(ctx, ctx->attn_pins == 0, -EBUSY,
                  "paged_attention_decode: the split workspace would have to grow (%zu -> %zu bytes) while %d captured "
                  "function(s) refer to it; record the larger operator before capturing",
                  ctx->attn_ws_bytes, plan.partial_bytes, ctx->attn_pins);
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    NNHIP_HIP(ctx, hipStreamIsCapturing(ctx->stream, &cs));
    NNHIP_REQUIRE(ctx, cs == hipStreamCaptureStatusNone, -EBUSY,
                  "paged_attention_decode: the split workspace cannot be allocated while the stream is capturing");
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    if (ctx->attn_ws_bytes < plan.partial_bytes) {
        if (ctx->attn_ws) NNHIP_HIP(ctx, hipFree(ctx->attn_ws));
        ctx->attn_ws = nullptr;
        ctx->attn_ws_bytes = 0;
        NNHIP_HIP(ctx, hipMalloc(&ctx->attn_ws, plan.partial_bytes));
        ctx->attn_ws_bytes = plan.partial_bytes;
    }
    if (ctx->attn_done_bytes < plan.counter_bytes) {
        if (ctx->attn_done) NNHIP_HIP(ctx, hipFree(ctx->attn_done));
        ctx->attn_done = nullptr;
        ctx->attn_done_bytes = 0;
        const size_t cap = (plan.counter_bytes + 4095) / 4096 * 4096;
        NNHIP_HIP(ctx, hipMalloc(&ctx->attn_done, cap));
        ctx->attn_done_bytes = cap;
        // zero before the first launch; every launch leaves the counters it used at zero again
        hipLaunchKernelGGL(attn_zero_u32_kernel, dim3(4), dim3(256), 0, ctx->stream, (uint32_t *)ctx->attn_done, cap / 4);
        NNHIP_LAUNCH_CHECK(ctx, "attn_zero_u32_kernel");
        NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    }
    return 0;
}

int attn_scratch_sizes(nncase_hip_ctx *ctx, const nncase_hip_paged_attn_args_t *p, size_t *partial_bytes, size_t *counter_bytes) {
    AttnPlan plan;
    const int rc = attn_plan(ctx, p, &plan);
    if (rc) return rc;
    *partial_bytes = plan.partial_bytes, *counter_bytes = plan.counter_bytes;
    return 0;
}

int attn_decode_on(nncase_hip_ctx *ctx, const void *q_dev, const void *k_cache_dev, const void *v_cache_dev, const int32_t *block_table_dev,
                   const int32_t *ctx_lens_dev, void *out_dev, const nncase_hip_paged_attn_args_t *p, void *partials,
                   size_t partial_bytes, void *counters, size_t counter_bytes) {
    AttnPlan plan;
    const int rc = attn_plan(ctx, p, &plan);
    if (rc) return rc;
    NNHIP_REQUIRE(ctx, partials && counters && plan.partial_bytes <= partial_bytes && plan.counter_bytes <= counter_bytes, -ENOSPC,
                  "paged_attention_decode: the scratch areas brought along hold %zu and %zu bytes, the geometry needs %zu and %zu",
                  partial_bytes, counter_bytes, plan.partial_bytes, plan.counter_bytes);
    return attn_launch(ctx, plan, q_dev, k_cache_dev, v_cache_dev, block_table_dev, ctx_lens_dev, out_dev, partials, counters);
}

} // namespace nnhip

using namespace nnhip;

extern "C" int nncase_hip_paged_attention_decode(nncase_hip_ctx_t *ctx, const void *q_dev, const void *k_cache_dev,
                                                 const void *v_cache_dev, const int32_t *block_table_dev,
                                                 const int32_t *ctx_lens_dev, void *out_dev,
                                                 const nncase_hip_paged_attn_args_t *p) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, q_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && out_dev && p, -EINVAL,
                  "paged_attention_decode: null argument");
    AttnPlan plan;
    int rc = attn_plan(ctx, p, &plan);
    if (rc) return rc;
    if (ctx->attn_ws_bytes < plan.partial_bytes || ctx->attn_done_bytes < plan.counter_bytes) {
        rc = attn_reserve(ctx, p);
        if (rc) return rc;
    }
    return attn_launch(ctx, plan, q_dev, k_cache_dev, v_cache_dev, block_table_dev, ctx_lens_dev, out_dev, ctx->attn_ws,
                       ctx->attn_done);
}

extern "C" int nncase_hip_paged_attention_decode_noalloc(nncase_hip_ctx_t *ctx, const void *q_dev, const void *k_cache_dev,
                                                         const void *v_cache_dev, const int32_t *block_table_dev,
                                                         const int32_t *ctx_lens_dev, void *out_dev,
                                                         const nncase_hip_paged_attn_args_t *p) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, q_dev && k_cache_dev && v_cache_dev && block_table_dev && ctx_lens_dev && out_dev && p, -EINVAL,
                  "paged_attention_decode_noalloc: null argument");
    AttnPlan plan;
    const int rc = attn_plan(ctx, p, &plan);
    if (rc) return rc;
    NNHIP_REQUIRE(ctx, plan.partial_bytes <= kScratchPartialBytes && plan.counter_bytes <= kScratchCounterBytes, -ENOSPC,
                  "paged_attention_decode_noalloc: needs %zu bytes of split partials and %zu of counters; the static "
                  "scratch holds %zu and %zu (use nncase_hip_paged_attention_decode)",
                  plan.partial_bytes, plan.counter_bytes, kScratchPartialBytes, kScratchCounterBytes);
    NNHIP_REQUIRE(ctx, ctx->attn_static, -ENOMEM, "paged_attention_decode_noalloc: the context has no address for the static scratch");
    unsigned char *base = reinterpret_cast<unsigned char *>(ctx->attn_static);
    // The array keeps the previous call's contents: the counters this launch uses must start at zero.
    hipLaunchKernelGGL(attn_zero_u32_kernel, dim3(1), dim3(256), 0, ctx->stream, (uint32_t *)base, plan.counter_bytes / 4);
    NNHIP_LAUNCH_CHECK(ctx, "attn_zero_u32_kernel");
    return attn_launch(ctx, plan, q_dev, k_cache_dev, v_cache_dev, block_table_dev, ctx_lens_dev, out_dev,
                       base + kScratchCounterBytes, base);
}
