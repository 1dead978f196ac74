// Two pointwise (1x1, stride 1, no padding) quantized convolutions, the second reading the first's result, as one
// launch:  y1 = conv_a(x) [table] [+ residual],  y2 = conv_b(y1) [table].
//
// A linear-bottleneck network alternates a projection (many -> few channels, src/Nncase.Importer/TFLite/Conv2D.cs:17-69
// imports each as its own Conv2D) with the next block's expansion (few -> many).  At small batches the two are
// launch-latency-bound kernels of a few microseconds; here the few-channel tensor between them stays in LDS (it is
// also stored: a later residual add reads it), and the second product starts as soon as the first's tile exists.
//
// Work split: a workgroup owns 16 pixels and a range of conv_b's channel tiles.  It computes ALL of conv_a for its
// pixels (every workgroup of a pixel tile repeats that: the reduction is the cheap side of the pair and recomputing
// keeps enough workgroups alive on 7x7 and 14x14 maps), requantises it exactly as nncase_hip_qconv2d does, and
// multiplies the LDS tile with its range of conv_b.  Results are bit-identical to the two nncase_hip_qconv2d calls.
//
// Weights are re-packed for this kernel: [channel tile][k-step][64 lanes][16 bytes], lane (i, g) holding
// w[16 t + i][64 ks + 16 g ..] - 128 as s8 (zero past the real extents), so that one 16-byte load per lane is an MFMA
// operand and lane (j, g) of the result holds channels 16 t + 4 g .. + 3 of pixel j: four neighbours, one dword.
//
// The second stage alone is the few-pixel path of nncase_hip_qconv2d (qpointwise_rows_kernel, further down): one dense
// 1x1 convolution over at most 32 pixels, optionally behind a global average pool computed by the same launch.
#include "qconv.hpp"

#include <new>
#include <vector>

using namespace nnhip;

struct nncase_hip_qpair {
    const nncase_hip_weights *first = nullptr, *second = nullptr;
    int k1 = 0, n1 = 0, n2 = 0;     // x channels, y1 channels, y2 channels
    int ks1 = 0, ks2 = 0;           // k-steps of 64 of the two reductions
    int t1 = 0, t2 = 0;             // 16-channel tiles of the two results
    uint8_t *d_wa = nullptr, *d_wb = nullptr;
    int32_t *d_wsum_a = nullptr, *d_wsum_b = nullptr; // sum_k (w - 128) per output channel (padded to whole tiles)
    int32_t *d_bias_a = nullptr, *d_bias_b = nullptr; // bias, padded to whole tiles
};

namespace nnhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kPairMaxK1 = 1024;  // x channels
constexpr int kPairMaxN1 = 512;   // y1 channels
constexpr int kRowPad = 16;       // bytes between LDS rows beyond the padded reduction (spreads the 16 rows over the banks)

// bytes of an LDS row: the reduction rounded up to whole chunks of `chunk` k-steps, and the pad
__host__ __device__ constexpr int pair_row_bytes(int ksteps, int chunk) { return (ksteps + chunk - 1) / chunk * chunk * 64 + kRowPad; }

struct PairArgs {
    const uint8_t *x;
    uint8_t *y1, *y2;
    const uint8_t *wa, *wb;
    const int32_t *bias_a, *wsum_a, *bias_b, *wsum_b;
    const uint32_t *lut_a, *lut_b;
    int m;                 // pixels
    int k1, n1, n2;
    int ks1, ks2, t1, t2;
    int tiles_per_block;   // conv_b channel tiles per workgroup (blockIdx.y selects the range)
    int zxa, zwa, zxb, zwb; // zero points - 128
    Epilogue ep_a, ep_b;
    ResidualEpilogue rep_a;
    // with a 3x3 depthwise convolution in front (the DW kernels): x is ITS input [batch, in_h, in_w, k1], and the pixel
    // tile the first convolution multiplies is computed here instead of loaded
    const int16_t *dw_w;             // [9][k1]  w - zw
    const int32_t *dw_bias, *dw_wsum; // [k1]; sum over the taps of w - zw
    int in_h, in_w, out_w, out_hw, stride, pad_h, pad_w;
    FastDiv d_out_hw, d_out_w;
    int dw_zx;
    Epilogue ep_dw;
    // the second convolution alone (qpointwise_rows_kernel): x holds ITS input rows [m][n1]; its result may leave as the
    // float32 value of the u8 code, and its rows may be the global average of x [m][pool_hw][n1]
    int deq, deq_zero;
    float deq_scale;
    int pool_hw;
    float pool_zx, pool_sx, pool_zy, pool_sy;
};

__device__ __forceinline__ uint32_t table4(const uint8_t *t, uint32_t v) {
    return (uint32_t)t[v & 0xffu] | ((uint32_t)t[(v >> 8) & 0xffu] << 8) | ((uint32_t)t[(v >> 16) & 0xffu] << 16) |
           ((uint32_t)t[v >> 24] << 24);
}

// What a wave fetches from global memory for one channel tile ahead of multiplying it: the first KC weight fragments,
// and the constants of the tile's epilogue (bias, weight sums and, for the first convolution, the residual bytes).
template <int KC> struct TileLoads {
    v4i frag[KC];
    v4i bias, wsum;
    uint32_t res;
};

// Loads KC weight fragments of one tile from k-step ks0 on; past the tile's last k-step the last one is loaded again
// (the activation tile is zero there, so what such a fragment holds does not matter, and no lane branches).
template <int KC> __device__ __forceinline__ void load_chunk(v4i (&f)[KC], const uint8_t *w, int tile, int ks0, int ksteps, int lane) {
    const v4i *src = reinterpret_cast<const v4i *>(w) + (size_t)tile * ksteps * 64 + lane;
#pragma unroll
    for (int c = 0; c < KC; c++) f[c] = src[min(ks0 + c, ksteps - 1) * 64];
}

template <int KC, bool FIRST>
__device__ __forceinline__ void load_tile(TileLoads<KC> &l, const PairArgs &a, int tile, int ks0, int lane, int p) {
    load_chunk<KC>(l.frag, FIRST ? a.wa : a.wb, tile, ks0, FIRST ? a.ks1 : a.ks2, lane);
    const int ch = tile * 16 + (lane >> 4) * 4;
    l.bias = *reinterpret_cast<const v4i *>((FIRST ? a.bias_a : a.bias_b) + ch);
    l.wsum = *reinterpret_cast<const v4i *>((FIRST ? a.wsum_a : a.wsum_b) + ch);
    l.res = 0;
    if (FIRST && a.rep_a.res && p < a.m && ch < a.n1) l.res = *reinterpret_cast<const uint32_t *>(a.rep_a.res + (size_t)p * a.n1 + ch);
}

// sum over k of the LDS tile's row j (every lane of pixel j gets it)
__device__ __forceinline__ int32_t row_sum(const uint8_t *rows, int stride, int ksteps, int lane) {
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    const uint8_t *row = rows + (lane & 15) * stride + (lane >> 4) * 16;
    v4i rs = {0, 0, 0, 0};
#pragma unroll 1
    for (int ks = 0; ks < ksteps; ks++) rs = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, *reinterpret_cast<const v4i *>(row + ks * 64), rs, 0, 0, 0);
    return rs[0];
}

// One convolution of the pair for this wave's channel tiles first, first + step, ... below end.  `rows` is the LDS
// activation tile ([16][stride] s8); `cur` holds the loads of the first tile already.  FIRST: results go to the LDS tile
// `ys` as s8 (and to y1 when store_y1); else to y2.
template <int KC, bool FIRST>
__device__ __forceinline__ void run_stage(const PairArgs &a, const uint8_t *rows, int stride, uint8_t *ys, int sy, const uint8_t *lut, int first,
                                          int step, int end, TileLoads<KC> &cur, int lane, int p, bool store_y1) {
    const int j = lane & 15, g = lane >> 4;
    const int ksteps = FIRST ? a.ks1 : a.ks2;
    const int zx = FIRST ? a.zxa : a.zxb, zw = FIRST ? a.zwa : a.zwb;
    const Epilogue &ep = FIRST ? a.ep_a : a.ep_b;
    const int32_t nrs = -zw * row_sum(rows, stride, ksteps, lane);
    const int32_t kzz = (FIRST ? a.k1 : a.n1) * zx * zw;
    const uint8_t *row = rows + j * stride + g * 16;
    v4i bias = cur.bias, ws = cur.wsum; // the constants of a tile arrive with its first chunk and are used after its last
    uint32_t rv = cur.res;
#pragma unroll 1
    for (int t = first; t < end; t += step) {
        v4i acc = {0, 0, 0, 0};
#pragma unroll 1
        for (int ks0 = 0; ks0 < ksteps; ks0 += KC) {
            // what follows this chunk (the tile's next one, else the next tile's first) travels while this one multiplies;
            // one wave-uniform branch around all of it: behind the last chunk nothing is requested, so nothing is waited for
            const bool more = ks0 + KC < ksteps;
            TileLoads<KC> nxt;
            if (more || t + step < end) load_tile<KC, FIRST>(nxt, a, more ? t : t + step, more ? ks0 + KC : 0, lane, p);
            if (!more) bias = cur.bias, ws = cur.wsum, rv = cur.res;
#pragma unroll
            for (int c = 0; c < KC; c++) {
                const v4i xf = *reinterpret_cast<const v4i *>(row + (ks0 + c) * 64);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(cur.frag[c], xf, acc, 0, 0, 0);
            }
            cur = nxt;
        }
        const int ch = t * 16 + g * 4;
        int32_t v[4];
#pragma unroll
        for (int r = 0; r < 4; r++) v[r] = acc[r] + (bias[r] - zx * ws[r] + kzz) + nrs;
        uint32_t q = requant4_u8_packed(v, ep);
        if (lut) q = table4(lut, q);
        if constexpr (FIRST) {
            if (ch < a.n1) {
                if (a.rep_a.res) q = residual4_packed(q, rv, a.rep_a);
                *reinterpret_cast<uint32_t *>(ys + j * sy + ch) = q ^ 0x80808080u;
                if (store_y1 && p < a.m) *reinterpret_cast<uint32_t *>(a.y1 + (size_t)p * a.n1 + ch) = q;
            }
        } else if (ch < a.n2 && p < a.m) {
            if (a.deq) { // the Dequantize behind the convolution: one float per channel
                u32x4 o;
#pragma unroll
                for (int r = 0; r < 4; r++) o[r] = __float_as_uint((float)((int)((q >> (8 * r)) & 0xffu) - a.deq_zero) * a.deq_scale);
                *reinterpret_cast<u32x4 *>(reinterpret_cast<float *>(a.y2) + (size_t)p * a.n2 + ch) = o;
            } else {
                *reinterpret_cast<uint32_t *>(a.y2 + (size_t)p * a.n2 + ch) = q;
            }
        }
    }
}

// The nine input dwords (four channels from c4) of output pixel `px`'s window; taps outside the image read as the
// zero point, whose share the accumulator's start value takes back out (addresses are clamped into the image, so the
// loads need no branch).
__device__ __forceinline__ void dw_fetch(uint32_t (&buf)[9], const PairArgs &a, int px, int c4) {
    px = min(px, a.m - 1);
    const int n = (int)fastdiv((uint32_t)px, a.d_out_hw), rem = px - n * a.out_hw;
    const int oy = (int)fastdiv((uint32_t)rem, a.d_out_w), ox = rem - oy * a.out_w;
    const int iy0 = oy * a.stride - a.pad_h, ix0 = ox * a.stride - a.pad_w;
    const uint32_t zx4 = (uint32_t)a.dw_zx * 0x01010101u;
#pragma unroll
    for (int ky = 0; ky < 3; ky++) {
        const int iy = iy0 + ky, iyc = min(max(iy, 0), a.in_h - 1);
        const uint8_t *rowp = a.x + (size_t)(n * a.in_h + iyc) * a.in_w * a.k1 + c4;
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const int ix = ix0 + kx, ixc = min(max(ix, 0), a.in_w - 1);
            const uint32_t v = *reinterpret_cast<const uint32_t *>(rowp + (size_t)ixc * a.k1);
            buf[ky * 3 + kx] = (iy == iyc && ix == ixc) ? v : zx4;
        }
    }
}

// The depthwise convolution's 16 pixels x k1 channels, requantised, into the LDS tile as s8.  A thread keeps the
// weights of four channels and walks the pixels pg, pg + pgs, ...: the next pixel's window is requested before this
// one is multiplied.
__device__ __forceinline__ void dw_stage(const PairArgs &a, uint8_t *xs, int sx, int p0, int tid, int threads) {
    const int quads = a.k1 >> 2;
    const bool wide = threads >= quads;            // a thread per channel quad, and pixel groups of them
    const int pgs = wide ? threads / quads : 1, pg = wide ? tid / quads : 0;
    if (pg >= pgs) return;
#pragma unroll 1
    for (int q = wide ? tid - pg * quads : tid; q < quads; q += wide ? quads : threads) {
        const int c4 = q * 4;
        uint32_t cur[9], w01[9], w23[9];
        dw_fetch(cur, a, p0 + pg, c4);
#pragma unroll
        for (int t = 0; t < 9; t++) {
            const uint2 wv = *reinterpret_cast<const uint2 *>(a.dw_w + (size_t)t * a.k1 + c4);
            w01[t] = wv.x, w23[t] = wv.y;
        }
        const v4i bias = *reinterpret_cast<const v4i *>(a.dw_bias + c4), ws = *reinterpret_cast<const v4i *>(a.dw_wsum + c4);
        int32_t ct[4];
#pragma unroll
        for (int c = 0; c < 4; c++) ct[c] = bias[c] - a.dw_zx * ws[c];
#pragma unroll 1
        for (int r = pg; r < 16; r += pgs) {
            uint32_t nxt[9];
            if (r + pgs < 16) dw_fetch(nxt, a, p0 + r + pgs, c4);
            int32_t acc[4] = {ct[0], ct[1], ct[2], ct[3]};
#pragma unroll
            for (int t = 0; t < 9; t++) {
                const uint32_t x01 = __builtin_amdgcn_perm(0, cur[t], 0x0c010c00u), x23 = __builtin_amdgcn_perm(0, cur[t], 0x0c030c02u);
                acc[0] = mad16_lo(x01, w01[t], acc[0]);
                acc[1] = mad16_hi(x01, w01[t], acc[1]);
                acc[2] = mad16_lo(x23, w23[t], acc[2]);
                acc[3] = mad16_hi(x23, w23[t], acc[3]);
            }
            uint32_t code = requant4_u8_packed(acc, a.ep_dw);
            if (p0 + r >= a.m) code = 0x80808080u; // rows past the tensor read as zero
            *reinterpret_cast<uint32_t *>(xs + r * sx + c4) = code ^ 0x80808080u;
#pragma unroll
            for (int t = 0; t < 9; t++) cur[t] = nxt[t];
        }
    }
}

// KA / KB: weight fragments a wave requests at a time for the first / second convolution (each twice in registers).
// MAXW: most waves a workgroup is launched with; OCC: waves per SIMD the register budget is held to.
// DW: a 3x3 depthwise convolution produces the pixel tile (dw_stage).
template <int KA, int KB, int MAXW, int OCC, bool DW>
__global__ __launch_bounds__(MAXW * 64, OCC) void qpointwise_pair_kernel(const PairArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    // rows hold whole chunks of k-steps, zero past the real reduction
    const int sx = pair_row_bytes(a.ks1, KA), sy = pair_row_bytes(a.ks2, KB);
    uint8_t *xs = smem;              // [16][sx]  x - 128
    uint8_t *ys = xs + 16 * sx;      // [16][sy]  y1 - 128
    uint8_t *lut_a = ys + 16 * sy;   // 256 bytes each
    uint8_t *lut_b = lut_a + 256;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, threads = blockDim.x, waves = threads >> 6;
    const int p0 = blockIdx.x * 16, p = p0 + (lane & 15);
    const int b_first = blockIdx.y * a.tiles_per_block;
    const int b_end = min(a.t2, b_first + a.tiles_per_block);

    // the first tiles' weights and constants travel while the pixel tile is staged
    TileLoads<KA> la;
    TileLoads<KB> lb;
    if (wave < a.t1) load_tile<KA, true>(la, a, wave, 0, lane, p);
    if (b_first + wave < b_end) load_tile<KB, false>(lb, a, b_first + wave, 0, lane, p);

    // x tile as s8 (x - 128); rows past the tensor and bytes past K read as zero
    const int pieces = (sx - kRowPad) / 16; // 16-byte pieces per row
    if constexpr (DW) {
        dw_stage(a, xs, sx, p0, tid, threads);
        const int first = a.k1 / 16, extra = pieces - first;
        for (int e = tid; e < 16 * extra; e += threads) {
            const int r = e / extra, c = first + (e - r * extra);
            *reinterpret_cast<u32x4 *>(xs + r * sx + c * 16) = u32x4{0u, 0u, 0u, 0u};
        }
    } else {
#pragma unroll 1
        for (int e = tid; e < 16 * pieces; e += threads) {
            const int r = e / pieces, c = e - r * pieces;
            u32x4 v = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
            if (p0 + r < a.m && c * 16 < a.k1) v = *reinterpret_cast<const u32x4 *>(a.x + (size_t)(p0 + r) * a.k1 + c * 16);
            *reinterpret_cast<u32x4 *>(xs + r * sx + c * 16) = v ^ 0x80808080u;
        }
    }
    for (int e = tid; e < 4 * sy; e += threads) reinterpret_cast<uint32_t *>(ys)[e] = 0; // channels past N1 stay zero
    for (int e = tid; e < 128; e += threads) {
        if (e < 64) {
            if (a.lut_a) reinterpret_cast<uint32_t *>(lut_a)[e] = a.lut_a[e];
        } else if (a.lut_b) {
            reinterpret_cast<uint32_t *>(lut_b)[e - 64] = a.lut_b[e - 64];
        }
    }
    __syncthreads();
    // the first convolution over the whole of its channels, into LDS (and, from the first channel range, into y1)
    if (wave < a.t1) run_stage<KA, true>(a, xs, sx, ys, sy, a.lut_a ? lut_a : nullptr, wave, waves, a.t1, la, lane, p, blockIdx.y == 0);
    __syncthreads();
    // the second: this workgroup's channel tiles from the LDS tile
    if (b_first + wave < b_end) run_stage<KB, false>(a, ys, sy, nullptr, 0, a.lut_b ? lut_b : nullptr, b_first + wave, waves, b_end, lb, lane, p, false);
}

// One dense 1x1 convolution over a few rows (pixels): the second stage of the pair kernel alone.  A workgroup stages 16
// rows as s8 in LDS and takes a range of the channel tiles, a wave per tile, the weights straight from global memory
// into MFMA operands with the first chunk requested before the rows are staged.  Against the tiled kernels, which
// stream k-step by k-step through LDS with a barrier each, a launch is one memory round trip long, not one per k-step.
// POOL: the rows are global averages over pool_hw pixels, computed here (global_avgpool4, a thread per four channels).
constexpr int kRowsChunk = 8, kRowsWaves = 12;
template <bool POOL> __global__ __launch_bounds__(kRowsWaves * 64, 3) void qpointwise_rows_kernel(const PairArgs a) {
    extern __shared__ __align__(16) uint8_t smem[];
    const int sy = pair_row_bytes(a.ks2, kRowsChunk);
    uint8_t *ys = smem;            // [16][sy]  rows - 128
    uint8_t *lut_b = ys + 16 * sy; // 256 bytes
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, threads = blockDim.x, waves = threads >> 6;
    const int p0 = blockIdx.x * 16, p = p0 + (lane & 15);
    const int b_first = blockIdx.y * a.tiles_per_block;
    const int b_end = min(a.t2, b_first + a.tiles_per_block);
    TileLoads<kRowsChunk> lb;
    if (b_first + wave < b_end) load_tile<kRowsChunk, false>(lb, a, b_first + wave, 0, lane, p);
    if constexpr (POOL) {
        const int quads = a.n1 >> 2;
#pragma unroll 1
        for (int e = tid; e < 16 * quads; e += threads) {
            const int r = e / quads, c4 = (e - r * quads) * 4;
            uint32_t code = 0x80808080u; // rows past the tensor read as zero
            if (p0 + r < a.m) code = global_avgpool4(a.x + (size_t)(p0 + r) * a.pool_hw * a.n1 + c4, a.pool_hw, a.n1, a.pool_zx, a.pool_sx, a.pool_zy, a.pool_sy);
            *reinterpret_cast<uint32_t *>(ys + r * sy + c4) = code ^ 0x80808080u;
        }
        const int first = a.n1 / 16, extra = (sy - kRowPad) / 16 - first; // pieces past the real reduction
        for (int e = tid; e < 16 * extra; e += threads) {
            const int r = e / extra, c = first + (e - r * extra);
            *reinterpret_cast<u32x4 *>(ys + r * sy + c * 16) = u32x4{0u, 0u, 0u, 0u};
        }
    } else {
        const int pieces = (sy - kRowPad) / 16;
#pragma unroll 1
        for (int e = tid; e < 16 * pieces; e += threads) {
            const int r = e / pieces, c = e - r * pieces;
            u32x4 v = {0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};
            if (p0 + r < a.m && c * 16 < a.n1) v = *reinterpret_cast<const u32x4 *>(a.x + (size_t)(p0 + r) * a.n1 + c * 16);
            *reinterpret_cast<u32x4 *>(ys + r * sy + c * 16) = v ^ 0x80808080u;
        }
    }
    if (a.lut_b)
        for (int e = tid; e < 64; e += threads) reinterpret_cast<uint32_t *>(lut_b)[e] = a.lut_b[e];
    __syncthreads();
    if (b_first + wave < b_end) run_stage<kRowsChunk, false>(a, ys, sy, nullptr, 0, a.lut_b ? lut_b : nullptr, b_first + wave, waves, b_end, lb, lane, p, false);
}

static bool pair_is_small(int ks1, int ks2) { return ks1 <= 4 && ks2 <= 2; }
static size_t pair_lds_bytes(const nncase_hip_qpair *pr) {
    const bool small = pair_is_small(pr->ks1, pr->ks2);
    return 16 * (size_t)pair_row_bytes(pr->ks1, small ? 4 : 8) + 16 * (size_t)pair_row_bytes(pr->ks2, small ? 2 : 4) + 512;
}

// [tile][k-step][lane][16] s8 of w - 128, zero beyond the real channels / reduction
static void pack_pair_weights(std::vector<uint8_t> &out, std::vector<int32_t> &wsum, const uint8_t *w_oihw, int n, int k, int tiles, int ksteps) {
    out.assign((size_t)tiles * ksteps * 1024, 0);
    wsum.assign((size_t)tiles * 16, 0);
    for (int ch = 0; ch < n; ch++) {
        int32_t s = 0;
        for (int kk = 0; kk < k; kk++) {
            const uint8_t raw = w_oihw[(size_t)ch * k + kk];
            s += (int32_t)raw - 128;
            const int t = ch >> 4, i = ch & 15, ks = kk >> 6, g = (kk >> 4) & 3, b = kk & 15;
            out[(((size_t)t * ksteps + ks) * 64 + g * 16 + i) * 16 + b] = raw ^ 0x80;
        }
        wsum[ch] = s;
    }
}

static void free_pair(nncase_hip_qpair *pr) {
    if (!pr) return;
    if (pr->d_wa) (void)hipFree(pr->d_wa);
    if (pr->d_wb) (void)hipFree(pr->d_wb);
    if (pr->d_wsum_a) (void)hipFree(pr->d_wsum_a);
    if (pr->d_wsum_b) (void)hipFree(pr->d_wsum_b);
    if (pr->d_bias_a) (void)hipFree(pr->d_bias_a);
    if (pr->d_bias_b) (void)hipFree(pr->d_bias_b);
    delete pr;
}

static bool pair_shapes_ok(int k1, int n1, int n2) {
    return k1 > 0 && n1 > 0 && n2 > 0 && k1 % 16 == 0 && n1 % 4 == 0 && n2 % 4 == 0 && k1 <= kPairMaxK1 && n1 <= kPairMaxN1;
}

static int upload(nncase_hip_ctx *ctx, void **dst, const void *src, size_t bytes) {
    NNHIP_HIP(ctx, hipMalloc(dst, bytes));
    NNHIP_HIP(ctx, hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
    return 0;
}

static bool pointwise_weights(const nncase_hip_weights *w) {
    return w && w->kind == nncase_hip_weights::kIgemm && w->groups == 1 && w->kernel_h == 1 && w->kernel_w == 1;
}

} // namespace nnhip

extern "C" int nncase_hip_qpointwise_pair_supported(int32_t in_channels, int32_t mid_channels, int32_t out_channels) {
    return pair_shapes_ok(in_channels, mid_channels, out_channels) ? 1 : 0;
}

extern "C" int nncase_hip_qpointwise_pair_create(nncase_hip_ctx_t *ctx, const nncase_hip_weights_t *first,
                                                 const uint8_t *first_oihw_host, const nncase_hip_weights_t *second,
                                                 const uint8_t *second_oihw_host, nncase_hip_qpair_t **pair) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, first && first_oihw_host && second && second_oihw_host && pair, -EINVAL, "qpointwise_pair_create: null argument");
    *pair = nullptr;
    NNHIP_REQUIRE(ctx, pointwise_weights(first) && pointwise_weights(second), -EINVAL,
                  "qpointwise_pair_create: both convolutions must be dense 1x1 convolutions");
    NNHIP_REQUIRE(ctx, first->out_channels == second->in_channels, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "qpointwise_pair_create: the first convolution has %d output channels, the second reads %d", first->out_channels,
                  second->in_channels);
    NNHIP_REQUIRE(ctx, pair_shapes_ok(first->in_channels, first->out_channels, second->out_channels), -EINVAL,
                  "qpointwise_pair_create: channels %d -> %d -> %d unsupported (first a multiple of 16 up to %d, second a multiple of 4 "
                  "up to %d, third a multiple of 4)",
                  first->in_channels, first->out_channels, second->out_channels, kPairMaxK1, kPairMaxN1);
    nncase_hip_qpair *pr = new (std::nothrow) nncase_hip_qpair();
    NNHIP_REQUIRE(ctx, pr, -ENOMEM, "qpointwise_pair_create: out of host memory");
    pr->first = first, pr->second = second;
    pr->k1 = first->in_channels, pr->n1 = first->out_channels, pr->n2 = second->out_channels;
    pr->ks1 = (pr->k1 + 63) / 64, pr->ks2 = (pr->n1 + 63) / 64;
    pr->t1 = (pr->n1 + 15) / 16, pr->t2 = (pr->n2 + 15) / 16;
    NNHIP_HIP(ctx, hipSetDevice(ctx->device));
    std::vector<uint8_t> packed;
    std::vector<int32_t> wsum, bias;
    int rc = 0;
    auto side = [&](const nncase_hip_weights *w, const uint8_t *host, int n, int k, int tiles, int ksteps, uint8_t **d_w, int32_t **d_wsum,
                    int32_t **d_bias) -> int {
        pack_pair_weights(packed, wsum, host, n, k, tiles, ksteps);
        bias.assign((size_t)tiles * 16, 0);
        NNHIP_HIP(ctx, hipMemcpy(bias.data(), w->d_bias, sizeof(int32_t) * n, hipMemcpyDeviceToHost));
        int r = upload(ctx, (void **)d_w, packed.data(), packed.size());
        if (!r) r = upload(ctx, (void **)d_wsum, wsum.data(), wsum.size() * sizeof(int32_t));
        if (!r) r = upload(ctx, (void **)d_bias, bias.data(), bias.size() * sizeof(int32_t));
        return r;
    };
    rc = side(first, first_oihw_host, pr->n1, pr->k1, pr->t1, pr->ks1, &pr->d_wa, &pr->d_wsum_a, &pr->d_bias_a);
    if (!rc) rc = side(second, second_oihw_host, pr->n2, pr->n1, pr->t2, pr->ks2, &pr->d_wb, &pr->d_wsum_b, &pr->d_bias_b);
    if (rc) {
        free_pair(pr);
        return rc;
    }
    *pair = pr;
    return 0;
}

extern "C" int nncase_hip_qpointwise_pair_destroy(nncase_hip_ctx_t *ctx, nncase_hip_qpair_t *pair) {
    NNHIP_CHECK_CTX(ctx);
    if (!pair) return 0;
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    free_pair(pair);
    return 0;
}

// ---- the few-pixel path of one dense 1x1 convolution ----------------------------------------------------------------
namespace nnhip {
constexpr int kRowsMaxK = 2048;                 // reduction length (an LDS row: 16 of them stay below 64 KiB)
constexpr int64_t kRowsStreamLimit = 4 << 20;   // weight bytes all pixel tiles stream between them
constexpr int64_t kRowsMaxPixels = 32;          // beyond two pixel tiles the tiled kernels, which share the weights of a tile
                                                // among many pixels, are the faster ones (measured on MobileNetV2's 7x7 layers)

bool rows_shapes_ok(int in_channels, int out_channels, int64_t pixels) {
    return pixels > 0 && pixels <= kRowsMaxPixels && in_channels % 16 == 0 && out_channels % 4 == 0 && in_channels <= kRowsMaxK &&
           (pixels + 15) / 16 * (int64_t)in_channels * out_channels <= kRowsStreamLimit;
}

// Every workgroup of the pooled launch pools its (up to 16) rows itself, on one compute unit: beyond this many values
// per workgroup the separate pool kernel, which spreads over the device, is the faster one.
bool pool_front_pays(int rows, int hw, int channels) { return (int64_t)std::min(rows, 16) * hw * channels <= (128 << 10); }

int rows_prepack(nncase_hip_ctx *ctx, nncase_hip_weights *w, const uint8_t *w_oihw) {
    if (!(pointwise_weights(w) && rows_shapes_ok(w->in_channels, w->out_channels, w->pixels_hint))) return 0; // not a call this path is for
    nncase_hip_qpair *pr = new (std::nothrow) nncase_hip_qpair();
    NNHIP_REQUIRE(ctx, pr, -ENOMEM, "qconv2d_prepack: out of host memory");
    pr->second = w;
    pr->n1 = w->in_channels, pr->n2 = w->out_channels;
    pr->ks2 = (pr->n1 + 63) / 64, pr->t2 = (pr->n2 + 15) / 16;
    std::vector<uint8_t> packed;
    std::vector<int32_t> wsum, bias((size_t)pr->t2 * 16, 0);
    pack_pair_weights(packed, wsum, w_oihw, pr->n2, pr->n1, pr->t2, pr->ks2);
    const hipError_t got = hipMemcpy(bias.data(), w->d_bias, sizeof(int32_t) * pr->n2, hipMemcpyDeviceToHost);
    int rc = got == hipSuccess ? 0 : hip_fail(ctx, got, "hipMemcpy(bias)");
    if (!rc) rc = upload(ctx, (void **)&pr->d_wb, packed.data(), packed.size());
    if (!rc) rc = upload(ctx, (void **)&pr->d_wsum_b, wsum.data(), wsum.size() * sizeof(int32_t));
    if (!rc) rc = upload(ctx, (void **)&pr->d_bias_b, bias.data(), bias.size() * sizeof(int32_t));
    if (rc) { // (the failing call has left its message)
        free_pair(pr);
        return rc;
    }
    w->rows_pack = pr;
    return 0;
}

void rows_free(nncase_hip_weights *w) {
    if (w && w->rows_pack) free_pair(w->rows_pack);
    if (w) w->rows_pack = nullptr;
}

bool rows_path_taken(const nncase_hip_weights *w, const nncase_hip_conv2d_args_t *c, int out_h, int out_w) {
    if (!w->rows_pack || c->residual_dev || c->out_channel_stride || c->out_channel_offset) return false;
    if (!(c->stride_h == 1 && c->stride_w == 1 && c->pad_h_before == 0 && c->pad_w_before == 0 && out_h == c->in_h && out_w == c->in_w)) return false;
    // (u8 codes, or their float32 values: the entry point turns the latter into a u8 call with the flag set)
    if (!(c->out_dtype == NNCASE_HIP_DT_U8 || (c->out_dtype == NNCASE_HIP_DT_F32 && c->dequantize_output != 0))) return false;
    return rows_shapes_ok(w->in_channels, w->out_channels, (int64_t)c->batch * out_h * out_w);
}

int launch_qconv_rows(nncase_hip_ctx *ctx, const uint8_t *x, const nncase_hip_weights *w, void *y, const nncase_hip_conv2d_args_t *c,
                      const PoolFront *pool) {
    const nncase_hip_qpair *pr = w->rows_pack;
    const int64_t m64 = (int64_t)c->batch * c->in_h * c->in_w;
    NNHIP_REQUIRE(ctx, m64 > 0 && m64 < ((int64_t)1 << 30), -EINVAL, "qconv2d: %lld output pixels unsupported", (long long)m64);
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (reinterpret_cast<uintptr_t>(y) & 15u) == 0,
                  -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION, "qconv2d: activation buffers must be 16-byte aligned");
    PairArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x, a.y2 = reinterpret_cast<uint8_t *>(y);
    a.wb = pr->d_wb, a.bias_b = pr->d_bias_b, a.wsum_b = pr->d_wsum_b;
    a.lut_b = w->d_post_lut;
    a.m = (int)m64;
    a.n1 = pr->n1, a.n2 = pr->n2, a.ks2 = pr->ks2, a.t2 = pr->t2;
    a.zxb = c->x_qp.zero_point - 128, a.zwb = w->zw - 128;
    const int rc = make_epilogue(ctx, &a.ep_b, c->x_qp.scale, w->sw, c->y_qp, c->clamp_min, c->clamp_max, NNCASE_HIP_DT_U8, "qconv2d");
    if (rc) return rc;
    if (c->dequantize_output != 0) {
        const nncase_hip_quant_param_t last = w->d_post_lut ? w->post_lut_qp : c->y_qp;
        a.deq = 1, a.deq_zero = last.zero_point, a.deq_scale = last.scale;
    }
    if (pool) {
        NNHIP_REQUIRE(ctx, pool->hw > 0 && (int64_t)m64 * pool->hw * pr->n1 < ((int64_t)1 << 31), -EINVAL, "qglobal_avgpool_qconv2d: input too large");
        a.pool_hw = pool->hw;
        a.pool_zx = (float)pool->x_qp.zero_point, a.pool_sx = pool->x_qp.scale;
        a.pool_zy = (float)c->x_qp.zero_point, a.pool_sy = c->x_qp.scale;
    }
    // pixel tiles x ranges of channel tiles, a wave per tile, enough workgroups to spread the weights over the device
    const int ptiles = (a.m + 15) / 16;
    int ranges = (a.t2 + kRowsWaves - 1) / kRowsWaves;
    const int want = std::max(1, 2 * ctx->compute_units / ptiles);
    int per = std::max(1, (a.t2 + want - 1) / want); // tiles per workgroup when as many workgroups as wanted
    if (pool) per = std::max(per, 4);                 // (every workgroup repeats the pooling)
    ranges = (a.t2 + per - 1) / per;
    a.tiles_per_block = per;
    int waves = std::min(kRowsWaves, per);
    if (pool) waves = kRowsWaves; // the pooling has a thread per four channels
    const size_t lds = 16 * (size_t)pair_row_bytes(a.ks2, kRowsChunk) + 256;
    NNHIP_HIP(ctx, hipSetDevice(ctx->device));
    if (pool) hipLaunchKernelGGL(qpointwise_rows_kernel<true>, dim3(ptiles, ranges), dim3(waves * 64), lds, ctx->stream, a);
    else hipLaunchKernelGGL(qpointwise_rows_kernel<false>, dim3(ptiles, ranges), dim3(waves * 64), lds, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "qpointwise_rows_kernel");
    return 0;
}
} // namespace nnhip

// dw / da: the depthwise convolution in front and its arguments, or null
static int launch_pair(nncase_hip_ctx *ctx, const char *who, const uint8_t *x_dev, const nncase_hip_weights *dw,
                       const nncase_hip_conv2d_args_t *da, const nncase_hip_qpair *pr, uint8_t *y1_dev, uint8_t *y2_dev,
                       const nncase_hip_conv2d_args_t *fa, const nncase_hip_conv2d_args_t *sa) {
    NNHIP_REQUIRE(ctx, x_dev && pr && y1_dev && y2_dev && fa && sa, -EINVAL, "%s: null argument", who);
    NNHIP_REQUIRE(ctx, fa->batch > 0 && fa->in_h > 0 && fa->in_w > 0, -EINVAL, "%s: non-positive input shape", who);
    NNHIP_REQUIRE(ctx, sa->batch == fa->batch && sa->in_h == fa->in_h && sa->in_w == fa->in_w, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "%s: the second convolution reads [%d,%d,%d], the first writes [%d,%d,%d]", who, sa->batch, sa->in_h, sa->in_w, fa->batch,
                  fa->in_h, fa->in_w);
    for (const nncase_hip_conv2d_args_t *c : {fa, sa}) {
        NNHIP_REQUIRE(ctx, c->stride_h == 1 && c->stride_w == 1 && c->pad_h_before == 0 && c->pad_h_after == 0 && c->pad_w_before == 0 &&
                               c->pad_w_after == 0,
                      -EINVAL, "%s: stride 1 and no padding only for the 1x1 convolutions", who);
    }
    for (const nncase_hip_conv2d_args_t *c : {fa, sa, da}) {
        if (!c) continue;
        NNHIP_REQUIRE(ctx, c->out_dtype == NNCASE_HIP_DT_U8 && c->dequantize_output == 0, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "%s: u8 results only",
                      who);
        NNHIP_REQUIRE(ctx, c->out_channel_stride == 0 && c->out_channel_offset == 0, -EINVAL, "%s: dense results only", who);
        NNHIP_REQUIRE(ctx, c->x_qp.zero_point >= 0 && c->x_qp.zero_point <= 255, -EINVAL, "%s: input zero point %d outside u8", who,
                      c->x_qp.zero_point);
        NNHIP_REQUIRE(ctx, c->y_qp.scale > 0.f && std::isfinite(c->y_qp.scale) && c->y_qp.zero_point >= 0 && c->y_qp.zero_point <= 255, -EINVAL,
                      "%s: output quantisation outside u8", who);
    }
    NNHIP_REQUIRE(ctx, !sa->residual_dev, -EINVAL, "%s: only the first 1x1 convolution takes a residual", who);
    if (fa->residual_dev)
        NNHIP_REQUIRE(ctx, fa->sum_qp.scale > 0.f && std::isfinite(fa->sum_qp.scale) && fa->sum_qp.zero_point >= 0 && fa->sum_qp.zero_point <= 255,
                      -EINVAL, "%s: sum quantisation outside u8", who);
    const int64_t m64 = (int64_t)fa->batch * fa->in_h * fa->in_w;
    NNHIP_REQUIRE(ctx, m64 < ((int64_t)1 << 30), -EINVAL, "%s: %lld pixels unsupported", who, (long long)m64);
    NNHIP_REQUIRE(ctx, ((reinterpret_cast<uintptr_t>(x_dev) | reinterpret_cast<uintptr_t>(y1_dev) | reinterpret_cast<uintptr_t>(y2_dev)) & 15u) == 0,
                  -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION, "%s: activation buffers must be 16-byte aligned", who);

    PairArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x_dev, a.y1 = y1_dev, a.y2 = y2_dev;
    a.wa = pr->d_wa, a.wb = pr->d_wb;
    a.bias_a = pr->d_bias_a, a.wsum_a = pr->d_wsum_a, a.bias_b = pr->d_bias_b, a.wsum_b = pr->d_wsum_b;
    a.lut_a = pr->first->d_post_lut, a.lut_b = pr->second->d_post_lut;
    a.m = (int)m64;
    a.k1 = pr->k1, a.n1 = pr->n1, a.n2 = pr->n2;
    a.ks1 = pr->ks1, a.ks2 = pr->ks2, a.t1 = pr->t1, a.t2 = pr->t2;
    a.zxa = fa->x_qp.zero_point - 128, a.zwa = pr->first->zw - 128;
    a.zxb = sa->x_qp.zero_point - 128, a.zwb = pr->second->zw - 128;
    int rc = make_epilogue(ctx, &a.ep_a, fa->x_qp.scale, pr->first->sw, fa->y_qp, fa->clamp_min, fa->clamp_max, NNCASE_HIP_DT_U8, who);
    if (!rc) rc = make_epilogue(ctx, &a.ep_b, sa->x_qp.scale, pr->second->sw, sa->y_qp, sa->clamp_min, sa->clamp_max, NNCASE_HIP_DT_U8, who);
    if (!rc) rc = make_residual_epilogue(ctx, &a.rep_a, fa, pr->first);
    if (rc) return rc;
    if (dw) {
        NNHIP_REQUIRE(ctx, da, -EINVAL, "%s: null argument", who);
        NNHIP_REQUIRE(ctx, dw->kind == nncase_hip_weights::kDepthwise && dw->kernel_h == 3 && dw->kernel_w == 3 && dw->out_channels == pr->k1, -EINVAL,
                      "%s: the convolution in front must be a 3x3 depthwise convolution over the first 1x1 convolution's %d channels", who, pr->k1);
        NNHIP_REQUIRE(ctx, !dw->d_post_lut && !da->residual_dev, -EINVAL, "%s: the depthwise convolution takes no table or residual", who);
        NNHIP_REQUIRE(ctx, da->stride_h == da->stride_w && (da->stride_h == 1 || da->stride_h == 2) && da->dilation_h == 1 && da->dilation_w == 1,
                      -EINVAL, "%s: depthwise stride 1 or 2, no dilation", who);
        NNHIP_REQUIRE(ctx, da->pad_h_before >= 0 && da->pad_h_after >= 0 && da->pad_w_before >= 0 && da->pad_w_after >= 0, -EINVAL,
                      "%s: negative padding", who);
        NNHIP_REQUIRE(ctx, da->in_h > 0 && da->in_w > 0, -EINVAL, "%s: non-positive input shape", who);
        const int out_h = windowed_output_size(da->in_h, 3, da->stride_h, 1, da->pad_h_before, da->pad_h_after);
        const int out_w = windowed_output_size(da->in_w, 3, da->stride_w, 1, da->pad_w_before, da->pad_w_after);
        NNHIP_REQUIRE(ctx, da->batch == fa->batch && out_h == fa->in_h && out_w == fa->in_w, -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                      "%s: the depthwise convolution writes [%d,%d,%d], the first 1x1 convolution reads [%d,%d,%d]", who, da->batch, out_h, out_w,
                      fa->batch, fa->in_h, fa->in_w);
        NNHIP_REQUIRE(ctx, da->y_qp.zero_point == fa->x_qp.zero_point && da->y_qp.scale == fa->x_qp.scale, -EINVAL,
                      "%s: the first 1x1 convolution must read the depthwise result with the quantisation it is written with", who);
        NNHIP_REQUIRE(ctx, (int64_t)da->batch * da->in_h * da->in_w * pr->k1 < ((int64_t)1 << 31), -EINVAL, "%s: input of 2 GiB or more", who);
        a.dw_w = reinterpret_cast<const int16_t *>(dw->d_packed), a.dw_bias = dw->d_bias, a.dw_wsum = dw->d_wsum;
        a.in_h = da->in_h, a.in_w = da->in_w, a.out_w = out_w, a.out_hw = out_h * out_w;
        a.stride = da->stride_h, a.pad_h = da->pad_h_before, a.pad_w = da->pad_w_before;
        a.d_out_hw = make_fastdiv((uint32_t)a.out_hw), a.d_out_w = make_fastdiv((uint32_t)out_w);
        a.dw_zx = da->x_qp.zero_point;
        rc = make_epilogue(ctx, &a.ep_dw, da->x_qp.scale, dw->sw, da->y_qp, da->clamp_min, da->clamp_max, NNCASE_HIP_DT_U8, who);
        if (rc) return rc;
    }

    // A wave per channel tile of whichever convolution has more of them in this workgroup (up to the variant's most),
    // and enough workgroups to occupy the device: pixel tiles x ranges of the second convolution's channel tiles.  With
    // a depthwise stage, also enough threads that none of them walks more than four of the 16 pixels.
    const bool small = pair_is_small(a.ks1, a.ks2);
    const int max_waves = small ? 16 : 12;
    const int ptiles = (a.m + 15) / 16;
    int ranges = (a.t2 + max_waves - 1) / max_waves;
    const int want = ptiles >= 512 ? 1 : 512 / ptiles;
    if (ranges > want) ranges = want;
    a.tiles_per_block = (a.t2 + ranges - 1) / ranges;
    ranges = (a.t2 + a.tiles_per_block - 1) / a.tiles_per_block;
    int waves = std::min(max_waves, std::max(a.t1, a.tiles_per_block));
    if (dw) waves = std::min(max_waves, std::max(waves, (a.k1 + 63) / 64));
    {
        // ... but no more than lets every workgroup be resident at once (a second round of workgroups doubles the
        // launch's latency chain; a wave that takes two channel tiles one after the other adds a fraction of it)
        const int occupancy = small ? (dw ? 4 : 5) : 3; // waves per SIMD the variant is built for
        const int per_cu = (ptiles * ranges + ctx->compute_units - 1) / std::max(ctx->compute_units, 1);
        waves = std::max(1, std::min(waves, 4 * occupancy / std::max(per_cu, 1)));
    }
    NNHIP_HIP(ctx, hipSetDevice(ctx->device));
    const dim3 grid(ptiles, ranges), block(waves * 64);
    const size_t lds = pair_lds_bytes(pr);
    if (small && dw)
        hipLaunchKernelGGL((qpointwise_pair_kernel<4, 2, 16, 4, true>), grid, block, lds, ctx->stream, a);
    else if (small)
        hipLaunchKernelGGL((qpointwise_pair_kernel<4, 2, 16, 5, false>), grid, block, lds, ctx->stream, a);
    else if (dw)
        hipLaunchKernelGGL((qpointwise_pair_kernel<8, 4, 12, 3, true>), grid, block, lds, ctx->stream, a);
    else
        hipLaunchKernelGGL((qpointwise_pair_kernel<8, 4, 12, 3, false>), grid, block, lds, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "qpointwise_pair_kernel");
    return 0;
}

extern "C" int nncase_hip_qpointwise_pair(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_qpair_t *pair, uint8_t *y1_dev,
                                          uint8_t *y2_dev, const nncase_hip_conv2d_args_t *first_args,
                                          const nncase_hip_conv2d_args_t *second_args) {
    NNHIP_CHECK_CTX(ctx);
    return launch_pair(ctx, "qpointwise_pair", x_dev, nullptr, nullptr, pair, y1_dev, y2_dev, first_args, second_args);
}

extern "C" int nncase_hip_qdepthwise_pointwise_pair(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_weights_t *depthwise,
                                                    const nncase_hip_conv2d_args_t *depthwise_args, const nncase_hip_qpair_t *pair,
                                                    uint8_t *y1_dev, uint8_t *y2_dev, const nncase_hip_conv2d_args_t *first_args,
                                                    const nncase_hip_conv2d_args_t *second_args) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, depthwise && depthwise_args, -EINVAL, "qdepthwise_pointwise_pair: null argument");
    return launch_pair(ctx, "qdepthwise_pointwise_pair", x_dev, depthwise, depthwise_args, pair, y1_dev, y2_dev, first_args, second_args);
}
