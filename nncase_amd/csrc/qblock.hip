// Fused inverted-residual block: 1x1 expansion -> 3x3 depthwise -> 1x1 projection (+ input),
// u8/u8, NHWC, one kernel.  The two expanded tensors are the largest of the block (6x the
// input) and, run as three operators, are each written to and read back from HBM; here a
// workgroup (8 or 16 waves) owns a 7x7 tile of OUTPUT pixels of one image and keeps everything
// between the block's input and output in LDS:
//
//   input tile   the in-image part of the (6S+3)^2 input pixels the tile needs, as s8
//   per chunk of 64 expanded channels:
//     E  expansion on the matrix cores for every in-image pixel of the halo, requantised to
//        u8 (kept as s8) into the expansion tile; positions outside the image keep the zero
//        point the tile was initialised with: they are the depthwise stage's padding
//     D  depthwise 3x3 on the matrix cores as well: the reduction index is (tap, channel) and
//        the weight operand is zero off its own channel; requantised into the depthwise tile
//     P  projection: the depthwise tile is one k-step of the matrix-core reduction over the
//        expanded channels, accumulated in registers across the chunks
//   epilogue of P: zero points, requantisation, optional residual add, NHWC store.
//
// The stages are software-pipelined over the chunks: between two barriers a workgroup runs
// E of chunk r, D of chunk r - 1 and P of chunk r - 2 on double-buffered tiles, and the
// constants travel global -> registers -> the other half of a double-buffered LDS area two
// steps ahead of their use (one step is shorter than a memory round trip).
//
// Every stage uses the arithmetic of the stand-alone kernels (same zero-point identity, same
// fp32 requantisation sequence), so the output bytes equal those of three separate operators.
// Tiles need a one-pixel halo of the expansion around them (recomputed per tile: 81 pixels
// for 49 at stride 1, 225 input pixels for 49 outputs at stride 2).  What bounds the kernel is
// the requantisation arithmetic on the vector ALU (two u8 tensors are requantised that never
// leave the compute unit), not memory: it pays on mid-sized feature maps, where the separate
// operators are latency-bound launches.
#include "qconv_igemm.hpp"

#include <algorithm>
#include <new>
#include <vector>

struct nncase_hip_qblock_weights {
    int cin = 0, mid = 0, cout = 0;
    int ke = 0;      // k-steps of the expansion (ceil(cin / 64))
    int et = 0;      // 16-channel tiles per chunk of expanded channels
    int tpt = 0;     // 16-channel tiles of the projection's output held by every wave
    int nchunks = 0, chunk_bytes = 0;
    int off_p = 0, off_wd = 0, off_bd = 0, off_sd = 0, off_be = 0, off_se = 0; // byte offsets inside a chunk
    int32_t zw_e = 0, zw_d = 0, zw_p = 0;
    float sw_e = 1.f, sw_d = 1.f, sw_p = 1.f;
    void *d_blob = nullptr;      // [nchunks][chunk_bytes]
    int32_t *d_wsum_p = nullptr; // [cout]
    int32_t *d_bias_p = nullptr; // [cout]
};

namespace nnhip {

constexpr int kBlkTile = 7;  // output tile edge (divides every MobileNet resolution from 112 down to 7)
constexpr int kBlkRowB = 80; // bytes per pixel of the two mid tiles: 64 channels + 16 so that rows spread over the banks

struct BlockArgs {
    const uint8_t *x;
    const uint8_t *blob;
    int chunk_bytes, nchunks;
    int cin, mid, ke;
    int xs; // bytes per pixel of the input tile (ke * 64 + 16)
    int in_h, in_w, out_h, out_w, pad_h, pad_w, tiles_y, tiles_x;
    int zxp_e, zwp_e, kzz_e; // expansion: zx - 128, zw - 128, cin * zxp * zwp
    int zxp_d, zwp_d, kzz_d; // depthwise: zx - 128, zw - 128, 9 * zxp * zwp
    uint32_t zmid_splat;     // zero point of the expansion's output as s8, in all four bytes
    Epilogue ep_e, ep_d;
    int off_p, off_wd, off_bd, off_sd, off_be, off_se;
    int lds_pix, lds_xin, lds_et, lds_dt, lds_w;
    IgemmArgs p; // projection stage: y, m, n, k, ldy, zxp, zwp, wsum, bias, ep, rep
};

// What the expansion needs to know about one in-image halo pixel: where its row of the expansion tile
// starts and the zero-point term of its sum of inputs.
struct HaloPix {
    int32_t tile_off; // byte offset of the pixel's row in the expansion tile
    int32_t nrsz;     // cin * zx' * zw' - zw' * sum_k x'
};

// NW = waves per workgroup: 8, or 16 for launches of few workgroups (one per compute unit or less), where the
// stages are chains of LDS and matrix-core round trips and more, shorter chains per SIMD hide them better.
template <int S, int TPT, int NW>
__global__ __launch_bounds__(NW * 64) void qblock_kernel(const BlockArgs a) {
    constexpr int kBlkWaves = NW, kBlkThreads = NW * 64;
    constexpr int NQ = NW / 4; // waves per channel tile = pixel-group phases
    constexpr int ET = 4;                      // 16-channel tiles per chunk of expanded channels
    constexpr int HH = (kBlkTile - 1) * S + 3; // halo edge in input pixels
    constexpr int HP = HH * HH;
    constexpr int TP = kBlkTile * kBlkTile;
    constexpr int CE = ET * 16;
    constexpr int NG = (HP + 15) / 16;                        // pixel groups of the halo at most
    constexpr int MAXU = (NG + NQ - 1) / NQ;                  // expansion units (16 pixels x 16 channels) per wave at most
    constexpr int DU = 4 / NQ;                                // depthwise units per wave
    constexpr int NS = (3 * ET * 1024 + TPT * 1024 + 9 * CE + 16 * CE + 16 * kBlkThreads - 1) / (16 * kBlkThreads); // vectors staged per thread
    constexpr int NSPLIT = (NW == 16 && TPT % 4 == 0) ? 4 : 2; // waves that share a projection pixel group
    constexpr int TPW = TPT / NSPLIT;                          // projection tiles per wave
    static_assert(TPT % 2 == 0 && (NW == 8 || NW == 16), "four channel tiles per chunk, 2 or 4 waves per tile");

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    int32_t *cterm_p = reinterpret_cast<int32_t *>(smem);             // [TPT * 16]
    HaloPix *hpix = reinterpret_cast<HaloPix *>(smem + a.lds_pix);   // [groups * 16]
    uint8_t *xin = smem + a.lds_xin;                                 // [groups * 16][xs] s8
    uint8_t *etile = smem + a.lds_et;                                // [2][HP][kBlkRowB] s8
    uint8_t *dtile = smem + a.lds_dt;                                // [2][64][kBlkRowB] s8
    uint8_t *wbuf = smem + a.lds_w;                                  // [2][chunk_bytes]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 15, gq = lane >> 4;
    // Every stage gives a wave one 16-channel tile (wave & 3) of half of the pixel groups (wave >> 2).
    const int wtile = wave & 3, whalf = wave >> 2; // whalf: 0 .. NQ - 1

    uint32_t b = blockIdx.x;
    const int tx = (int)(b % (uint32_t)a.tiles_x);
    b /= (uint32_t)a.tiles_x;
    const int ty = (int)(b % (uint32_t)a.tiles_y);
    const int img = (int)(b / (uint32_t)a.tiles_y);
    const int oy0 = ty * kBlkTile, ox0 = tx * kBlkTile;
    const int iy0 = oy0 * S - a.pad_h, ix0 = ox0 * S - a.pad_w; // halo origin in input coordinates
    // the part of the halo that lies inside the image
    const int cy0 = max(iy0, 0), cy1 = min(iy0 + HH, a.in_h);
    const int cx0 = max(ix0, 0), cx1 = min(ix0 + HH, a.in_w);
    const int CW = max(cx1 - cx0, 1);
    const int cnt = max(cy1 - cy0, 0) * max(cx1 - cx0, 0);
    const int offy = cy0 - iy0, offx = cx0 - ix0;
    const uint32_t rcw = 65536u / (uint32_t)CW + 1u; // idx / CW = (idx * rcw) >> 16 for idx < 256
    const int ngroups = (cnt + 15) >> 4;
    const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};

    // ---- one-time fills ---------------------------------------------------------------------------
    // Every global load of the set-up (input tile, constants, first chunk of weights) is issued before
    // anything waits for one of them: a dependent load -> store pair per loop trip would expose a full
    // memory round trip each time.
    const int nvec = a.chunk_bytes / 16;
    {
        constexpr int NPI = (NG * 16 + kBlkThreads / 16 - 1) / (kBlkThreads / 16); // pixels per thread
        const int ps = tid >> 4, dl = tid & 15;
        uint32_t xv[NPI][3];
#pragma unroll
        for (int it = 0; it < NPI; it++) {
            const int idx = ps + it * (kBlkThreads / 16);
            const int cy = (int)(((uint32_t)idx * rcw) >> 16), cx = idx - cy * CW;
            const bool pix = idx < cnt;
            const uint32_t src = (uint32_t)((img * a.in_h + cy0 + (pix ? cy : 0)) * a.in_w + cx0 + (pix ? cx : 0)) * (uint32_t)a.cin;
#pragma unroll
            for (int s = 0; s < 3; s++) {
                const int d = s * 16 + dl;
                xv[it][s] = 0x80808080u;
                if (s < a.ke && pix && d * 4 < a.cin) xv[it][s] = *reinterpret_cast<const uint32_t *>(a.x + src + d * 4);
            }
        }
        u32x4 w0[NS];
        {
            const u32x4 *src = reinterpret_cast<const u32x4 *>(a.blob);
#pragma unroll
            for (int i = 0; i < NS; i++) {
                const int v = i * kBlkThreads + tid;
                w0[i] = src[v < nvec ? v : 0];
            }
        }
        int32_t cb = 0, cs = 0;
        if (tid < a.p.n) cb = a.p.bias[tid], cs = a.p.wsum[tid];

        const u32x4 z = {a.zmid_splat, a.zmid_splat, a.zmid_splat, a.zmid_splat};
        for (int i = tid; i < 2 * HP * (kBlkRowB / 16); i += kBlkThreads) reinterpret_cast<u32x4 *>(etile)[i] = z;
        const u32x4 zero = {0, 0, 0, 0};
        for (int i = tid; i < 2 * 64 * (kBlkRowB / 16); i += kBlkThreads) reinterpret_cast<u32x4 *>(dtile)[i] = zero;

        if (tid < TPT * 16) cterm_p[tid] = tid < a.p.n ? cb - a.p.zxp * cs + a.p.k * a.p.zxp * a.p.zwp : 0;
        // input tile: 16 lanes hold one pixel's channels a dword each; re-biased to s8, zero past the channels
#pragma unroll
        for (int it = 0; it < NPI; it++) {
            const int idx = ps + it * (kBlkThreads / 16);
            if (idx < ngroups * 16) {
#pragma unroll
                for (int s = 0; s < 3; s++)
                    if (s < a.ke) *reinterpret_cast<uint32_t *>(xin + idx * a.xs + (s * 16 + dl) * 4) = xv[it][s] ^ 0x80808080u;
            }
        }
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const int v = i * kBlkThreads + tid;
            if (v < nvec) reinterpret_cast<u32x4 *>(wbuf)[v] = w0[i];
        }
    }
    __syncthreads();
    // per halo pixel: row offset in the expansion tile and the zero-point term of its input sum
    for (int g = wave; g < ngroups; g += kBlkWaves) {
        const int idx = g * 16 + j;
        v4i rs = {0, 0, 0, 0};
        for (int ks = 0; ks < a.ke; ks++) {
            const v4i xf = *reinterpret_cast<const v4i *>(xin + idx * a.xs + ks * 64 + gq * 16);
            rs = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, xf, rs, 0, 0, 0);
        }
        if (gq == 0) {
            const int cy = (int)(((uint32_t)idx * rcw) >> 16), cx = idx - cy * CW;
            HaloPix hp;
            hp.tile_off = idx < cnt ? ((cy + offy) * HH + cx + offx) * kBlkRowB : -1;
            hp.nrsz = a.kzz_e - a.zwp_e * rs[0];
            hpix[idx] = hp;
        }
    }
    __syncthreads();

    // ---- what stays the same for every chunk -------------------------------------------------------------------
    // E: the wave's units are pixel groups whalf, whalf + NQ, ... of channel tile wtile (their halo records are read
    // from LDS where they are used)
    const uint8_t *exrow = xin + (whalf * 16 + j) * a.xs + gq * 16; // + k * 32 * xs + ks * 64
    const int ecl = gq * (4 * ET) + wtile * 4;                        // the lane's 4 channels within the chunk
    // D: pixel groups whalf (+ NQ ...) of channel tile wtile; the lane's tap in k-step ks is ks * 4 + gq
    int dxoff[DU], dtap[3];
    bool dpv[DU];
#pragma unroll
    for (int k = 0; k < DU; k++) {
        const int pp = (whalf + NQ * k) * 16 + j;
        dpv[k] = pp < TP;
        const int p = min(pp, TP - 1);
        const int py = p / kBlkTile, px = p - py * kBlkTile;
        dxoff[k] = ((py * S) * HH + px * S) * kBlkRowB + wtile * 16;
    }
#pragma unroll
    for (int ks = 0; ks < 3; ks++) {
        const int t = ks * 4 + gq;
        const int tt = t < 9 ? t : 0;
        const int ky = tt / 3, kx = tt - ky * 3;
        dtap[ks] = (ky * HH + kx) * kBlkRowB;
    }
    // byte j of the 16-byte k-chunk belongs to channel j of the tile: a mask for the weight, a one for the window sum
    u32x4 dmask, done;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        dmask[d] = (j >> 2) == d ? 0xffu << (8 * (j & 3)) : 0u;
        done[d] = dmask[d] & 0x01010101u;
    }
    const v4i done_f = __builtin_bit_cast(v4i, done);
    const v4i done_last = gq == 0 ? done_f : v4i{0, 0, 0, 0}; // k-step 2 only holds tap 8
    const int dcl = wtile * 16 + gq * 4; // the lane's 4 channels within the chunk

    v4i accp[TPW];
    v4i rsp = {0, 0, 0, 0};
#pragma unroll
    for (int nt = 0; nt < TPW; nt++) accp[nt] = v4i{0, 0, 0, 0};

    // Record r of the constants holds the expansion weights of chunk r, the depthwise weights of chunk r - 1 and
    // the projection weights of chunk r - 2: phase r runs E(r), D(r - 1) and P(r - 2) between two barriers, on
    // double-buffered tiles, so the three stages of different chunks overlap inside the workgroup.
    // The constants travel global -> registers -> LDS two phases ahead of their use (one phase is shorter than a
    // memory round trip): record r + 1 is committed to the other half of the LDS area at the end of phase r from
    // the register set it was loaded into at the end of phase r - 2, and that set is reloaded with record r + 3.
    // The loads are unconditional (a record index past the end re-reads the last one) so that the number of
    // younger loads in flight is a compile-time constant and waiting for one set does not drain the other.
    const int nrec = a.nchunks + 2;
    u32x4 stage_a[NS], stage_b[NS];
    auto issue = [&](int rec, u32x4 (&st)[NS]) {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(a.blob + (size_t)min(rec, nrec - 1) * a.chunk_bytes);
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const int v = i * kBlkThreads + tid;
            st[i] = src[v < nvec ? v : 0];
        }
    };
    auto commit = [&](int rec, const u32x4 (&st)[NS]) {
        if (rec < nrec) {
            u32x4 *dst = reinterpret_cast<u32x4 *>(wbuf + (rec & 1) * a.chunk_bytes);
#pragma unroll
            for (int i = 0; i < NS; i++) {
                const int v = i * kBlkThreads + tid;
                if (v < nvec) dst[v] = st[i];
            }
        }
    };
    issue(1, stage_a);
    issue(2, stage_b);
    auto phase = [&](int r) {
        const uint8_t *wb = wbuf + (r & 1) * a.chunk_bytes;

        // ---- P(r - 2): one k-step of the projection ----------------------------------------------------------
        if (r >= 2 && whalf < NSPLIT) {
            const v4i xf = *reinterpret_cast<const v4i *>(dtile + (r & 1) * (64 * kBlkRowB) + (wtile * 16 + j) * kBlkRowB + gq * 16);
            rsp = __builtin_amdgcn_mfma_i32_16x16x64_i8(ones, xf, rsp, 0, 0, 0);
            const uint8_t *wfr = wb + a.off_p + whalf * (TPW * 1024) + lane * 16;
#pragma unroll
            for (int nt = 0; nt < TPW; nt++) {
                const v4i wf = *reinterpret_cast<const v4i *>(wfr + nt * 1024);
                accp[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf, xf, accp[nt], 0, 0, 0);
            }
        }

        // ---- E(r): expansion of the in-image halo pixels, 16 pixels x 16 channels per unit ---------------------
        if (r < a.nchunks) {
            uint8_t *et = etile + (r & 1) * (HP * kBlkRowB);
            v4i wf[3];
#pragma unroll
            for (int ks = 0; ks < 3; ks++)
                if (ks < a.ke) wf[ks] = *reinterpret_cast<const v4i *>(wb + (ks * ET + wtile) * 1024 + lane * 16);
            const v4i be = *reinterpret_cast<const v4i *>(wb + a.off_be + ecl * 4);
            const v4i se = *reinterpret_cast<const v4i *>(wb + a.off_se + ecl * 4);
            int32_t cst[4];
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) cst[r4] = be[r4] - a.zxp_e * se[r4];
#pragma unroll
            for (int k = 0; k < MAXU; k++) {
                if (whalf + NQ * k < ngroups) {
                    v4i acc = {0, 0, 0, 0};
#pragma unroll
                    for (int ks = 0; ks < 3; ks++)
                        if (ks < a.ke) {
                            const v4i xf = *reinterpret_cast<const v4i *>(exrow + k * (NQ * 16) * a.xs + ks * 64);
                            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[ks], xf, acc, 0, 0, 0);
                        }
                    const HaloPix hpk = hpix[(whalf + NQ * k) * 16 + j];
                    int32_t v4[4];
#pragma unroll
                    for (int r4 = 0; r4 < 4; r4++) v4[r4] = add3(acc[r4], cst[r4], hpk.nrsz);
                    const uint32_t q = requant4_u8_packed(v4, a.ep_e);
                    if (hpk.tile_off >= 0) *reinterpret_cast<uint32_t *>(et + hpk.tile_off + ecl) = q ^ 0x80808080u;
                }
            }
        }

        // ---- D(r - 1): depthwise 3x3 on the matrix cores: 16 pixels x 16 channels per unit --------------------------
        // The reduction index is (tap, channel): a 16-byte k-chunk of the pixel operand is one tap's 16 channels
        // (one LDS read), and the weight operand carries w' = w - 128 of channel i at byte i of the chunk and
        // zeros elsewhere, so row i of the product only sees its own channel.  A second product against ones in
        // the same places gives the window sum of x', which the weight zero point multiplies:
        //   sum (x - zx)(w - zw) = sum x'w' - zw' * sum x' - zx' * sum w' + 9 zx' zw'.
        if (r >= 1 && r <= a.nchunks) {
            const uint8_t *et = etile + ((r - 1) & 1) * (HP * kBlkRowB);
            uint8_t *dt = dtile + ((r - 1) & 1) * (64 * kBlkRowB);
            v4i wfr[3];
#pragma unroll
            for (int ks = 0; ks < 3; ks++) {
                const int t = ks * 4 + gq;
                const uint32_t wbyte = t < 9 ? (uint32_t)wb[a.off_wd + t * CE + wtile * 16 + j] : 0u;
                const uint32_t splat = wbyte * 0x01010101u;
                wfr[ks] = __builtin_bit_cast(v4i, u32x4{dmask[0] & splat, dmask[1] & splat, dmask[2] & splat, dmask[3] & splat});
            }
            const v4i bd = *reinterpret_cast<const v4i *>(wb + a.off_bd + dcl * 4);
            const v4i sd = *reinterpret_cast<const v4i *>(wb + a.off_sd + dcl * 4);
            int32_t ct[4];
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) ct[r4] = bd[r4] - a.zxp_d * sd[r4] + a.kzz_d;
            const bool chv = (r - 1) * CE + dcl < a.mid;
#pragma unroll
            for (int k = 0; k < DU; k++) {
                const uint8_t *xb = et + dxoff[k];
                v4i aw = {0, 0, 0, 0}, a1 = {0, 0, 0, 0};
#pragma unroll
                for (int ks = 0; ks < 3; ks++) {
                    const v4i xf = *reinterpret_cast<const v4i *>(xb + dtap[ks]);
                    aw = __builtin_amdgcn_mfma_i32_16x16x64_i8(wfr[ks], xf, aw, 0, 0, 0);
                    a1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(ks == 2 ? done_last : done_f, xf, a1, 0, 0, 0);
                }
                int32_t v4[4];
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) v4[r4] = aw[r4] - a.zwp_d * a1[r4] + ct[r4];
                const uint32_t packed = requant4_u8_packed(v4, a.ep_d) ^ 0x80808080u; // kept as s8
                if (dpv[k]) *reinterpret_cast<uint32_t *>(dt + ((whalf + NQ * k) * 16 + j) * kBlkRowB + dcl) = chv ? packed : 0u;
            }
        }

    };
    for (int r = 0; r < nrec; r += 2) {
        phase(r);
        commit(r + 1, stage_a);
        issue(r + 3, stage_a);
        __syncthreads();
        if (r + 1 < nrec) {
            phase(r + 1);
            commit(r + 2, stage_b);
            issue(r + 4, stage_b);
            __syncthreads();
        }
    }

    // ---- epilogue of the projection: pixel group wtile, the wave's TPW tiles are 4 * TPW consecutive channels per lane ----
    const int pl = wtile * 16 + j;
    const int py = pl / kBlkTile, px = pl - py * kBlkTile;
    const int oy = oy0 + py, ox = ox0 + px;
    const bool valid = pl < TP && oy < a.out_h && ox < a.out_w;
    const int pg = valid ? (img * a.out_h + oy) * a.out_w + ox : a.p.m;
    const int ch0 = gq * (4 * TPT) + whalf * (4 * TPW);
    // igemm_store_tile reads its constants at cterm + gq * 4 * TPW + nt * 4; they sit at cterm_p + ch0 + nt * 4
    if (whalf < NSPLIT) igemm_store_tile<TPW>(a.p, accp, rsp[0], pg, ch0, gq, cterm_p + ch0 - gq * (4 * TPW), nullptr);
}

template <int S, int TPT, int NW> static int launch_block_inst(nncase_hip_ctx *ctx, const BlockArgs &a, int blocks, size_t lds) {
    // the dynamic LDS limit of a kernel is raised once per device (the attribute call is slow next to a launch)
    static int raised_on_device = -1;
    if (lds > 48 * 1024 && raised_on_device != ctx->device) {
        NNHIP_HIP(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(&qblock_kernel<S, TPT, NW>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        raised_on_device = ctx->device;
    }
    hipLaunchKernelGGL((qblock_kernel<S, TPT, NW>), dim3(blocks), dim3(NW * 64), lds, ctx->stream, a);
    NNHIP_LAUNCH_CHECK(ctx, "qblock_kernel");
    return 0;
}

// 16 waves when the launch has at most one workgroup per compute unit (and the projection is narrow enough for
// the register budget of 16 waves), else 8: measured, launches of two workgroups per compute unit run 20% longer
// with 16 waves than with 8.
static bool block_wide(const nncase_hip_ctx *ctx, int tpt, long long blocks) { return tpt <= 6 && blocks <= (long long)ctx->compute_units; }

template <int S> static int launch_block_s(nncase_hip_ctx *ctx, const BlockArgs &a, int tpt, int blocks, size_t lds) {
    const bool wide = block_wide(ctx, tpt, blocks);
    switch (tpt) {
    case 2: return wide ? launch_block_inst<S, 2, 16>(ctx, a, blocks, lds) : launch_block_inst<S, 2, 8>(ctx, a, blocks, lds);
    case 4: return wide ? launch_block_inst<S, 4, 16>(ctx, a, blocks, lds) : launch_block_inst<S, 4, 8>(ctx, a, blocks, lds);
    case 6: return wide ? launch_block_inst<S, 6, 16>(ctx, a, blocks, lds) : launch_block_inst<S, 6, 8>(ctx, a, blocks, lds);
    case 10: return launch_block_inst<S, 10, 8>(ctx, a, blocks, lds);
    default: return launch_block_inst<S, 20, 8>(ctx, a, blocks, lds);
    }
}

static int block_tiles(int cout) {
    const int t = ceil_div(cout, 16);
    for (int v : {2, 4, 6, 10, 20})
        if (v >= t) return v;
    return 0;
}

} // namespace nnhip

using namespace nnhip;

extern "C" int nncase_hip_qblock_supported(const nncase_hip_qblock_desc_t *d) {
    if (!d) return 0;
    return d->in_channels > 0 && d->in_channels % 4 == 0 && d->in_channels <= 192 && d->mid_channels > 0 &&
                   d->mid_channels % 4 == 0 && d->mid_channels < 65536 && d->out_channels > 0 && block_tiles(d->out_channels) > 0
               ? 1
               : 0;
}

void nncase_hip_qblock_describe(const nncase_hip_qblock_t *b, const nncase_hip_qblock_args_t *a, char *buf, size_t cap) {
    snprintf(buf, cap, "qblock%s<S=%d,P=%d>", a->add_input ? "+add" : "", a->stride, b->tpt);
}

static void free_block(nncase_hip_qblock_t *b) {
    if (!b) return;
    if (b->d_blob) (void)hipFree(b->d_blob);
    if (b->d_wsum_p) (void)hipFree(b->d_wsum_p);
    if (b->d_bias_p) (void)hipFree(b->d_bias_p);
    delete b;
}

extern "C" int nncase_hip_qblock_prepack(nncase_hip_ctx_t *ctx, const nncase_hip_qblock_desc_t *desc, const uint8_t *w_expand,
                                         const int32_t *bias_expand, const uint8_t *w_dw, const int32_t *bias_dw,
                                         const uint8_t *w_project, const int32_t *bias_project, nncase_hip_qblock_t **block) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, desc && w_expand && w_dw && w_project && block, -EINVAL, "qblock_prepack: null argument");
    *block = nullptr;
    NNHIP_REQUIRE(ctx, nncase_hip_qblock_supported(desc), -NNCASE_HIP_ERR_SHAPE_MISMATCH,
                  "qblock_prepack: channels %d -> %d -> %d are outside what the fused kernel is built for", desc->in_channels,
                  desc->mid_channels, desc->out_channels);
    for (const nncase_hip_quant_param_t *q : {&desc->expand_w_qp, &desc->dw_w_qp, &desc->project_w_qp})
        NNHIP_REQUIRE(ctx, q->zero_point >= 0 && q->zero_point <= 255, -EINVAL, "qblock_prepack: weight zero point %d outside u8",
                      q->zero_point);
    nncase_hip_qblock_t *b = new (std::nothrow) nncase_hip_qblock_t();
    NNHIP_REQUIRE(ctx, b, -ENOMEM, "qblock_prepack: out of host memory");
    const int cin = b->cin = desc->in_channels, mid = b->mid = desc->mid_channels, cout = b->cout = desc->out_channels;
    b->zw_e = desc->expand_w_qp.zero_point, b->sw_e = desc->expand_w_qp.scale;
    b->zw_d = desc->dw_w_qp.zero_point, b->sw_d = desc->dw_w_qp.scale;
    b->zw_p = desc->project_w_qp.zero_point, b->sw_p = desc->project_w_qp.scale;
    b->ke = ceil_div(cin, 64);
    b->et = 4;
    const int ce = b->et * 16;
    b->tpt = block_tiles(cout);
    b->nchunks = ceil_div(mid, ce);
    b->off_p = b->ke * b->et * 1024;
    b->off_wd = b->off_p + b->tpt * 1024;
    b->off_bd = b->off_wd + 9 * ce;
    b->off_sd = b->off_bd + ce * 4;
    b->off_be = b->off_sd + ce * 4;
    b->off_se = b->off_be + ce * 4;
    b->chunk_bytes = b->off_se + ce * 4;

    // record r: expansion part of chunk r, depthwise part of chunk r - 1, projection part of chunk r - 2
    std::vector<uint8_t> blob((size_t)(b->nchunks + 2) * b->chunk_bytes, 0);
    // expansion: [chunk][ks][tile] fragments, chunk = 16 * et channels
    {
        std::vector<uint8_t> frags((size_t)b->nchunks * b->ke * b->et * 1024);
        std::vector<int32_t> wsum(mid);
        pack_group(frags.data(), wsum.data(), mid, cin, b->ke, b->et, b->nchunks,
                   [&](int oc, int kk) -> uint8_t { return w_expand[(size_t)oc * cin + kk]; });
        for (int c = 0; c < b->nchunks; c++) {
            uint8_t *dst = blob.data() + (size_t)c * b->chunk_bytes;
            memcpy(dst, frags.data() + (size_t)c * b->ke * b->et * 1024, (size_t)b->ke * b->et * 1024);
            int32_t *be = reinterpret_cast<int32_t *>(dst + b->off_be), *se = reinterpret_cast<int32_t *>(dst + b->off_se);
            for (int i = 0; i < ce; i++) {
                const int ch = c * ce + i;
                be[i] = (ch < mid && bias_expand) ? bias_expand[ch] : 0;
                se[i] = ch < mid ? wsum[ch] : 0;
            }
        }
    }
    // projection: chunk c of the expanded channels is k-step c, channels past the chunk's width are zero weights
    std::vector<int32_t> wsum_p(cout), bias_p(cout, 0);
    {
        std::vector<uint8_t> frags((size_t)b->nchunks * b->tpt * 1024);
        pack_group(frags.data(), wsum_p.data(), cout, b->nchunks * 64, b->nchunks, b->tpt, 1, [&](int oc, int kk) -> uint8_t {
            const int ks = kk / 64, pos = kk % 64, ch = ks * ce + pos;
            return (pos < ce && ch < mid) ? w_project[(size_t)oc * mid + ch] : (uint8_t)0x80;
        });
        for (int c = 0; c < b->nchunks; c++)
            memcpy(blob.data() + (size_t)(c + 2) * b->chunk_bytes + b->off_p, frags.data() + (size_t)c * b->tpt * 1024, (size_t)b->tpt * 1024);
        if (bias_project) std::copy(bias_project, bias_project + cout, bias_p.begin());
    }
    // depthwise: w - 128 as s8 [tap][channel of the chunk], bias and tap sum of (w - 128) per channel
    for (int c = 0; c < b->nchunks; c++) {
        uint8_t *dst = blob.data() + (size_t)(c + 1) * b->chunk_bytes;
        uint8_t *wd = dst + b->off_wd;
        int32_t *bd = reinterpret_cast<int32_t *>(dst + b->off_bd), *sd = reinterpret_cast<int32_t *>(dst + b->off_sd);
        for (int i = 0; i < ce; i++) {
            const int ch = c * ce + i;
            int32_t s = 0;
            for (int t = 0; t < 9; t++) {
                const uint8_t v = ch < mid ? (uint8_t)(w_dw[(size_t)ch * 9 + t] ^ 0x80) : (uint8_t)0;
                wd[t * ce + i] = v;
                s += (int32_t)(int8_t)v;
            }
            bd[i] = (ch < mid && bias_dw) ? bias_dw[ch] : 0;
            sd[i] = s;
        }
    }
    hipError_t e = hipSetDevice(ctx->device);
    if (e == hipSuccess) e = hipMalloc(&b->d_blob, blob.size());
    if (e == hipSuccess) e = hipMalloc((void **)&b->d_wsum_p, sizeof(int32_t) * cout);
    if (e == hipSuccess) e = hipMalloc((void **)&b->d_bias_p, sizeof(int32_t) * cout);
    if (e == hipSuccess) e = hipMemcpy(b->d_blob, blob.data(), blob.size(), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(b->d_wsum_p, wsum_p.data(), sizeof(int32_t) * cout, hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(b->d_bias_p, bias_p.data(), sizeof(int32_t) * cout, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        free_block(b);
        return hip_fail(ctx, e, "qblock_prepack");
    }
    *block = b;
    return 0;
}

extern "C" int nncase_hip_qblock_destroy(nncase_hip_ctx_t *ctx, nncase_hip_qblock_t *block) {
    NNHIP_CHECK_CTX(ctx);
    if (!block) return 0;
    NNHIP_HIP(ctx, hipStreamSynchronize(ctx->stream));
    free_block(block);
    return 0;
}

extern "C" int nncase_hip_qblock(nncase_hip_ctx_t *ctx, const uint8_t *x_dev, const nncase_hip_qblock_t *blk, uint8_t *y_dev,
                                 const nncase_hip_qblock_args_t *g) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, x_dev && blk && y_dev && g, -EINVAL, "qblock: null argument");
    NNHIP_REQUIRE(ctx, g->batch > 0 && g->in_h > 0 && g->in_w > 0, -EINVAL, "qblock: non-positive input shape");
    NNHIP_REQUIRE(ctx, g->stride == 1 || g->stride == 2, -EINVAL, "qblock: depthwise stride %d (1 or 2)", g->stride);
    for (int pad : {g->pad_h_before, g->pad_h_after, g->pad_w_before, g->pad_w_after})
        NNHIP_REQUIRE(ctx, pad == 0 || pad == 1, -EINVAL, "qblock: depthwise padding %d (0 or 1)", pad);
    for (const nncase_hip_quant_param_t *q : {&g->x_qp, &g->expand_qp, &g->dw_qp})
        NNHIP_REQUIRE(ctx, q->zero_point >= 0 && q->zero_point <= 255, -EINVAL, "qblock: zero point %d outside u8", q->zero_point);
    const int out_h = windowed_output_size(g->in_h, 3, g->stride, 1, g->pad_h_before, g->pad_h_after);
    const int out_w = windowed_output_size(g->in_w, 3, g->stride, 1, g->pad_w_before, g->pad_w_after);
    NNHIP_REQUIRE(ctx, out_h > 0 && out_w > 0, -NNCASE_HIP_ERR_SHAPE_MISMATCH, "qblock: window larger than padded input");
    NNHIP_REQUIRE(ctx, !g->add_input || (g->stride == 1 && blk->cin == blk->cout && out_h == g->in_h && out_w == g->in_w),
                  -NNCASE_HIP_ERR_SHAPE_MISMATCH, "qblock: the residual needs an output of the input's shape");
    const int64_t m64 = (int64_t)g->batch * out_h * out_w;
    NNHIP_REQUIRE(ctx, m64 < ((int64_t)1 << 30) && (int64_t)g->batch * g->in_h * g->in_w * blk->cin < ((int64_t)1 << 31) &&
                           m64 * blk->cout < ((int64_t)1 << 31),
                  -EINVAL, "qblock: tensors of 2^31 bytes or more are not supported");
    NNHIP_REQUIRE(ctx, (reinterpret_cast<uintptr_t>(x_dev) & 15u) == 0 && (reinterpret_cast<uintptr_t>(y_dev) & 15u) == 0,
                  -NNCASE_HIP_ERR_INVALID_MEMORY_LOCATION, "qblock: activation buffers must be 16-byte aligned");

    BlockArgs a;
    memset(&a, 0, sizeof(a));
    a.x = x_dev;
    a.blob = reinterpret_cast<const uint8_t *>(blk->d_blob);
    a.chunk_bytes = blk->chunk_bytes;
    a.nchunks = blk->nchunks;
    a.cin = blk->cin;
    a.mid = blk->mid;
    a.ke = blk->ke;
    a.xs = blk->ke * 64 + 16;
    a.in_h = g->in_h, a.in_w = g->in_w, a.out_h = out_h, a.out_w = out_w;
    a.pad_h = g->pad_h_before, a.pad_w = g->pad_w_before;
    a.tiles_y = ceil_div(out_h, kBlkTile), a.tiles_x = ceil_div(out_w, kBlkTile);
    a.zxp_e = g->x_qp.zero_point - 128;
    a.zwp_e = blk->zw_e - 128;
    a.kzz_e = blk->cin * a.zxp_e * a.zwp_e;
    a.zxp_d = g->expand_qp.zero_point - 128;
    a.zwp_d = blk->zw_d - 128;
    a.kzz_d = 9 * a.zxp_d * a.zwp_d;
    a.zmid_splat = (uint32_t)((g->expand_qp.zero_point ^ 0x80) & 0xff) * 0x01010101u;
    int rc = make_epilogue(ctx, &a.ep_e, g->x_qp.scale, blk->sw_e, g->expand_qp, g->expand_clamp_min, g->expand_clamp_max,
                           NNCASE_HIP_DT_U8, "qblock(expand)");
    if (rc) return rc;
    rc = make_epilogue(ctx, &a.ep_d, g->expand_qp.scale, blk->sw_d, g->dw_qp, g->dw_clamp_min, g->dw_clamp_max, NNCASE_HIP_DT_U8,
                       "qblock(depthwise)");
    if (rc) return rc;
    a.off_p = blk->off_p, a.off_wd = blk->off_wd, a.off_bd = blk->off_bd, a.off_sd = blk->off_sd, a.off_be = blk->off_be,
    a.off_se = blk->off_se;
    a.p.y = y_dev;
    a.p.m = (int)m64;
    a.p.n = blk->cout;
    a.p.k = blk->mid;
    a.p.ldy = a.p.ldr = blk->cout;
    a.p.zxp = g->dw_qp.zero_point - 128;
    a.p.zwp = blk->zw_p - 128;
    a.p.wsum = blk->d_wsum_p;
    a.p.bias = blk->d_bias_p;
    rc = make_epilogue(ctx, &a.p.ep, g->dw_qp.scale, blk->sw_p, g->y_qp, g->clamp_min, g->clamp_max, NNCASE_HIP_DT_U8, "qblock(project)");
    if (rc) return rc;
    {
        nncase_hip_conv2d_args_t c;
        memset(&c, 0, sizeof(c));
        c.out_dtype = NNCASE_HIP_DT_U8;
        c.y_qp = g->y_qp;
        if (g->add_input) {
            NNHIP_REQUIRE(ctx, g->sum_qp.scale > 0.f && std::isfinite(g->sum_qp.scale) && g->sum_qp.zero_point >= 0 &&
                                   g->sum_qp.zero_point <= 255,
                          -EINVAL, "qblock: quant param of the sum outside u8 / positive scale");
            c.residual_dev = x_dev;
            c.residual_qp = g->x_qp;
            c.sum_qp = g->sum_qp;
            c.sum_clamp_min = g->sum_clamp_min;
            c.sum_clamp_max = g->sum_clamp_max;
        }
        rc = make_residual_epilogue(ctx, &a.p.rep, &c, nullptr);
        if (rc) return rc;
    }
    const int hh = (kBlkTile - 1) * g->stride + 3, hp = hh * hh;
    const int cterm_bytes = blk->tpt * 16 * 4;
    a.lds_pix = cterm_bytes;
    a.lds_xin = a.lds_pix + ceil_div(hp, 16) * 16 * (int)sizeof(HaloPix);
    a.lds_et = a.lds_xin + ceil_div(hp, 16) * 16 * a.xs;
    a.lds_dt = a.lds_et + 2 * hp * kBlkRowB;
    a.lds_w = a.lds_dt + 2 * 64 * kBlkRowB;
    const size_t lds = (size_t)a.lds_w + 2 * (size_t)blk->chunk_bytes;
    NNHIP_REQUIRE(ctx, lds <= 160 * 1024, -EINVAL, "qblock: %zu bytes of LDS needed", lds);
    const int64_t blocks = (int64_t)g->batch * a.tiles_y * a.tiles_x;
    NNHIP_REQUIRE(ctx, blocks < ((int64_t)1 << 31), -EINVAL, "qblock: too many tiles");
    NNHIP_HIP(ctx, hipSetDevice(ctx->device));
    return g->stride == 1 ? launch_block_s<1>(ctx, a, blk->tpt, (int)blocks, lds) : launch_block_s<2>(ctx, a, blk->tpt, (int)blocks, lds);
}
