// Pure data-movement kernels: pack / unpack (lane-blocked layouts) and the
// NCHW <-> NHWC relayout.  All are permutations with optional zero padding,
// bound by HBM bandwidth.  Where the innermost dimension of the packed tensor
// runs against the innermost axis of the plain one (the layouts matrix
// operands want, and the relayout of narrow elements) a block moves a tile
// through LDS with dword accesses on both sides (pack_tile_kernel); every
// other permutation has a thread produce one output element -- a 16- or
// 4-byte group of elements where the two innermost dimensions coincide -- so
// that writes are coalesced; 4-byte transposes go through a 32 x 33 LDS tile.
#include "common.hpp"

#include <algorithm>
#include <type_traits>

namespace nnhip {

constexpr int kMaxRank = 8;
constexpr int kLayoutThreads = 256;

struct PackDesc {
    int out_rank;                 // rank of the tensor being written
    uint32_t out_dims[2 * kMaxRank];
    // pack: output dim k adds coord * mul[k] to input axis axis[k]
    // unpack: output dim d reads packed outer dim d and, if lanes[d] > 1, lane dim lane_dim[d]
    int axis[2 * kMaxRank];
    uint32_t mul[2 * kMaxRank];
    uint32_t in_dims[2 * kMaxRank];
    uint64_t in_strides[2 * kMaxRank];
    uint32_t lanes[kMaxRank];
    int lane_dim[kMaxRank];
    int in_rank;
    uint64_t total;
    FastDiv out_div[2 * kMaxRank]; // of out_dims (the SMALL kernels: fewer than 2^31 output elements)
};

// SMALL: fewer than 2^31 output elements, so that the coordinates come from 32-bit multiply-shift divisions.
template <typename T, bool SMALL> __global__ __launch_bounds__(kLayoutThreads) void pack_kernel(const T *in, T *out, const PackDesc d) {
    const uint64_t gid = (uint64_t)blockIdx.x * kLayoutThreads + threadIdx.x;
    if (gid >= d.total) return;
    uint32_t coord[kMaxRank];
#pragma unroll
    for (int i = 0; i < kMaxRank; i++) coord[i] = 0;
    if constexpr (SMALL) {
        uint32_t rem = (uint32_t)gid;
        for (int k = d.out_rank - 1; k >= 0; k--) {
            const uint32_t q = fastdiv(rem, d.out_div[k]);
            coord[d.axis[k]] += (rem - q * d.out_dims[k]) * d.mul[k];
            rem = q;
        }
    } else {
        uint64_t rem = gid;
        for (int k = d.out_rank - 1; k >= 0; k--) {
            const uint32_t c = (uint32_t)(rem % d.out_dims[k]);
            rem /= d.out_dims[k];
            coord[d.axis[k]] += c * d.mul[k];
        }
    }
    bool ok = true;
    uint64_t off = 0;
    for (int i = 0; i < d.in_rank; i++) {
        ok = ok && coord[i] < d.in_dims[i];
        off += (uint64_t)coord[i] * d.in_strides[i];
    }
    out[gid] = ok ? in[off] : (T)0;
}

// Pixels of c <= 4 elements -> 4-byte pixels, the missing channels zero; with FOLD = 2 the four pixels of a 2 x 2
// block become one 16-byte pixel of the half-size image, (dy, dx) major: out[n][y][x] = {in[n][2y][2x], in[n][2y][2x+1],
// in[n][2y+1][2x], in[n][2y+1][2x+1]}, which is what pack by lanes (2, 2, 4) on the (H, W, C) axes of an NHWC tensor
// writes.  Float input is quantised to u8 on the way (Quantize, then Pack, in one pass).  One thread per output pixel;
// rows counts image rows over the whole batch (H is even, so a block never straddles two images).
template <typename TIn> __device__ __forceinline__ uint32_t pixel_to_dword(const TIn *p, int c, float scale, float bias) {
    uint32_t v = 0;
    for (int i = 0; i < c; i++) {
        uint32_t b;
        if constexpr (std::is_same<TIn, float>::value) b = quantize_one<uint8_t>(p[i], scale, bias);
        else b = p[i];
        v |= b << (8 * i);
    }
    return v;
}

template <typename TIn, int FOLD>
__global__ __launch_bounds__(kLayoutThreads) void pack_pixels_kernel(const TIn *__restrict__ in, uint32_t *__restrict__ out, uint32_t total,
                                                                   uint32_t w_out, FastDiv d_w, int c, float scale, float bias) {
    const uint32_t gid = blockIdx.x * kLayoutThreads + threadIdx.x;
    if (gid >= total) return;
    if constexpr (FOLD == 1) {
        out[gid] = c == 3 ? pixel_to_dword(in + (size_t)gid * 3, 3, scale, bias) : pixel_to_dword(in + (size_t)gid * c, c, scale, bias);
    } else {
        const uint32_t r = fastdiv(gid, d_w), x = gid - r * w_out;
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        u32x4 v;
#pragma unroll
        for (int dy = 0; dy < 2; dy++) {
            const size_t pix = (size_t)(2 * r + dy) * (2 * w_out) + 2 * x;
            if (c == 3) { // (the uniform special case lets the loads of a row's six elements be scheduled together)
                TIn e[6];
#pragma unroll
                for (int i = 0; i < 6; i++) e[i] = in[pix * 3 + i];
                v[dy * 2] = pixel_to_dword(e, 3, scale, bias);
                v[dy * 2 + 1] = pixel_to_dword(e + 3, 3, scale, bias);
            } else {
                v[dy * 2] = pixel_to_dword(in + pix * c, c, scale, bias);
                v[dy * 2 + 1] = pixel_to_dword(in + (pix + 1) * c, c, scale, bias);
            }
        }
        reinterpret_cast<u32x4 *>(out)[gid] = v;
    }
}

// The two layouts the stem convolutions read: NHWC with <= 4 channels packed by (4) on C or by (2, 2, 4) on (H, W, C).
// Returns 1 when the arguments are neither.
template <typename TIn>
static int launch_pack_pixels(nncase_hip_ctx *ctx, const TIn *in, void *out, int rank, const int32_t *shape, int n_axes, const int *nax,
                              const int32_t *lanes, float scale, float bias) {
    if (shape[rank - 1] > 4 || (reinterpret_cast<uintptr_t>(out) & 15u) != 0) return 1;
    uint64_t rows = 1;
    for (int i = 0; i < rank - 1; i++) rows *= (uint64_t)shape[i];
    const int c = shape[rank - 1];
    if (n_axes == 1 && nax[0] == rank - 1 && lanes[0] == 4) {
        NNHIP_REQUIRE(ctx, rows < ((uint64_t)1 << 31), -EINVAL, "pack: tensor too large");
        if (rows == 0) return 0;
        hipLaunchKernelGGL((pack_pixels_kernel<TIn, 1>), dim3((unsigned)((rows + kLayoutThreads - 1) / kLayoutThreads)), dim3(kLayoutThreads),
                           0, ctx->stream, in, (uint32_t *)out, (uint32_t)rows, 1u, make_fastdiv(1), c, scale, bias);
        NNHIP_LAUNCH_CHECK(ctx, "pack_pixels_kernel");
        return 0;
    }
    if (rank == 4 && n_axes == 3 && nax[0] == 1 && nax[1] == 2 && nax[2] == 3 && lanes[0] == 2 && lanes[1] == 2 && lanes[2] == 4 &&
        shape[1] % 2 == 0 && shape[2] % 2 == 0) {
        const uint64_t total = rows / 4;
        NNHIP_REQUIRE(ctx, rows < ((uint64_t)1 << 31), -EINVAL, "pack: tensor too large");
        if (total == 0) return 0;
        const uint32_t w_out = (uint32_t)shape[2] / 2;
        hipLaunchKernelGGL((pack_pixels_kernel<TIn, 2>), dim3((unsigned)((total + kLayoutThreads - 1) / kLayoutThreads)), dim3(kLayoutThreads),
                           0, ctx->stream, in, (uint32_t *)out, (uint32_t)total, w_out, make_fastdiv(w_out), c, scale, bias);
        NNHIP_LAUNCH_CHECK(ctx, "pack_pixels_kernel");
        return 0;
    }
    return 1;
}

template <typename T, bool SMALL> __global__ __launch_bounds__(kLayoutThreads) void unpack_kernel(const T *in, T *out, const PackDesc d) {
    const uint64_t gid = (uint64_t)blockIdx.x * kLayoutThreads + threadIdx.x;
    if (gid >= d.total) return;
    uint64_t rem = gid, off = 0;
    for (int k = d.out_rank - 1; k >= 0; k--) {
        uint32_t c;
        if constexpr (SMALL) {
            const uint32_t q = fastdiv((uint32_t)rem, d.out_div[k]);
            c = (uint32_t)rem - q * d.out_dims[k];
            rem = q;
        } else {
            c = (uint32_t)(rem % d.out_dims[k]);
            rem /= d.out_dims[k];
        }
        const uint32_t l = d.lanes[k];
        if (l > 1) {
            const uint32_t g = c / l;
            off += (uint64_t)g * d.in_strides[k] + (uint64_t)(c - g * l) * d.in_strides[d.lane_dim[k]];
        } else {
            off += (uint64_t)c * d.in_strides[k];
        }
    }
    out[gid] = in[off];
}

// ---- pack / unpack through an LDS tile ------------------------------------------------------------------------------
// The layouts pack exists for (NCHW -> NC/32 HW 32 for a matrix operand, [K, N] -> weight tiles) put the lanes of the LAST
// packed axis A innermost, and A is not the innermost axis of the plain tensor: every run of the packed tensor is a
// strided column of the plain one.  One thread per output element then reads single elements a row apart.  Here a
// block moves a tile of (one lane group of A) x (a stretch of the plain tensor's innermost axis X) through LDS: dword
// loads along the source's contiguous axis, dword stores along the destination's, and the E x E elements of a dword
// pair (E = 4 / element size) transposed in registers between the two, so that every LDS access is a dword as well
// (rows padded to a dword count that is 1 mod 32: neither phase meets a bank conflict worth the name).
// X is the trailing run of unpacked axes taken as one (NCHW: H x W), or the innermost axis when that is packed under
// an earlier lane entry ([K, N] by (N: 16, K: 64)).  Everything else -- other axes, the lane group of A, the stretch of
// X -- is decoded from the block index.
struct TwoTerm { // offset(i) = (i / lanes) * hi + (i % lanes) * lo, in elements
    uint32_t lanes;
    uint64_t hi, lo;
};
__device__ __forceinline__ uint64_t two_term(const TwoTerm &t, uint32_t i) {
    const uint32_t q = t.lanes == 1 ? i : i / t.lanes;
    return (uint64_t)q * t.hi + (uint64_t)(i - q * t.lanes) * t.lo;
}
struct TileDesc {
    int nrest;
    uint32_t r_extent[kMaxRank], r_valid[kMaxRank]; // coordinates from r_valid on have no source: their tiles are zeros (pack)
    TwoTerm r_plain[kMaxRank], r_packed[kMaxRank];
    uint32_t a_groups, a_extent, la; // lane groups of A, its plain extent, its lanes
    uint64_t a_plain_stride;          // plain elements between consecutive coordinates of A
    uint64_t a_packed_group;          // packed elements between consecutive lane groups of A
    uint32_t x_extent, x_padded, tx, x_tiles; // plain extent of X, its extent in the packed tensor, elements per tile
    TwoTerm x_packed;                 // packed offset of a coordinate of X (the plain one is the coordinate itself)
    uint32_t exact;                   // 1: the destination has no padding: lanes past the plain extent of A are not stored (transposes)
    uint32_t pitch;                   // dwords per LDS row
    FastDiv d_cols, d_rowq;           // dwords per row of the tile; rows / E
    uint32_t wide;                    // packing: every row of the source tile is whole 16-byte pieces at 16-byte addresses
    FastDiv d_cols4;                  // ... of which a row has this many
};

template <int E> __device__ __forceinline__ void transpose_dwords(const uint32_t (&d)[E], uint32_t (&o)[E]) {
    if constexpr (E == 1) {
        o[0] = d[0];
    } else if constexpr (E == 2) {
        o[0] = __builtin_amdgcn_perm(d[1], d[0], 0x05040100u);
        o[1] = __builtin_amdgcn_perm(d[1], d[0], 0x07060302u);
    } else {
        const uint32_t a_lo = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u), a_hi = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
        const uint32_t b_lo = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u), b_hi = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
        o[0] = __builtin_amdgcn_perm(b_lo, a_lo, 0x05040100u);
        o[1] = __builtin_amdgcn_perm(b_lo, a_lo, 0x07060302u);
        o[2] = __builtin_amdgcn_perm(b_hi, a_hi, 0x05040100u);
        o[3] = __builtin_amdgcn_perm(b_hi, a_hi, 0x07060302u);
    }
}

// E = elements per dword.  PACK: plain -> packed (LDS rows = lanes of A, columns = X); else packed -> plain (rows = X,
// columns = lanes of A).  in / out are byte pointers, 4-byte aligned like every row the host admits.
template <int E, bool PACK> __global__ __launch_bounds__(kLayoutThreads) void pack_tile_kernel(const uint8_t *in, uint8_t *out, const TileDesc d) {
    extern __shared__ uint32_t tile[];
    constexpr int ES = 4 / E;
    // ---- which tile ----
    uint32_t b = blockIdx.x;
    const uint32_t xt = b % d.x_tiles;
    b /= d.x_tiles;
    const uint32_t ag = b % d.a_groups;
    b /= d.a_groups;
    uint64_t plain = (uint64_t)ag * d.la * d.a_plain_stride, packed = (uint64_t)ag * d.a_packed_group;
    bool has_source = true;
    for (int i = d.nrest - 1; i >= 0; i--) {
        const uint32_t c = b % d.r_extent[i];
        b /= d.r_extent[i];
        has_source = has_source && c < d.r_valid[i];
        plain += two_term(d.r_plain[i], c);
        packed += two_term(d.r_packed[i], c);
    }
    const uint32_t x0 = xt * d.tx;
    plain += x0;
    const uint32_t vlim = min(d.la, d.a_extent - ag * d.la); // lanes of this group that exist in the plain tensor
    const uint32_t rows = PACK ? d.la : d.tx, cols = d.d_cols.div; // (cols in dwords)
    // ---- in: eight dwords per thread requested before the first is parked, or four 16-byte pieces where the plain
    // tensor's rows allow (the bytes in flight, not the instruction count, are what this phase lives on) ----
    constexpr int U = 8, UW = 4; // loads in flight per thread: dwords, 16-byte pieces
    if (PACK && d.wide) {
        const uint32_t cols4 = d.d_cols4.div;
        for (uint32_t base = threadIdx.x; base < rows * cols4; base += UW * kLayoutThreads) {
            uint4 v[UW];
            uint32_t at[UW];
#pragma unroll
            for (int u = 0; u < UW; u++) {
                const uint32_t idx = min(base + u * kLayoutThreads, rows * cols4 - 1);
                const uint32_t r = fastdiv(idx, d.d_cols4), c = (idx - r * cols4) * 4;
                at[u] = r * d.pitch + c;
                v[u] = uint4{0u, 0u, 0u, 0u};
                if (has_source && r < vlim && x0 + c * E < d.x_extent)
                    v[u] = *reinterpret_cast<const uint4 *>(in + (plain + (uint64_t)r * d.a_plain_stride) * ES + c * 4);
            }
#pragma unroll
            for (int u = 0; u < UW; u++) tile[at[u]] = v[u].x, tile[at[u] + 1] = v[u].y, tile[at[u] + 2] = v[u].z, tile[at[u] + 3] = v[u].w;
        }
    } else
    for (uint32_t base = threadIdx.x; base < rows * cols; base += U * kLayoutThreads) {
        uint32_t v[U], at[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const uint32_t idx = min(base + u * kLayoutThreads, rows * cols - 1); // (a repeat of the last dword: the same value to the same place)
            const uint32_t r = fastdiv(idx, d.d_cols), c = idx - r * cols;
            at[u] = r * d.pitch + c;
            v[u] = 0;
            if (PACK) { // row r = lane l, column c = E coordinates of X from x0 + c * E
                if (has_source && r < vlim && x0 + c * E < d.x_extent)
                    v[u] = *reinterpret_cast<const uint32_t *>(in + (plain + (uint64_t)r * d.a_plain_stride) * ES + c * 4);
            } else { // row r = coordinate x0 + r of X, column c = E lanes
                if (x0 + r < d.x_extent && c * E < vlim)
                    v[u] = *reinterpret_cast<const uint32_t *>(in + (packed + two_term(d.x_packed, x0 + r)) * ES + c * 4);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) tile[at[u]] = v[u];
    }
    __syncthreads();
    // ---- out: E rows x one dword column at a time, the lanes of a wave along the destination's contiguous axis ----
    // (packing, a lane's E dwords go to E different runs of the destination; parking the transposed tile in a second
    // LDS area so that it leaves in address order was measured and is no quicker)
    const uint32_t rowq = d.d_rowq.div;
    for (uint32_t idx = threadIdx.x; idx < rowq * cols; idx += kLayoutThreads) {
        const uint32_t c = fastdiv(idx, d.d_rowq), rq = idx - c * rowq;
        uint32_t w[E], o[E];
#pragma unroll
        for (int k = 0; k < E; k++) w[k] = tile[(rq * E + k) * d.pitch + c];
        transpose_dwords<E>(w, o);
#pragma unroll
        for (int j = 0; j < E; j++) {
            if (PACK) { // o[j]: lanes rq * E .. of coordinate x0 + c * E + j
                const uint32_t x = x0 + c * E + j;
                if (x < d.x_padded && (!d.exact || rq * E < vlim))
                    *reinterpret_cast<uint32_t *>(out + (packed + two_term(d.x_packed, x)) * ES + rq * 4) = o[j];
            } else { // o[j]: coordinates x0 + rq * E .. of lane c * E + j
                const uint32_t l = c * E + j;
                if (l < vlim && x0 + rq * E < d.x_extent)
                    *reinterpret_cast<uint32_t *>(out + (plain + (uint64_t)l * d.a_plain_stride) * ES + rq * 4) = o[j];
            }
        }
    }
}

// Elements of X per tile: about 16 KiB per tile, rows of the plain tensor of 64 bytes to 2 KiB.
// The extent is then split evenly over its tiles (3136 = 7 x 448 rather than 6 x 512 + 64).
static uint32_t tile_stretch(uint32_t la, int es, uint32_t x_extent, bool wide) {
    const uint32_t e = (wide ? 16 : 4) / es; // tiles begin at whole dwords (16-byte pieces) of a row
    uint32_t tx = 16384 / (la * es);
    tx = std::min<uint32_t>(std::max<uint32_t>(tx, 64 / es), 2048 / es) / e * e;
    const uint32_t tiles = (x_extent + tx - 1) / tx;
    return ((x_extent + tiles - 1) / tiles + e - 1) / e * e;
}
// Dwords per LDS row: odd, so that the E rows a lane reads and the rows of neighbouring lanes spread over the banks.
static uint32_t tile_pitch(uint32_t cols) { return cols | 1u; }
// Fills the tile description for pack (plain -> packed) or unpack of `shape` by (axes, lanes); false when the layout is
// not one the tile kernel moves (then the element-wise kernels do).
static bool make_tile_desc(TileDesc &d, int es, int rank, const int32_t *shape, int n_axes, const int *nax, const int32_t *lanes, bool pack,
                           const void *in, const void *out, uint64_t &blocks, size_t &lds) {
    if (n_axes < 1 || (es != 1 && es != 2 && es != 4)) return false;
    const int e = 4 / es;
    if (((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 3u) != 0) return false;
    uint32_t L[kMaxRank], O[kMaxRank];
    int jpos[kMaxRank];
    uint64_t lp_all = 1;
    for (int i = 0; i < rank; i++) L[i] = 1, jpos[i] = -1;
    for (int j = 0; j < n_axes; j++) L[nax[j]] = (uint32_t)lanes[j], jpos[nax[j]] = j, lp_all *= (uint64_t)lanes[j];
    uint64_t sp[kMaxRank], sqo[kMaxRank], sql[kMaxRank];
    uint64_t st = 1;
    for (int i = rank - 1; i >= 0; i--) sp[i] = st, st *= (uint64_t)shape[i];
    if (st >= ((uint64_t)1 << 40)) return false;
    st = 1;
    for (int j = n_axes - 1; j >= 0; j--) sql[j] = st, st *= (uint64_t)lanes[j];
    for (int i = rank - 1; i >= 0; i--) O[i] = ((uint32_t)shape[i] + L[i] - 1) / L[i], sqo[i] = st, st *= O[i];
    const int a = nax[n_axes - 1];
    const uint32_t la = (uint32_t)lanes[n_axes - 1];
    if (a == rank - 1 || la % e != 0 || la < (uint32_t)e || la > 128) return false;
    memset(&d, 0, sizeof(d));
    // X: the trailing unpacked axes as one, or the (packed) innermost axis
    int xs = rank;
    while (xs > 0 && L[xs - 1] == 1) xs--;
    uint64_t xe = 1;
    if (xs < rank) {
        for (int i = xs; i < rank; i++) xe *= (uint64_t)shape[i];
        if (xe >= ((uint64_t)1 << 31)) return false;
        d.x_extent = d.x_padded = (uint32_t)xe;
        d.x_packed = TwoTerm{1, lp_all, 0};
    } else {
        xs = rank - 1;
        d.x_extent = (uint32_t)shape[xs];
        d.x_padded = O[xs] * L[xs];
        d.x_packed = TwoTerm{L[xs], sqo[xs], sql[jpos[xs]]};
    }
    if (a >= xs || ((uint64_t)d.x_extent * es) % 4 != 0) return false;
    if (!pack) d.x_padded = d.x_extent;
    d.wide = pack && ((uint64_t)d.x_extent * es) % 16 == 0 && (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
    d.tx = tile_stretch(la, es, d.x_padded, d.wide);
    d.x_tiles = (d.x_padded + d.tx - 1) / d.tx;
    d.la = la, d.a_extent = (uint32_t)shape[a], d.a_groups = O[a];
    d.a_plain_stride = sp[a], d.a_packed_group = sqo[a];
    blocks = (uint64_t)d.x_tiles * d.a_groups;
    for (int i = 0; i < xs; i++) {
        if (i == a) continue;
        const int k = d.nrest++;
        d.r_extent[k] = pack ? O[i] * L[i] : (uint32_t)shape[i];
        d.r_valid[k] = (uint32_t)shape[i];
        d.r_plain[k] = TwoTerm{1, sp[i], 0};
        d.r_packed[k] = L[i] == 1 ? TwoTerm{1, sqo[i], 0} : TwoTerm{L[i], sqo[i], sql[jpos[i]]};
        blocks *= d.r_extent[k];
    }
    if (blocks == 0 || blocks >= ((uint64_t)1 << 31)) return false;
    const uint32_t rows = pack ? la : d.tx, cols = (pack ? d.tx : la) / e;
    d.pitch = tile_pitch(cols);
    d.d_cols = make_fastdiv(cols);
    d.d_rowq = make_fastdiv(rows / e);
    d.d_cols4 = make_fastdiv(std::max<uint32_t>(cols / 4, 1));
    lds = (size_t)rows * d.pitch * 4;
    return lds <= 48 * 1024;
}

template <bool PACK> static int launch_pack_tile(nncase_hip_ctx *ctx, const void *in, void *out, int es, const TileDesc &d, uint64_t blocks, size_t lds) {
    const dim3 grid((unsigned)blocks), block(kLayoutThreads);
    if (lds > 48 * 1024) return 1; // (not asked for: the tiles are sized to stay below)
    switch (es) {
    case 1: hipLaunchKernelGGL((pack_tile_kernel<4, PACK>), grid, block, lds, ctx->stream, (const uint8_t *)in, (uint8_t *)out, d); break;
    case 2: hipLaunchKernelGGL((pack_tile_kernel<2, PACK>), grid, block, lds, ctx->stream, (const uint8_t *)in, (uint8_t *)out, d); break;
    default: hipLaunchKernelGGL((pack_tile_kernel<1, PACK>), grid, block, lds, ctx->stream, (const uint8_t *)in, (uint8_t *)out, d); break;
    }
    NNHIP_LAUNCH_CHECK(ctx, "pack_tile_kernel");
    return 0;
}

// [batch][rows][cols] -> [batch][cols][rows] through a 32x32 LDS tile.
template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T *__restrict__ in, T *__restrict__ out, int rows, int cols) {
    __shared__ T tile[32][33];
    const size_t boff = (size_t)blockIdx.z * rows * cols;
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int r = r0 + ty + i, c = c0 + tx;
        if (r < rows && c < cols) tile[ty + i][tx] = in[boff + (size_t)r * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 32; i += 8) {
        const int c = c0 + ty + i, r = r0 + tx;
        if (r < rows && c < cols) out[boff + (size_t)c * rows + r] = tile[tx][ty + i];
    }
}

template <typename T> static int launch_transpose(nncase_hip_ctx *ctx, const void *in, void *out, int batch, int rows, int cols) {
    const dim3 grid(ceil_div(cols, 32), ceil_div(rows, 32), batch);
    hipLaunchKernelGGL(transpose_kernel<T>, grid, dim3(256), 0, ctx->stream, (const T *)in, (T *)out, rows, cols);
    NNHIP_LAUNCH_CHECK(ctx, "transpose_kernel");
    return 0;
}

// [batch][rows][cols] -> [batch][cols][rows] as the tile kernel sees it.  Packing: the source is the plain tensor
// (A = rows in groups of up to 128 lanes, X = cols), the destination the "packed" one, whose runs along A have no
// padding.  Unpacking (short source rows): the destination is the plain tensor (A = cols, X = rows).
static bool make_transpose_desc(TileDesc &d, int es, int batch, int rows, int cols, bool packing, const void *in, const void *out,
                                uint64_t &blocks, size_t &lds) {
    if (es != 1 && es != 2 && es != 4) return false;
    const int e = 4 / es;
    if (((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 3u) != 0 || rows % e != 0 || cols % e != 0) return false;
    memset(&d, 0, sizeof(d));
    const int na = packing ? rows : cols, nx = packing ? cols : rows; // extents of A and X
    const uint32_t la = (uint32_t)std::min(na, 128 / e * e);
    d.la = la, d.a_extent = (uint32_t)na, d.a_groups = ((uint32_t)na + la - 1) / la;
    d.a_plain_stride = (uint64_t)nx, d.a_packed_group = la;
    d.x_extent = d.x_padded = (uint32_t)nx;
    d.x_packed = TwoTerm{1, (uint64_t)na, 0};
    d.exact = 1;
    d.wide = packing && ((uint64_t)nx * es) % 16 == 0 && (reinterpret_cast<uintptr_t>(in) & 15u) == 0;
    d.tx = tile_stretch(la, es, d.x_padded, d.wide);
    d.x_tiles = (d.x_padded + d.tx - 1) / d.tx;
    d.nrest = 1;
    d.r_extent[0] = d.r_valid[0] = (uint32_t)batch;
    d.r_plain[0] = d.r_packed[0] = TwoTerm{1, (uint64_t)rows * cols, 0};
    blocks = (uint64_t)d.x_tiles * d.a_groups * batch;
    if (blocks >= ((uint64_t)1 << 31)) return false;
    const uint32_t trows = packing ? la : d.tx, tcols = (packing ? d.tx : la) / e;
    d.pitch = tile_pitch(tcols);
    d.d_cols = make_fastdiv(tcols);
    d.d_rowq = make_fastdiv(trows / e);
    d.d_cols4 = make_fastdiv(std::max<uint32_t>(tcols / 4, 1));
    lds = (size_t)trows * d.pitch * 4;
    return lds <= 48 * 1024;
}

static int transpose(nncase_hip_ctx *ctx, const void *in, void *out, int es, int batch, int rows, int cols) {
    NNHIP_REQUIRE(ctx, in && out, -EINVAL, "transpose: null buffer");
    NNHIP_REQUIRE(ctx, batch > 0 && rows > 0 && cols > 0, -EINVAL, "transpose: non-positive shape");
    // The tile kernel for elements narrower than a dword (its accesses stay dwords) and for matrices with a short
    // side (its tiles follow the long one); 4-byte elements of other shapes are the 32 x 32 tiles' case (measured:
    // 255 x 6400 floats 34 us there, 58 us here).
    if (es < 4 || std::min(rows, cols) < 32) {
        TileDesc t;
        uint64_t blocks = 0;
        size_t lds = 0;
        const bool packing = (size_t)cols * es >= 128; // source rows long enough to be read as rows
        if (make_transpose_desc(t, es, batch, rows, cols, packing, in, out, blocks, lds)) {
            const int rc = packing ? launch_pack_tile<true>(ctx, in, out, es, t, blocks, lds) : launch_pack_tile<false>(ctx, in, out, es, t, blocks, lds);
            if (rc <= 0) return rc;
        }
    }
    NNHIP_REQUIRE(ctx, batch <= 65535 && ceil_div(rows, 32) <= 65535, -EINVAL, "transpose: grid too large");
    switch (es) {
    case 1: return launch_transpose<uint8_t>(ctx, in, out, batch, rows, cols);
    case 2: return launch_transpose<uint16_t>(ctx, in, out, batch, rows, cols);
    case 4: return launch_transpose<uint32_t>(ctx, in, out, batch, rows, cols);
    default: return fail(ctx, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "transpose: element size %d", es);
    }
}

static int build_common(nncase_hip_ctx *ctx, int rank, const int32_t *shape, int n_axes, const int32_t *axes,
                        const int32_t *lanes, int (&norm_axes)[kMaxRank]) {
    NNHIP_REQUIRE(ctx, shape && (n_axes == 0 || (axes && lanes)), -EINVAL, "pack: null argument");
    NNHIP_REQUIRE(ctx, rank > 0 && rank <= kMaxRank && n_axes >= 0 && n_axes <= rank, -EINVAL, "pack: rank %d / %d axes",
                  rank, n_axes);
    for (int i = 0; i < rank; i++) NNHIP_REQUIRE(ctx, shape[i] > 0, -EINVAL, "pack: non-positive extent");
    for (int i = 0; i < n_axes; i++) {
        int ax = axes[i] < 0 ? axes[i] + rank : axes[i];
        NNHIP_REQUIRE(ctx, ax >= 0 && ax < rank && lanes[i] > 0, -EINVAL, "pack: bad axis/lanes");
        for (int j = 0; j < i; j++) NNHIP_REQUIRE(ctx, norm_axes[j] != ax, -EINVAL, "pack: repeated axis");
        norm_axes[i] = ax;
    }
    return 0;
}

// Where the packed tensor's innermost dimension runs along the plain tensor's innermost axis (no packed axis, or that
// axis packed last), groups of elements of it move together: the same permutation on 16- or 4-byte elements, that many
// times fewer of them.  Rewrites (es, shape, lanes) in place when extents, lanes and addresses allow.
static void vector_view(int &es, int rank, int32_t *shape, int n_axes, const int *nax, int32_t *lanes, const void *in, const void *out) {
    for (int j = 0; j < n_axes; j++)
        if (nax[j] == rank - 1 && j != n_axes - 1) return;
    if (n_axes > 0 && nax[n_axes - 1] != rank - 1) return; // (the innermost lanes belong to another axis)
    for (int bytes = 16; bytes > es; bytes /= 4) {
        if (bytes % es != 0) continue;
        const int e = bytes / es;
        if (((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & (uintptr_t)(bytes - 1)) != 0 || shape[rank - 1] % e != 0) continue;
        if (n_axes > 0 && lanes[n_axes - 1] % e != 0) continue;
        shape[rank - 1] /= e;
        if (n_axes > 0) lanes[n_axes - 1] /= e;
        es = bytes;
        return;
    }
}

// Neighbouring axes that are both unpacked are one axis to the permutation (their outer dimensions are neighbours in
// the packed tensor too): fewer coordinates for every thread to take apart.  Rewrites (rank, shape, axes) in place.
static void merge_unpacked_axes(int &rank, int32_t *shape, int n_axes, int *nax) {
    bool packed[kMaxRank] = {false};
    for (int j = 0; j < n_axes; j++) packed[nax[j]] = true;
    int to[kMaxRank], r = 0;
    for (int i = 0; i < rank; i++) {
        if (i > 0 && !packed[i] && !packed[i - 1] && (int64_t)shape[r - 1] * shape[i] < ((int64_t)1 << 31)) {
            shape[r - 1] *= shape[i];
        } else {
            shape[r] = shape[i];
            packed[r] = packed[i]; // (r <= i: entries below i are no longer read)
            r++;
        }
        to[i] = r - 1;
    }
    for (int j = 0; j < n_axes; j++) nax[j] = to[nax[j]];
    rank = r;
}

typedef uint32_t layout_u32x4 __attribute__((ext_vector_type(4)));

template <typename K> static int launch_by_size(nncase_hip_ctx *ctx, int es, K &&k) {
    switch (es) {
    case 1: return k((uint8_t *)nullptr);
    case 2: return k((uint16_t *)nullptr);
    case 4: return k((uint32_t *)nullptr);
    case 16: return k((layout_u32x4 *)nullptr); // (vector_view's groups only)
    default: return fail(ctx, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "pack: element size %d", es);
    }
}

} // namespace nnhip

using namespace nnhip;

extern "C" int nncase_hip_pack(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size, int32_t rank,
                               const int32_t *shape, int32_t n_axes, const int32_t *axes, const int32_t *lanes) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "pack: null buffer");
    NNHIP_REQUIRE(ctx, elem_size == 1 || elem_size == 2 || elem_size == 4, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "pack: element size %d", elem_size);
    int nax[kMaxRank];
    int rc = build_common(ctx, rank, shape, n_axes, axes, lanes, nax);
    if (rc) return rc;
    // the stem layouts (RGB -> RGBX, and 2 x 2 blocks of RGBX pixels -> 16-channel pixels): one thread per output pixel
    if (elem_size == 1) {
        rc = launch_pack_pixels<uint8_t>(ctx, (const uint8_t *)in_dev, out_dev, rank, shape, n_axes, nax, lanes, 1.f, 0.f);
        if (rc <= 0) return rc;
    }
    {
        TileDesc t;
        uint64_t blocks = 0;
        size_t lds = 0;
        if (make_tile_desc(t, elem_size, rank, shape, n_axes, nax, lanes, true, in_dev, out_dev, blocks, lds)) {
            rc = launch_pack_tile<true>(ctx, in_dev, out_dev, elem_size, t, blocks, lds);
            if (rc <= 0) return rc;
        }
    }
    int32_t shp[kMaxRank], lns[kMaxRank];
    for (int i = 0; i < rank; i++) shp[i] = shape[i];
    for (int j = 0; j < n_axes; j++) lns[j] = lanes[j];
    int es = elem_size;
    vector_view(es, rank, shp, n_axes, nax, lns, in_dev, out_dev);
    {
        int merged = rank;
        merge_unpacked_axes(merged, shp, n_axes, nax);
        rank = merged;
    }
    PackDesc d;
    memset(&d, 0, sizeof(d));
    d.in_rank = rank;
    d.out_rank = rank + n_axes;
    uint64_t stride = 1;
    for (int i = rank - 1; i >= 0; i--) {
        d.in_dims[i] = (uint32_t)shp[i];
        d.in_strides[i] = stride;
        stride *= (uint64_t)shp[i];
    }
    d.total = 1;
    for (int i = 0; i < rank; i++) {
        uint32_t l = 1;
        for (int j = 0; j < n_axes; j++)
            if (nax[j] == i) l = (uint32_t)lns[j];
        d.out_dims[i] = ((uint32_t)shp[i] + l - 1) / l;
        d.axis[i] = i;
        d.mul[i] = l;
        d.total *= d.out_dims[i];
    }
    for (int j = 0; j < n_axes; j++) {
        d.out_dims[rank + j] = (uint32_t)lns[j];
        d.axis[rank + j] = nax[j];
        d.mul[rank + j] = 1;
        d.total *= (uint64_t)lns[j];
    }
    NNHIP_REQUIRE(ctx, d.total < ((uint64_t)1 << 40), -EINVAL, "pack: tensor too large");
    for (int k = 0; k < d.out_rank; k++) d.out_div[k] = make_fastdiv(d.out_dims[k]);
    const uint64_t blocks = (d.total + kLayoutThreads - 1) / kLayoutThreads;
    NNHIP_REQUIRE(ctx, blocks < ((uint64_t)1 << 31), -EINVAL, "pack: tensor too large");
    return launch_by_size(ctx, es, [&](auto *tag) -> int {
        typedef typename std::remove_pointer<decltype(tag)>::type T;
        if (d.total < ((uint64_t)1 << 31))
            hipLaunchKernelGGL((pack_kernel<T, true>), dim3((unsigned)blocks), dim3(kLayoutThreads), 0, ctx->stream, (const T *)in_dev, (T *)out_dev, d);
        else
            hipLaunchKernelGGL((pack_kernel<T, false>), dim3((unsigned)blocks), dim3(kLayoutThreads), 0, ctx->stream, (const T *)in_dev, (T *)out_dev, d);
        NNHIP_LAUNCH_CHECK(ctx, "pack_kernel");
        return 0;
    });
}

extern "C" int nncase_hip_quantize_pack(nncase_hip_ctx_t *ctx, const float *in_dev, uint8_t *out_dev, int32_t rank, const int32_t *shape,
                                        int32_t n_axes, const int32_t *axes, const int32_t *lanes, nncase_hip_quant_param_t qp) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "quantize_pack: null buffer");
    NNHIP_REQUIRE(ctx, qp.scale != 0.f, -EINVAL, "quantize_pack: scale is zero");
    int nax[kMaxRank];
    int rc = build_common(ctx, rank, shape, n_axes, axes, lanes, nax);
    if (rc) return rc;
    rc = launch_pack_pixels<float>(ctx, in_dev, out_dev, rank, shape, n_axes, nax, lanes, qp.scale, (float)qp.zero_point);
    if (rc <= 0) return rc;
    return fail(ctx, -EINVAL,
                "quantize_pack: only <= 4 innermost channels packed by (4), or NHWC with even H and W packed by (2, 2, 4) on (H, W, C), "
                "into a 16-byte aligned buffer");
}

extern "C" int nncase_hip_unpack(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size, int32_t rank,
                                 const int32_t *unpacked_shape, int32_t n_axes, const int32_t *axes, const int32_t *lanes) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, in_dev && out_dev, -EINVAL, "unpack: null buffer");
    NNHIP_REQUIRE(ctx, elem_size == 1 || elem_size == 2 || elem_size == 4, -NNCASE_HIP_ERR_DATATYPE_MISMATCH, "unpack: element size %d", elem_size);
    int nax[kMaxRank];
    int rc = build_common(ctx, rank, unpacked_shape, n_axes, axes, lanes, nax);
    if (rc) return rc;
    {
        TileDesc t;
        uint64_t blocks = 0;
        size_t lds = 0;
        if (make_tile_desc(t, elem_size, rank, unpacked_shape, n_axes, nax, lanes, false, in_dev, out_dev, blocks, lds)) {
            rc = launch_pack_tile<false>(ctx, in_dev, out_dev, elem_size, t, blocks, lds);
            if (rc <= 0) return rc;
        }
    }
    int32_t shp[kMaxRank], lns[kMaxRank];
    for (int i = 0; i < rank; i++) shp[i] = unpacked_shape[i];
    for (int j = 0; j < n_axes; j++) lns[j] = lanes[j];
    int es = elem_size;
    vector_view(es, rank, shp, n_axes, nax, lns, in_dev, out_dev);
    {
        int merged = rank;
        merge_unpacked_axes(merged, shp, n_axes, nax);
        rank = merged;
    }
    PackDesc d;
    memset(&d, 0, sizeof(d));
    d.out_rank = rank;
    d.in_rank = rank + n_axes;
    // packed (input) dims and strides
    for (int i = 0; i < rank; i++) {
        uint32_t l = 1;
        d.lane_dim[i] = 0;
        for (int j = 0; j < n_axes; j++)
            if (nax[j] == i) {
                l = (uint32_t)lns[j];
                d.lane_dim[i] = rank + j;
            }
        d.lanes[i] = l;
        d.in_dims[i] = ((uint32_t)shp[i] + l - 1) / l;
        d.out_dims[i] = (uint32_t)shp[i];
    }
    for (int j = 0; j < n_axes; j++) d.in_dims[rank + j] = (uint32_t)lns[j];
    uint64_t stride = 1;
    for (int i = d.in_rank - 1; i >= 0; i--) {
        d.in_strides[i] = stride;
        stride *= d.in_dims[i];
    }
    d.total = 1;
    for (int i = 0; i < rank; i++) d.total *= d.out_dims[i];
    for (int k = 0; k < d.out_rank; k++) d.out_div[k] = make_fastdiv(d.out_dims[k]);
    const uint64_t blocks = (d.total + kLayoutThreads - 1) / kLayoutThreads;
    NNHIP_REQUIRE(ctx, blocks < ((uint64_t)1 << 31), -EINVAL, "unpack: tensor too large");
    return launch_by_size(ctx, es, [&](auto *tag) -> int {
        typedef typename std::remove_pointer<decltype(tag)>::type T;
        if (d.total < ((uint64_t)1 << 31))
            hipLaunchKernelGGL((unpack_kernel<T, true>), dim3((unsigned)blocks), dim3(kLayoutThreads), 0, ctx->stream, (const T *)in_dev, (T *)out_dev, d);
        else
            hipLaunchKernelGGL((unpack_kernel<T, false>), dim3((unsigned)blocks), dim3(kLayoutThreads), 0, ctx->stream, (const T *)in_dev, (T *)out_dev, d);
        NNHIP_LAUNCH_CHECK(ctx, "unpack_kernel");
        return 0;
    });
}

extern "C" int nncase_hip_nchw_to_nhwc(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size, int32_t n,
                                       int32_t c, int32_t h, int32_t w) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, h > 0 && w > 0 && (int64_t)h * w < ((int64_t)1 << 31), -EINVAL, "nchw_to_nhwc: bad shape");
    return transpose(ctx, in_dev, out_dev, elem_size, n, c, h * w); // [n][c][hw] -> [n][hw][c]
}

extern "C" int nncase_hip_nhwc_to_nchw(nncase_hip_ctx_t *ctx, const void *in_dev, void *out_dev, int32_t elem_size, int32_t n,
                                       int32_t c, int32_t h, int32_t w) {
    NNHIP_CHECK_CTX(ctx);
    NNHIP_REQUIRE(ctx, h > 0 && w > 0 && (int64_t)h * w < ((int64_t)1 << 31), -EINVAL, "nhwc_to_nchw: bad shape");
    return transpose(ctx, in_dev, out_dev, elem_size, n, h * w, c); // [n][hw][c] -> [n][c][hw]
}
