// Instantiations of the wide-tile implicit-GEMM kernels for contiguous reduction rows (1x1 windows, matmul).
#include "qconv_wide.hpp"

namespace nnhip {
int launch_wide_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks) {
    return a.k % 64 == 0 ? launch_wide_lm<kWideRowsFull>(ctx, a, tiles, nchunks) : launch_wide_lm<kWideRows>(ctx, a, tiles, nchunks);
}
int launch_wide_small_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int variant, int nchunks) {
    return a.k % 64 == 0 ? launch_wide_small_lm<kWideRowsFull>(ctx, a, variant, nchunks) : launch_wide_small_lm<kWideRows>(ctx, a, variant, nchunks);
}
} // namespace nnhip
