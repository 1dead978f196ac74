// Instantiations of the wide-tile implicit-GEMM kernels for windows (any kernel size, stride, dilation, padding).
#include "qconv_wide.hpp"

namespace nnhip {
int launch_wide_vec16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks) {
    return a.g_ic % 64 == 0 ? launch_wide_lm<kWideTap>(ctx, a, tiles, nchunks) : launch_wide_lm<kWideWindow>(ctx, a, tiles, nchunks);
}
int launch_wide_small_vec16(nncase_hip_ctx *ctx, const IgemmArgs &a, int variant, int nchunks) {
    return a.g_ic % 64 == 0 ? launch_wide_small_lm<kWideTap>(ctx, a, variant, nchunks) : launch_wide_small_lm<kWideWindow>(ctx, a, variant, nchunks);
}
} // namespace nnhip
