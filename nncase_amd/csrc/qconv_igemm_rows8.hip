// Instantiates the implicit-GEMM kernel for the kRows8 activation loader.
#include "qconv_igemm.hpp"

namespace nnhip {
int launch_igemm_rows8(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    return launch_mode<kRows8>(ctx, a, tiles, nchunks, rg);
}
} // namespace nnhip
