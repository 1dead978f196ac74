// Instantiates the implicit-GEMM kernel for the kRows16 activation loader.
#include "qconv_igemm.hpp"

namespace nnhip {
int launch_igemm_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    return launch_mode<kRows16>(ctx, a, tiles, nchunks, rg);
}
} // namespace nnhip
