// Instantiates the implicit-GEMM kernel for the kBytes activation loader.
#include "qconv_igemm.hpp"

namespace nnhip {
int launch_igemm_bytes(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    return launch_mode<kBytes>(ctx, a, tiles, nchunks, rg);
}
} // namespace nnhip
