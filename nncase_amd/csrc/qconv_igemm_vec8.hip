// Instantiates the implicit-GEMM kernel for the kVec8 activation loader.
#include "qconv_igemm.hpp"

namespace nnhip {
int launch_igemm_vec8(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    return launch_mode<kVec8>(ctx, a, tiles, nchunks, rg);
}
} // namespace nnhip
