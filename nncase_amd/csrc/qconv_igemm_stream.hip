// Instantiations of the weight-streaming implicit-GEMM kernels (long reductions).
#include "qconv_igemm.hpp"

namespace nnhip {
int launch_igemm_stream_rows16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    return launch_stream_mode<kRows16>(ctx, a, tiles, nchunks, rg);
}
int launch_igemm_stream_vec16(nncase_hip_ctx *ctx, const IgemmArgs &a, int tiles, int nchunks, int rg) {
    return launch_stream_mode<kVec16>(ctx, a, tiles, nchunks, rg);
}
} // namespace nnhip
