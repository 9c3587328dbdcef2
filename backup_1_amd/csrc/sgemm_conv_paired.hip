// fp32 fused im2col convolution: the tile kernels (sgemm_tile.hpp) for the loaders of
// a channel pitch that is a multiple of 8 (the 8 consecutive k of a staging task never straddle a tap).
#include "sgemm_launch.hpp"

namespace decx_hip {

int conv_dispatch_paired(int variant, const Im2colA<true>& a, const FilterB<true>& b, const float* bias, float* dst,
                     const TensorOut& out, int M, int N, int K, const Batch& batch) {
    // a bias is the "+ C" operand with row stride 0: every output pixel adds the same N values
    return dispatch_sgemm(variant, a, b, bias, 0, dst, out, M, N, K, batch);
}

}  // namespace decx_hip
