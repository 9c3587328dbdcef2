// fp32 dense GEMM on tiles fed by LDS-DMA loads (sgemm_dma_tile.hpp): the 256x192 tile on eight waves.
#include "sgemm_dma_launch.hpp"

namespace decx_hip {

int launch_sgemm_dma_wide(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu) {
    if (shape == 28) return launch_sgemm_dma<DmaTile<256, 192, 16, 2, 32, 8, 1>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    return fail(DECX_HIP_FAIL_ERROR_PARAMS, "unknown tile shape\n");
}

}  // namespace decx_hip
