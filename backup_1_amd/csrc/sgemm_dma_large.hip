// fp32 dense GEMM on tiles fed by LDS-DMA loads (sgemm_dma_tile.hpp): 256x256 and 256x224 tiles on eight waves.
#include "sgemm_dma_launch.hpp"

namespace decx_hip {

int launch_sgemm_dma_large(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu) {
    if (shape == 26) return launch_sgemm_dma<DmaTile<256, 256, 16, 2, 32, 4, 2>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 27) return launch_sgemm_dma<DmaTile<256, 224, 16, 2, 32, 8, 1>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    return fail(DECX_HIP_FAIL_ERROR_PARAMS, "unknown tile shape\n");
}

}  // namespace decx_hip
