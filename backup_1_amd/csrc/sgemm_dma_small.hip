// fp32 dense GEMM on tiles fed by LDS-DMA loads (sgemm_dma_tile.hpp): 64x64, 64x128 and 128x64 tiles on 32x32 blocks.
#include "sgemm_dma_launch.hpp"

namespace decx_hip {

int launch_sgemm_dma_small(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu) {
    if (shape == 18) return launch_sgemm_dma<DmaTile<64, 64, 32, 4>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 19) return launch_sgemm_dma<DmaTile<64, 64, 64, 3>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 21) return launch_sgemm_dma<DmaTile<64, 128, 32, 4>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 22) return launch_sgemm_dma<DmaTile<128, 64, 32, 4>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    return fail(DECX_HIP_FAIL_ERROR_PARAMS, "unknown tile shape\n");
}

}  // namespace decx_hip
