// fp32 dense GEMM on tiles fed by LDS-DMA loads (sgemm_dma_tile.hpp): the 128x128 tile on 32x32 blocks and the tiles on 16x16 blocks.
#include "sgemm_dma_launch.hpp"

namespace decx_hip {

int launch_sgemm_dma_blocks16(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu) {
    if (shape == 20) return launch_sgemm_dma<DmaTile<128, 128, 16, 2, 32, 4, 2>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 24) return launch_sgemm_dma<DmaTile<32, 32, 64, 3, 16>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 25) return launch_sgemm_dma<DmaTile<64, 32, 64, 3, 16>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    return fail(DECX_HIP_FAIL_ERROR_PARAMS, "unknown tile shape\n");
}

}  // namespace decx_hip
