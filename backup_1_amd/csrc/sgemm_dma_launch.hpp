// Launch of one shape of the kernel of sgemm_dma_tile.hpp; instantiated in sgemm_dma_small.hip, sgemm_dma_blocks16.hip and
// sgemm_dma_large.hip and sgemm_dma_wide.hip (the shapes compile for 15 - 30 s each, side by side in four translation units).
#pragma once
#include "sgemm_launch.hpp"
#include "sgemm_dma_tile.hpp"

namespace decx_hip {

template <class S>
int launch_sgemm_dma(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                       int N, int K, const Batch& batch, bool relu) {
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL || batch.count > 65535) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    auto kern = Cin ? sgemm_dma_kernel<S, true> : sgemm_dma_kernel<S, false>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_dma_kernel<S, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_dma_kernel<S, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)batch.count), dim3(S::NT), S::LDS_BYTES, batch.stream, A, lda, B, ldb,
                       Cin, ldc, D, ldd, M, N, K, tiles_m, tiles_n, group_m, relu, batch.stride_a, batch.stride_b, batch.stride_c,
                       batch.stride_d);
    HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace decx_hip
