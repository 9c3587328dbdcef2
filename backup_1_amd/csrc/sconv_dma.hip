// fp32 fused im2col convolution on the LDS-DMA kernel of 16x16 blocks (sconv_dma.hpp): its shapes and their launch.
#include "sgemm_launch.hpp"
#include "sconv_dma.hpp"

namespace decx_hip {

template <class S>
static int launch_sconv_dma(const Im2colA<true>& img, const FilterB<true>& fb, const float* bias, float* dst, const TensorOut& out,
                            int M, int N, int K) {
    // tiles are patches of 16 output rows x BM / 16 columns (sconv_tiles counts them the same way)
    const int Hout = M / out.Wout, tiles_x = cdiv(out.Wout, S::BM / 16), tiles_m = cdiv(Hout, 16) * tiles_x, tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sconv_dma_kernel<S>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    hipLaunchKernelGGL(sconv_dma_kernel<S>, dim3((unsigned)total), dim3(S::NT), S::LDS_BYTES, g_rt.stream, img, fb, bias, dst, out, Hout, N, K, tiles_x, tiles_m, tiles_n);
    HIP_TRY(hipGetLastError());
    return 0;
}

// shape 29: 208 x 128 (eight waves of 13 x 1 blocks); 30: 256 x 256 (2 x 4 waves of 8 x 4 blocks)
int launch_sconv_dma_shape(int shape, const Im2colA<true>& img, const FilterB<true>& fb, const float* bias, float* dst,
                           const TensorOut& out, int M, int N, int K) {
    if (shape == 29) return launch_sconv_dma<SconvDmaShape<13, 1, 1, 8>>(img, fb, bias, dst, out, M, N, K);
    return launch_sconv_dma<SconvDmaShape<8, 4, 2, 4>>(img, fb, bias, dst, out, M, N, K);
}

}  // namespace decx_hip
