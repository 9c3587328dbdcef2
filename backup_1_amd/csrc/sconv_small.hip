// fp32 fused im2col convolution of small images on tiles of 16x16 blocks fed by LDS-DMA loads (sconv_small.hpp): its
// shapes and their launch.
#include "sgemm_launch.hpp"
#include "sconv_small.hpp"

namespace decx_hip {

template <class S>
static int launch_sconv_small(const Im2colA<true>& img, const FilterB<true>& fb, const float* bias, float* dst, const TensorOut& out,
                              int M, int N, int K) {
    const int Hout = M / out.Wout, tiles_x = cdiv(out.Wout, S::PX), tiles_m = cdiv(Hout, S::PY) * tiles_x, tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sconv_small_kernel<S>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    hipLaunchKernelGGL(sconv_small_kernel<S>, dim3((unsigned)total), dim3(S::NT), S::LDS_BYTES, g_rt.stream, img, fb, bias, dst, out, Hout, N, K, tiles_x, tiles_m, tiles_n);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Tiles of 32 pixels (8 x 4) x 32 filters, one block per wave; K steps of 64 in three buffers where the channel pitch
// allows it, else of 32 in four.  (Tiles of 64 x 32, 32 x 64 and 64 x 64 were measured on 27 layer shapes from 7x7x512 to
// 224x224x64: never more than 2 % ahead, 64 x 64 up to twice slower -- a wave's four blocks are four chains on one SIMD.)
int launch_sconv_small_shape(const Im2colA<true>& img, const FilterB<true>& fb, const float* bias, float* dst, const TensorOut& out,
                             int M, int N, int K) {
    return img.dpitch % 64 == 0 ? launch_sconv_small<SconvSmallShape<1, 1, 64, 3>>(img, fb, bias, dst, out, M, N, K)
                                : launch_sconv_small<SconvSmallShape<1, 1, 32, 4>>(img, fb, bias, dst, out, M, N, K);
}

}  // namespace decx_hip
