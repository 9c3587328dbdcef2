// extern "C" entry points of libdecx_hip_probe.so and the copy kernel.
#include <hip/hip_runtime.h>
#include "hgemm_probe_impl.hpp"

namespace decx_hip_probe {
// Plain streaming copy, 16 bytes per lane and iteration: the known-size kernel that hardware traffic counters
// (FETCH_SIZE / WRITE_SIZE) are calibrated against.
__global__ __launch_bounds__(256) void copy_kernel(f32x4* __restrict__ dst, const f32x4* __restrict__ src, size_t quads) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < quads; i += stride) dst[i] = src[i];
}
}  // namespace decx_hip_probe

extern "C" {

int decx_probe_hgemm(int kind, int ablate, void* stream, const uint16_t* A, int lda, const uint16_t* B, int ldb, uint16_t* D,
                     int ldd, int M, int N, int K, int group_m, int grid) {
    using namespace decx_hip_probe;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (kind) {
        case 0: return (ablate & 48) ? probe_kind0_orders(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid)
                                     : probe_kind0(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        case 1: return probe_kind1(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        case 2: return probe_kind2(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        case 3: return probe_kind3(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        case 4: return probe_kind4(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        case 6: return probe_kind6(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        case 5: return probe_kind5(ablate, s, A, lda, B, ldb, D, ldd, M, N, K, group_m, grid);
        default: return 0x0d;
    }
}

int decx_probe_copy(void* stream, void* dst, const void* src, size_t bytes) {
    using namespace decx_hip_probe;
    if (!dst || !src || bytes % 16 != 0 || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15)) return 0x0d;
    if (bytes == 0) return 0;
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return 1000 + (int)e;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipLaunchKernelGGL(copy_kernel, dim3(cus > 0 ? cus * 8 : 2048), dim3(256), 0, s, static_cast<decx_hip::f32x4*>(dst),
                       static_cast<const decx_hip::f32x4*>(src), bytes / 16);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    return e == hipSuccess ? 0 : 1000 + (int)e;
}

}  // extern "C"
