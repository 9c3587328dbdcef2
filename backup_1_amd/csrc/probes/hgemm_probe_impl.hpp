// One build ("kind") of the large fp16 tile kernel in its measurement variants; each kind is a translation unit of its
// own (hgemm_probe_k*.hip define DECX_PROBE_KIND and include this file) so that they compile side by side.
#pragma once
#include <hip/hip_runtime.h>
#include "../hgemm_mfma16_tile.hpp"
#include "decx_hip_probe.h"

namespace decx_hip_probe {
using namespace decx_hip;

typedef void (*HgemmKernel)(const _Float16*, int, const _Float16*, int, const _Float16*, int, _Float16*, int, int, int, int, int, int, int,
                            size_t, size_t, size_t, size_t);

template <class S, bool PERSIST, int... ABLATES>
struct Variants {
    static HgemmKernel pick(int ablate) {
        HgemmKernel k = nullptr;
        ((ablate == ABLATES ? (void)(k = hgemm_mfma16_kernel<S, false, ABLATES, PERSIST>) : (void)0), ...);
        return k;
    }
};

template <class S, bool PERSIST, class V>
int launch(int ablate, hipStream_t stream, const uint16_t* A, int lda, const uint16_t* B, int ldb, uint16_t* D, int ldd, int M, int N,
           int K, int group_m, int grid) {
    HgemmKernel kern = V::pick(ablate);
    if (!kern) return 0x0d;
    if (M <= 0 || N <= 0 || K <= 0 || M % S::BM || N % S::BN || K % S::BK || K < S::BK * S::STAGES) return 0x0d;
    if (PERSIST && K % (S::BK * S::WALK)) return 0x0d;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15 || lda % 8 || ldb % 8 || lda < K || ldb < N || ldd < N) return 0x0d;
    if ((size_t)lda * S::BM * 2 >= ((size_t)1 << 32) || (size_t)ldb * S::BK * 2 >= ((size_t)1 << 32)) return 0x0d;
    const size_t lds = PERSIST ? S::PERSIST_LDS_BYTES : S::LDS_BYTES;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return 1000 + (int)e;
    const int tiles_m = M / S::BM, tiles_n = N / S::BN, total = tiles_m * tiles_n;
    if (group_m <= 0) group_m = 8;
    if (group_m > tiles_m) group_m = tiles_m;
    unsigned blocks = (unsigned)total;
    if (PERSIST) {
        if (grid <= 0) {
            int dev = 0, cus = 0;
            if ((e = hipGetDevice(&dev)) != hipSuccess) return 1000 + (int)e;
            if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return 1000 + (int)e;
            grid = cus;
        }
        blocks = (unsigned)(grid < total ? grid : total);
    }
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(S::NT), lds, stream, reinterpret_cast<const _Float16*>(A), lda,
                       reinterpret_cast<const _Float16*>(B), ldb, static_cast<const _Float16*>(nullptr), 0,
                       reinterpret_cast<_Float16*>(D), ldd, M, N, K, tiles_m, tiles_n, group_m, (size_t)0, (size_t)0, (size_t)0, (size_t)0);
    e = hipGetLastError();
    return e == hipSuccess ? 0 : 1000 + (int)e;
}

typedef Hgemm16Shape<256, 256, 64, 2, 4, 2> Shape2x64;
typedef Hgemm16Shape<256, 256, 32, 2, 4, 4> Shape4x32;
typedef Hgemm16Shape<256, 256, 32, 2, 4, 5> Shape5x32;
typedef Hgemm16Shape<256, 256, 32, 2, 2, 4> ShapeFat4x32;
typedef Hgemm16Shape<256, 256, 64, 2, 2, 2> ShapeFat;     // 4 waves of 128 x 128, one per SIMD

int probe_kind0(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind0_orders(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind1(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind2(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind3(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind4(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind6(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);
int probe_kind5(int, hipStream_t, const uint16_t*, int, const uint16_t*, int, uint16_t*, int, int, int, int, int, int);

#define DECX_PROBE_DEFINE(NAME, SHAPE, PERSIST, ...)                                                                              \
    int NAME(int ablate, hipStream_t stream, const uint16_t* A, int lda, const uint16_t* B, int ldb, uint16_t* D, int ldd, int M, \
             int N, int K, int group_m, int grid) {                                                                               \
        return launch<SHAPE, PERSIST, Variants<SHAPE, PERSIST, __VA_ARGS__>>(ablate, stream, A, lda, B, ldb, D, ldd, M, N, K,     \
                                                                             group_m, grid);                                      \
    }

}  // namespace decx_hip_probe
