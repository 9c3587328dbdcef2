// C ABI of libdecx_hip.so: device bring-up, memory, and the dispatch of the GEMM / convolution kernels.
// Declarations and the reference interface each entry point stands in for: include/decx_hip.h.
#include "../../include/decx_hip.h"

#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "hgemm_dma_tile.hpp"
#include "hgemm_tile.hpp"
#include "sgemm_tile.hpp"
#include "sgemm_chain16.hpp"
#include "conv_chain16.hpp"
#include "hconv_tile.hpp"
#include "hconv_dma.hpp"
#include "hconv_taprow.hpp"

using namespace decx_hip;

namespace {

struct Runtime {
    bool is_init = false;
    int device = -1;
    int compute_units = 0;
    int clock_khz = 0;
    size_t hbm_bytes = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int sgemm_variant = 0;
    int hgemm_variant = 0;
    float* partial = nullptr;      // fp32 workspace of the fp16 split-K path, grown on demand, kept until the process ends
    size_t partial_bytes = 0;
    int group_m = 8;   // tile-rows per raster group of the XCD-aware tile walk (env DECX_HIP_GROUP_M overrides, for tuning)
};
Runtime g_rt;

thread_local char g_err[512] = "No error\n";   // SUCCESS string of the reference, core/error.h:61

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    return fail(DECX_HIP_FAIL_HIP_BASE + (int)e, "%s: %s\n", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

int need_init() { return fail(DECX_HIP_FAIL_NOT_INIT, "CUDA should be initialized first\n"); }   // core/error.h:60

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// A batch of `count` independent, equally shaped problems; the strides are in elements between consecutive problems.
// Every launcher enqueues on `stream`.
struct Batch {
    int count = 1;
    size_t stride_a = 0, stride_b = 0, stride_c = 0, stride_d = 0;
    hipStream_t stream = nullptr;
};

// ---------------------------------------------------------------------------------------------------------------
// fp32 launchers
// ---------------------------------------------------------------------------------------------------------------
template <class S, class ASrc, class BSrc, class Out, bool HAS_C>
int launch_sgemm_tile_c(const ASrc& a, const BSrc& b, const float* Cin, int ldc, float* D, const Out& out, int M, int N,
                        int K, const Batch& batch) {
    auto kern = sgemm_tile_kernel<S, ASrc, BSrc, Out, HAS_C>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)S::template lds_bytes<BSrc>()));
        attr_done = true;
    }
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL || batch.count > 65535) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)batch.count), dim3(S::NT), S::template lds_bytes<BSrc>(), batch.stream, a, b, Cin,
                       ldc, D, out, M, N, K, tiles_m, tiles_n, group_m, batch.stride_c, batch.stride_d, 0);
    HIP_TRY(hipGetLastError());
    return 0;
}

// zero-fills the M x N region of a pitched matrix (the split-K kernel accumulates into it)
__global__ __launch_bounds__(256) void zero_region_kernel(float* D, int ldd, int M, int N) {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        D[(i / N) * ldd + i % N] = 0.f;
}

// Split-K launch of one tile shape: `splits` K ranges of k_split_len each accumulate into D with atomics.
template <class S>
int launch_sgemm_splitk(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                        int N, int K, int splits, int k_split_len) {
    typedef DenseA<true> ASrc;
    typedef DenseB<true> BSrc;
    const bool in_place = Cin == D;               // D already holds C: accumulate straight onto it
    const bool add_c = Cin != nullptr && !in_place;
    auto kern = add_c ? sgemm_tile_kernel<S, ASrc, BSrc, DenseOut, true, true> : sgemm_tile_kernel<S, ASrc, BSrc, DenseOut, false, true>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_tile_kernel<S, ASrc, BSrc, DenseOut, true, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::template lds_bytes<BSrc>()));
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_tile_kernel<S, ASrc, BSrc, DenseOut, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::template lds_bytes<BSrc>()));
        attr_done = true;
    }
    if (!in_place) {
        const size_t total = (size_t)M * N;
        const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
        hipLaunchKernelGGL(zero_region_kernel, dim3(blocks), dim3(256), 0, g_rt.stream, D, ldd, M, N);
    }
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    ASrc a{A, lda, M, K, 0};
    BSrc b{B, ldb, N, K, 0};
    DenseOut out{ldd};
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), 1, (unsigned)splits), dim3(S::NT), S::template lds_bytes<BSrc>(), g_rt.stream, a,
                       b, Cin, ldc, D, out, M, N, K, tiles_m, tiles_n, group_m, (size_t)0, (size_t)0, k_split_len);
    HIP_TRY(hipGetLastError());
    return 0;
}

template <class S, class ASrc, class BSrc, class Out>
int launch_sgemm_tile(const ASrc& a, const BSrc& b, const float* Cin, int ldc, float* D, const Out& out, int M, int N,
                      int K, const Batch& batch) {
    if (Cin != nullptr) return launch_sgemm_tile_c<S, ASrc, BSrc, Out, true>(a, b, Cin, ldc, D, out, M, N, K, batch);
    return launch_sgemm_tile_c<S, ASrc, BSrc, Out, false>(a, b, Cin, ldc, D, out, M, N, K, batch);
}

// Tile shapes (variant numbers of decx_hip_set_sgemm_variant; results are identical for all of them):
//   1: 256x256x16, 2x2 waves of 128x128   -- one wave per SIMD, highest reuse per LDS byte
//   2: 128x128x16, 2x2 waves of  64x64    -- mid-size problems, several workgroups per CU
//   3: 256x128x16, 2x2 waves of 128x64    -- narrow N
//   4: 224x128x16, 1x4 waves of 224x32    -- 7/8 of shape 3 per tile: fills more CUs when M/256 tiles leave many idle
//   5, 6: shapes 3 and 4 compiled for one wave per SIMD (512 registers, two staging sets) -- for long K walks and for
//         launches that put at most one workgroup on a CU anyway
//   7: 256x256x16, 4x2 waves of  64x128   -- two waves per SIMD: the matrix pipe takes the next MFMA from the other wave
//         while one wave issues its loads and LDS traffic (a lone wave leaves ~3.5 idle cycles between 64-cycle MFMAs);
//         the default for large problems, 1-2 % ahead of shape 1
//   8:  64x64x16,  2x2 waves of  32x32    -- small problems: 1024^3 has only 64 tiles of 128x128 for 256 CUs
//   9: 128x64x16,  2x2 waves of  64x32
//  10: 224x256x16, 1x8 waves of 224x32    -- two waves per SIMD like 7; 7/8 of its tile, for tile counts that 7 rounds badly
//  14: 192x192x16, 2x2 waves of  96x96    -- dense GEMM only: sizes that 256 and 128 divide into a bad number of tiles
//         (3072^2 is 144 tiles of 256^2, 576 of 128^2, and exactly 256 of these)
//  15: 224x128x16, 2x4 waves of 128x32 (upper row) and 96x32 (lower row) -- shape 6 on two waves per SIMD: each SIMD
//         carries a 4-block and a 3-block wave
// and, for dense GEMM only, the one-wave-per-16x16-block kernel of sgemm_chain16.hpp:
//  11:  32x32x64,  2x2 computing + 4 moving waves, two workgroups per CU -- results too small to fill the chip with tiles
//  12:  16x16x64,  1 computing + 2 moving waves -- at most one 16x16 block per CU: the fastest a single chain can walk K
//  13:  64x64x64,  8 computing waves of two blocks each + 4 moving waves -- results of about one such tile per CU (1024^2)
typedef SgemmShape<256, 256, 16, 2, 2> SShapeBig;
typedef SgemmShape<128, 128, 16, 2, 2, 2> SShapeSmall;
typedef SgemmShape<256, 128, 16, 2, 2, 2> SShapeTall;
typedef SgemmShape<224, 128, 16, 1, 4, 2> SShape224;
typedef SgemmShape<256, 128, 16, 2, 2, 1> SShapeTallSolo;
typedef SgemmShape<224, 128, 16, 1, 4, 1> SShape224Solo;
typedef SgemmShape<256, 256, 16, 4, 2, 2, 2> SShapeBig8;
typedef SgemmShape<224, 256, 16, 1, 8, 2, 2> SShape224Wide;   // 8 waves of 224x32, two per SIMD
typedef SgemmShape<192, 192, 16, 2, 2, 1> SShape192;
typedef SgemmShape<224, 128, 16, 2, 4, 2, 2, true> SShape224Split;   // 8 waves, 4 + 3 row blocks per SIMD
typedef SgemmShape<64, 64, 16, 2, 2, 4> SShapeTiny;      // 2x2 waves of 32x32
typedef SgemmShape<128, 64, 16, 2, 2, 4> SShapeTiny2;    // 2x2 waves of 64x32

// Tile shape by a small cost model: a CU works through ceil(tiles / CUs) tiles one after another (tiles that share a CU
// share its matrix pipe, so residency does not change this), a tile costs its area divided by how well that shape keeps
// the pipe busy (measured on large squares, relative to shape 7).  The 256x128 and 224x128 shapes come in a
// two-workgroups-per-CU build, better on short K walks where one tile's prologue and epilogue overlap the other's loop,
// and a one-workgroup-per-CU build with deeper prefetch, better on long ones (224x128: shape 15, which measured 5-6 %
// ahead of shape 6 on the 224x224x64 convolution under 128 filters; the same split of the 224x256 tile, and 256x128 on
// 8 waves of 128x32, measured no better than shapes 10 and 5 and are not built).
int pick_sgemm_variant(int M, int N, int K, int batch, bool dense = false) {
    if ((g_rt.sgemm_variant >= 1 && g_rt.sgemm_variant <= 10) || g_rt.sgemm_variant == 15) return g_rt.sgemm_variant;
    if (g_rt.sgemm_variant == 14) return dense ? 14 : 2;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    struct Cand { int variant, bm, bn; double eff; };
    const Cand cands[] = {{7, 256, 256, 1.00}, {10, 224, 256, 0.96}, {3, 256, 128, 0.95}, {4, 224, 128, 0.94}, {2, 128, 128, 0.89},
                          {9, 128, 64, 0.83}, {8, 64, 64, 0.78}, {14, 192, 192, 0.93}};
    int best = 7;
    double best_cost = 0.0;
    for (const Cand& c : cands) {
        if (c.variant == 14 && !dense) continue;
        const long tiles = (long)cdiv(M, c.bm) * cdiv(N, c.bn) * batch;
        const double cost = (double)((tiles + cus - 1) / cus) * c.bm * c.bn / c.eff;
        if (best_cost == 0.0 || cost < best_cost) {
            best_cost = cost;
            const bool one_per_cu = tiles <= cus || K >= 1024;
            best = one_per_cu && c.variant == 3 ? 5 : one_per_cu && c.variant == 4 ? 15 : c.variant;
        }
    }
    return best;
}

template <class ASrc, class BSrc, class Out>
int dispatch_sgemm(int variant, const ASrc& a, const BSrc& b, const float* Cin, int ldc, float* D, const Out& out, int M,
                   int N, int K, const Batch& batch) {
    switch (variant) {
        case 1: return launch_sgemm_tile<SShapeBig>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 3: return launch_sgemm_tile<SShapeTall>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 4: return launch_sgemm_tile<SShape224>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 5: return launch_sgemm_tile<SShapeTallSolo>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 6: return launch_sgemm_tile<SShape224Solo>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 7: return launch_sgemm_tile<SShapeBig8>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 8: return launch_sgemm_tile<SShapeTiny>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 9: return launch_sgemm_tile<SShapeTiny2>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 10: return launch_sgemm_tile<SShape224Wide>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 15: return launch_sgemm_tile<SShape224Split>(a, b, Cin, ldc, D, out, M, N, K, batch);
        default: return launch_sgemm_tile<SShapeSmall>(a, b, Cin, ldc, D, out, M, N, K, batch);
    }
}

int check_gemm_args(const void* A, int lda, const void* B, int ldb, const void* Cin, int ldc, const void* D, int ldd, int M,
                    int N, int K, const Batch& batch) {
    if (!g_rt.is_init) return need_init();
    if (!A || !B || !D) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null matrix pointer\n");
    if (M <= 0 || N <= 0 || K <= 0 || batch.count <= 0) return fail(DECX_HIP_FAIL_DIMS, "Matrix Dims don't match each other");
    if (lda < K || ldb < N || ldd < N || (Cin && ldc < N))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "leading dimension smaller than the row length\n");
    if (batch.count > 1 && (batch.stride_a < (size_t)(M - 1) * lda + K || batch.stride_b < (size_t)(K - 1) * ldb + N ||
                            batch.stride_d < (size_t)(M - 1) * ldd + N || (Cin && batch.stride_c < (size_t)(M - 1) * ldc + N)))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "batch stride smaller than one matrix\n");
    return 0;
}

// One wave per 16x16 block (sgemm_chain16.hpp): for results with few tiles and a long K.
template <class S>
int launch_sgemm_chain16(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                         int N, int K, const Batch& batch, bool relu) {
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL || batch.count > 65535) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    auto kern = Cin ? sgemm_chain16_kernel<S, true> : sgemm_chain16_kernel<S, false>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_chain16_kernel<S, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(sgemm_chain16_kernel<S, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)batch.count), dim3(S::NT), S::LDS_BYTES, batch.stream, A, lda, B, ldb,
                       Cin, ldc, D, ldd, M, N, K, tiles_n, relu, batch.stride_a, batch.stride_b, batch.stride_c, batch.stride_d);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Which shape of the one-wave-per-block kernel (sgemm_chain16.hpp) a result of M x N takes, or 0 for the tiles.
// Measured: ahead of the tiles up to about ten 32x32 tiles per CU -- 1536x1536 on 256 CUs -- 1.7x at 1024x8192x1024, 9x at
// 64x65536x1024.  All paths give the same bits, so this is a choice of speed only.
int pick_chain_shape(int M, int N, int K, int batch) {
    if (g_rt.sgemm_variant >= 11 && g_rt.sgemm_variant <= 13) return g_rt.sgemm_variant;
    if ((g_rt.sgemm_variant >= 1 && g_rt.sgemm_variant <= 10) || g_rt.sgemm_variant >= 14) return 0;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long blocks16 = (long)cdiv(M, 16) * cdiv(N, 16) * batch, tiles32 = (long)cdiv(M, 32) * cdiv(N, 32) * batch;
    // In units of one round of 32x32 tiles (two per CU, 512 on 256 CUs): a round of 64x64 tiles (one per CU) costs
    // 1.55, further rounds of 32x32 tiles overlap with the first and cost 0.9 each once there is more than
    // one (measured on squares of 640 .. 2560 at K = 512 and 2048).  Beyond 10 (K < 1024: 4) 32x32 tiles per CU
    // the 32x32x2 tiles are ahead -- the block-chain kernels have the longer prologue.
    const long tiles64 = (long)cdiv(M, 64) * cdiv(N, 64) * batch;
    const double cost64 = 1.55 * (double)((tiles64 + cus - 1) / cus), pairs = (double)tiles32 / (2.0 * cus);
    const double cost32 = pairs <= 1.0 ? 1.0 : 0.9 * (pairs + 0.5);
    const long tile_limit = (K >= 1024 ? 10 : 4) * cus;
    return blocks16 <= cus ? 12 : tiles32 > tile_limit ? 0 : cost64 < cost32 ? 13 : 11;
}

int sgemm_enqueue(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                  int N, int K, const Batch& batch, bool relu = false) {
    if (int rc = check_gemm_args(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch)) return rc;
    const int variant = pick_sgemm_variant(M, N, K, batch.count, true);
    const bool vec_a = aligned16(A) && lda % 4 == 0 && batch.stride_a % 4 == 0;
    const bool vec_b = aligned16(B) && ldb % 4 == 0 && ldb >= 4 && batch.stride_b % 4 == 0;
    DenseOut out{ldd, relu, aligned16(D) && ldd % 4 == 0 && batch.stride_d % 4 == 0};
    if (vec_a && vec_b) {
        const int chain = pick_chain_shape(M, N, K, batch.count);
        if (chain == 11) return launch_sgemm_chain16<Chain16<2, 1, 4, 4>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
        if (chain == 12) return launch_sgemm_chain16<Chain16<1, 1, 8, 2>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
        if (chain == 13) return launch_sgemm_chain16<Chain16<4, 2, 2, 3>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    }
    if (vec_a && vec_b) {
        DenseA<true> a{A, lda, M, K, batch.stride_a};
        DenseB<true> b{B, ldb, N, K, batch.stride_b};
        if (variant == 14) return launch_sgemm_tile<SShape192>(a, b, Cin, ldc, D, out, M, N, K, batch);
        return dispatch_sgemm(variant, a, b, Cin, ldc, D, out, M, N, K, batch);
    }
    // unaligned operands: element-wise loaders, one tile shape only
    DenseA<false> a{A, lda, M, K, batch.stride_a};
    DenseB<false> b{B, ldb, N, K, batch.stride_b};
    return launch_sgemm_tile<SShapeSmall>(a, b, Cin, ldc, D, out, M, N, K, batch);
}

// Split-K GEMM for problems whose M x N tile count leaves most CUs idle while K is long (the short-M / long-K shapes of
// GEMM_Long_Lr, or a 1024^3 square).  splits <= 0 picks a count that fills the CUs about twice over.
int sgemm_splitk_enqueue(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                         int N, int K, int splits) {
    Batch one;
    one.stream = g_rt.stream;
    if (int rc = check_gemm_args(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, one)) return rc;
    if (!(aligned16(A) && aligned16(B) && lda % 4 == 0 && ldb % 4 == 0 && ldb >= 4))
        return sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, one);            // unaligned: plain path
    const bool big_tiles = (long)cdiv(M, 256) * cdiv(N, 128) >= 16 && M > 128;
    const int bm = big_tiles ? 256 : 128, bk = 16;
    const long tiles = (long)cdiv(M, bm) * cdiv(N, 128);
    const int cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const int max_splits = cdiv(K, 8 * bk) < 1024 ? cdiv(K, 8 * bk) : 1024;              // at least 8 K steps per range
    if (splits <= 0) splits = (int)((2L * cus + tiles - 1) / tiles);
    if (splits > max_splits) splits = max_splits;
    if (splits <= 1) return sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, one);
    const int k_split_len = cdiv(cdiv(K, splits), bk) * bk;
    splits = cdiv(K, k_split_len);                                                        // no empty range
    if (big_tiles) return launch_sgemm_splitk<SShapeTall>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, splits, k_split_len);
    return launch_sgemm_splitk<SShapeSmall>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, splits, k_split_len);
}

template <class S>
int launch_conv_chain16(const Im2colA<false>& img, const FilterB<false>& fb, const float* bias, float* dst, const TensorOut& out,
                        int M, int N, int K) {
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(conv_chain16_kernel<S>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)S::LDS_BYTES));
        attr_done = true;
    }
    hipLaunchKernelGGL(conv_chain16_kernel<S>, dim3((unsigned)total), dim3(S::NT), S::LDS_BYTES, g_rt.stream, img, fb, bias, dst, out,
                       M, N, K, tiles_n);
    HIP_TRY(hipGetLastError());
    return 0;
}

int conv_enqueue(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt, int N, int kh,
                 int kw, size_t filt_stride, size_t filt_row_stride, float* dst, int dst_dpitch, size_t dst_row_stride,
                 int flag, const float* bias = nullptr, bool relu = false) {
    if (!g_rt.is_init) return need_init();
    if (flag != DECX_HIP_CONV_NO_COMPENSATE && flag != DECX_HIP_CONV_ZERO_COMPENSATE)
        return fail(DECX_HIP_FAIL_ERROR_FLAG, "This flag is meaningless in current context\n");   // core/error.h:67
    if (!src || !filt || !dst) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null tensor pointer\n");
    if (H <= 0 || W <= 0 || N <= 0 || kh <= 0 || kw <= 0 || dpitch <= 0)
        return fail(DECX_HIP_FAIL_DIMS, "Tensor Dims don't match each other");
    if (dpitch % 4 != 0 || src_row_stride % 4 != 0 || filt_stride % 4 != 0 || filt_row_stride % 4 != 0 ||
        !aligned16(src) || !aligned16(filt))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "tensors must be 16-byte aligned with channel pitch a multiple of 4\n");
    const int Hout = flag ? H : H - 2 * (kh / 2), Wout = flag ? W : W - 2 * (kw / 2);
    if (Hout <= 0 || Wout <= 0) return fail(DECX_HIP_FAIL_DIMS, "kernel larger than the image\n");
    if (src_row_stride < (size_t)W * dpitch || filt_row_stride < (size_t)kw * dpitch ||
        filt_stride < (size_t)(kh - 1) * filt_row_stride + (size_t)kw * dpitch || dst_dpitch < N ||
        dst_row_stride < (size_t)Wout * dst_dpitch)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "stride smaller than the extent it spans\n");
    const long Ml = (long)Hout * Wout, Kl = (long)kh * kw * dpitch;
    if (Ml > 0x7fffffffL || Kl > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large\n");
    const int M = (int)Ml, K = (int)Kl;
    // the loaders address both tensors with 32-bit byte offsets through buffer resources
    const size_t src_bytes = ((size_t)(H - 1) * src_row_stride + (size_t)W * dpitch) * sizeof(float);
    const size_t filt_bytes = ((size_t)(N - 1) * filt_stride + (size_t)(kh - 1) * filt_row_stride + (size_t)kw * dpitch) * sizeof(float);
    if (src_bytes >= 0x80000000ull || filt_bytes >= 0x80000000ull)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "source tensor and filter bank must each stay below 2 GiB\n");
    TensorOut out{Wout, dst_dpitch, dst_row_stride, dst_row_stride == (size_t)Wout * dst_dpitch, relu};
    Batch one;
    one.stream = g_rt.stream;
    const int variant = pick_sgemm_variant(M, N, K, 1);
    const int oy = flag ? kh / 2 : 0, ox = flag ? kw / 2 : 0;
    // a bias is the "+ C" operand with row stride 0: every output pixel adds the same N values
    // small images: too few tiles for the chip, the one-wave-per-block kernel takes them (conv_chain16.hpp)
    if (const int chain = pick_chain_shape(M, N, K, 1)) {
        Im2colA<false> a{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes};
        FilterB<false> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
        if (chain == 11) return launch_conv_chain16<Chain16<2, 1, 4, 4>>(a, b, bias, dst, out, M, N, K);
        if (chain == 12) return launch_conv_chain16<Chain16<1, 1, 8, 2>>(a, b, bias, dst, out, M, N, K);
        return launch_conv_chain16<Chain16<4, 2, 2, 3>>(a, b, bias, dst, out, M, N, K);
    }
    if (dpitch % 16 == 0) {      // a whole K step inside one tap: the tap walk runs on the scalar unit
        Im2colAUniform a{{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes}};
        FilterBUniform b{{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes}};
        return dispatch_sgemm(variant, a, b, bias, 0, dst, out, M, N, K, one);
    }
    if (dpitch % 8 == 0) {       // the 8 consecutive k of a staging task never straddle a tap
        Im2colA<true> a{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes};
        FilterB<true> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
        return dispatch_sgemm(variant, a, b, bias, 0, dst, out, M, N, K, one);
    }
    Im2colA<false> a{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes};
    FilterB<false> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
    return dispatch_sgemm(variant, a, b, bias, 0, dst, out, M, N, K, one);
}

// ---------------------------------------------------------------------------------------------------------------
// fp16 launchers
// ---------------------------------------------------------------------------------------------------------------
// Tile shapes (variant numbers of decx_hip_set_hgemm_variant):
//   1: 256x256x32, 2x2 waves of 128x128, register-staged
//   2: 128x128x32, 2x2 waves of  64x64, register-staged (also the element-wise loader for unaligned operands)
//   3: 256x256x32, 2x2 waves of 128x128, 4-stage LDS-DMA pipeline
//   4: 256x256x64, 2x2 waves of 128x128, 2-stage LDS-DMA pipeline (whole 128-byte lines of A per row and step)
//   5: 256x256x32, 2x2 waves of 128x128, 5-stage LDS-DMA pipeline
//   8: 128x128x64, 2x2 waves of 64x64, 2-stage LDS-DMA pipeline (64 KB of LDS: two workgroups per CU) -- mid-size problems
//   9: as 8 with 3 stages (one workgroup per CU) -- small problems
//  10: 256x128x64, 2x2 waves of 128x64, 2-stage LDS-DMA pipeline
//   6: as 4 with 4x2 waves of 64x128 (two waves per SIMD)
//   7: as 4 with 2x4 waves of 128x64 (two waves per SIMD) -- the default for large problems: the chip is power-capped on
//      this kernel (MFMA busy x clock stays ~1.27 GHz-equivalents whatever the schedule), and this one is 1 % ahead
//  11: split-K on shape 8 through an fp32 workspace (hgemm_splitk_enqueue) -- few tiles and a long K
// and, for the fp16 convolution only: 12 keeps its register-staged kernels, 13 takes its LDS-DMA kernel for any image
// whose channel pitch allows it, 14 its tap-row kernel; each switches its split over K off (experiments and tests)
typedef HgemmShape<256, 256, 32, 2, 2> HShapeBig;
typedef HgemmShape<128, 128, 32, 2, 2> HShapeSmall;
typedef HgemmDmaShape<256, 256, 32, 2, 2, 4> HShapeDma;
typedef HgemmDmaShape<256, 256, 64, 2, 2, 2> HShapeDma64;
typedef HgemmDmaShape<256, 256, 32, 2, 2, 5> HShapeDma5;
typedef HgemmDmaShape<256, 256, 64, 4, 2, 2> HShapeDma64W8a;     // 8 waves, 64x128 each
typedef HgemmDmaShape<256, 256, 64, 2, 4, 2> HShapeDma64W8b;     // 8 waves, 128x64 each
typedef HgemmDmaShape<128, 128, 64, 2, 2, 2> HShapeDmaSmall;     // 4 waves, 64x64 each, 64 KB of LDS: two workgroups per CU
typedef HgemmDmaShape<128, 128, 64, 2, 2, 3> HShapeDmaSmall3;
typedef HgemmDmaShape<256, 128, 64, 2, 2, 2> HShapeDmaTall;      // 4 waves, 128x64 each

template <class S, bool VEC>
int launch_hgemm_tile(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                      int ldd, int M, int N, int K, const Batch& batch) {
    auto kern = hgemm_tile_kernel<S, VEC>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)S::LDS_BYTES));
        attr_done = true;
    }
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL || batch.count > 65535) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)batch.count), dim3(S::NT), S::LDS_BYTES, batch.stream,
                       reinterpret_cast<const _Float16*>(A), lda, reinterpret_cast<const _Float16*>(B), ldb,
                       reinterpret_cast<const _Float16*>(Cin), ldc, reinterpret_cast<_Float16*>(D), ldd, M, N, K,
                       tiles_m, tiles_n, group_m, batch.stride_a, batch.stride_b, batch.stride_c, batch.stride_d);
    HIP_TRY(hipGetLastError());
    return 0;
}

template <class S>
int launch_hgemm_dma_tile(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                          uint16_t* D, int ldd, int M, int N, int K, const Batch& batch) {
    auto kern = Cin ? hgemm_dma_kernel<S, true> : hgemm_dma_kernel<S, false>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_dma_kernel<S, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_dma_kernel<S, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL || batch.count > 65535) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)total, (unsigned)batch.count), dim3(S::NT), S::LDS_BYTES, batch.stream,
                       reinterpret_cast<const _Float16*>(A), lda, reinterpret_cast<const _Float16*>(B), ldb,
                       reinterpret_cast<const _Float16*>(Cin), ldc, reinterpret_cast<_Float16*>(D), ldd, M, N, K,
                       tiles_m, tiles_n, group_m, batch.stride_a, batch.stride_b, batch.stride_c, batch.stride_d,
                       static_cast<float*>(nullptr), 0);
    HIP_TRY(hipGetLastError());
    return 0;
}

// the fp32 workspace of the fp16 split-K paths: grown on demand, kept until the process ends
int ensure_partial(size_t need) {
    if (need <= g_rt.partial_bytes) return 0;
    HIP_TRY(hipDeviceSynchronize());               // earlier launches may still use the old workspace
    if (g_rt.partial) HIP_TRY(hipFree(g_rt.partial));
    g_rt.partial = nullptr;
    g_rt.partial_bytes = 0;
    if (hipMalloc(&g_rt.partial, need) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    }
    g_rt.partial_bytes = need;
    return 0;
}

// fp16 GEMM whose result has too few tiles to fill the chip while K is long: K is cut into ranges that run as separate
// workgroups (blockIdx.z) and add their fp32 partial sums to a workspace with atomics; a second kernel adds C and
// rounds to binary16 once.  fp32 sums in no fixed order: the result can differ in its last bit from run to run, inside
// the 2e-3 rule of the fp16 path.  (fp32 GEMM never does this: its results are bit-exact chains.)
int hgemm_splitk_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                         int ldd, int M, int N, int K, int splits, hipStream_t stream) {
    typedef HShapeDmaSmall S;                      // 128x128x64, LDS-DMA staged, two workgroups per CU
    if (int rc = ensure_partial((size_t)M * N * sizeof(float))) return rc;
    auto kern = hgemm_dma_kernel<S, false, true>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    const size_t total = (size_t)M * N;
    const unsigned fill_blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(zero_region_kernel, dim3(fill_blocks), dim3(256), 0, stream, g_rt.partial, N, M, N);
    const int k_split_len = cdiv(cdiv(K, splits), S::BK) * S::BK;
    splits = cdiv(K, k_split_len);                                                        // no empty range
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), 1, (unsigned)splits), dim3(S::NT), S::LDS_BYTES, stream,
                       reinterpret_cast<const _Float16*>(A), lda, reinterpret_cast<const _Float16*>(B), ldb,
                       static_cast<const _Float16*>(nullptr), 0, reinterpret_cast<_Float16*>(D), ldd, M, N, K, tiles_m, tiles_n,
                       group_m, (size_t)0, (size_t)0, (size_t)0, (size_t)0, g_rt.partial, k_split_len);
    hipLaunchKernelGGL(hgemm_split_finish_kernel, dim3(fill_blocks), dim3(256), 0, stream, g_rt.partial,
                       reinterpret_cast<const _Float16*>(Cin), ldc, reinterpret_cast<_Float16*>(D), ldd, M, N);
    HIP_TRY(hipGetLastError());
    return 0;
}

int hgemm_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                  int ldd, int M, int N, int K, const Batch& batch) {
    if (int rc = check_gemm_args(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch)) return rc;
    // the LDS-DMA tiles address a tile's rows with 32-bit byte offsets from the tile's first row: 256 rows of A, 64 of B
    const bool narrow = (size_t)lda * 256 * sizeof(uint16_t) < ((size_t)1 << 32) && (size_t)ldb * 64 * sizeof(uint16_t) < ((size_t)1 << 32);
    const bool vec = aligned16(A) && aligned16(B) && lda % 8 == 0 && ldb % 8 == 0 && ldb >= 8 && batch.stride_a % 8 == 0 &&
                     batch.stride_b % 8 == 0 && narrow;
    if (!vec) return launch_hgemm_tile<HShapeSmall, false>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    int variant = g_rt.hgemm_variant;
    {
        // few 128x128 tiles and a long K: split K (variant 11 forces it, any other fixed variant switches it off).
        // Measured, in us: a tile walks K at 6.7 ns per k (1.6 times that when two workgroups share a CU); a launch costs
        // about 4, the zero fill and the finishing kernel 9 together, an atomic add to the workspace 3.1 ps.
        const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
        const long tiles = (long)cdiv(M, 128) * cdiv(N, 128);
        long splits = (2 * cus + tiles - 1) / tiles;
        if (splits > K / 512) splits = K / 512;                        // at least 8 K steps per range
        if (splits >= 2 && batch.count == 1 && (size_t)M * N <= ((size_t)1 << 26)) {
            const double t_whole = 4.0 + 0.0067 * K * (double)((tiles + cus - 1) / cus);
            const double share = tiles * splits > cus ? 1.6 : 1.0;
            const double t_split = 9.0 + 3.1e-6 * M * N * splits +
                                   0.0067 * ((double)K / splits) * share * (double)((tiles * splits + 2 * cus - 1) / (2 * cus));
            if (variant == 11 || ((variant < 1 || variant > 11) && t_split < 0.85 * t_whole))
                return hgemm_splitk_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, (int)splits, batch.stream);
        }
        if (variant == 11) variant = 0;
    }
    if (variant < 1 || variant > 10) {
        // same cost model as the fp32 picker: rounds of tiles per CU x tile area / measured shape efficiency
        const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
        const long big = (long)cdiv(M, 256) * cdiv(N, 256) * batch.count, small = (long)cdiv(M, 128) * cdiv(N, 128) * batch.count;
        const double cost_big = (double)((big + cus - 1) / cus) * 65536.0;
        const double cost_small = (double)((small + cus - 1) / cus) * 16384.0 / 0.75;
        // the small tile with three LDS stages holds one workgroup per CU: only worth it when there is at most one to hold
        variant = cost_big <= cost_small ? 7 : (small <= cus ? 9 : 8);
    }
    if (variant == 3) return launch_hgemm_dma_tile<HShapeDma>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 4) return launch_hgemm_dma_tile<HShapeDma64>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 5) return launch_hgemm_dma_tile<HShapeDma5>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 6) return launch_hgemm_dma_tile<HShapeDma64W8a>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 7) return launch_hgemm_dma_tile<HShapeDma64W8b>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 8) return launch_hgemm_dma_tile<HShapeDmaSmall>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 9) return launch_hgemm_dma_tile<HShapeDmaSmall3>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 10) return launch_hgemm_dma_tile<HShapeDmaTall>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 1) return launch_hgemm_tile<HShapeBig, true>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    return launch_hgemm_tile<HShapeSmall, true>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
}

// fp16 convolution (hconv_tile.hpp).  Strides and pitches in halves, as the binary16 containers hold them.
typedef HconvShape<128, 128, 2, 2, 4> HconvSquare;   // 2x2 waves of 64x64
typedef HconvShape<256, 128, 4, 2, 4> HconvTall;     // 4x2 waves of 64x64, two per SIMD: half the filter reads per pixel
typedef HconvDmaShape<256, 128, 4, 2, 3> HconvDma;   // the tall tile fed by LDS-DMA loads, three K steps in LDS
int hconv_enqueue(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt, int N, int kh,
                  int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst, int dst_dpitch, size_t dst_row_stride,
                  int flag, const uint16_t* bias, bool relu) {
    if (!g_rt.is_init) return need_init();
    if (flag != DECX_HIP_CONV_NO_COMPENSATE && flag != DECX_HIP_CONV_ZERO_COMPENSATE)
        return fail(DECX_HIP_FAIL_ERROR_FLAG, "This flag is meaningless in current context\n");   // core/error.h:67
    if (!src || !filt || !dst) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null tensor pointer\n");
    if (H <= 0 || W <= 0 || N <= 0 || kh <= 0 || kw <= 0 || dpitch <= 0)
        return fail(DECX_HIP_FAIL_DIMS, "Tensor Dims don't match each other");
    if (dpitch % 8 != 0 || src_row_stride % 8 != 0 || filt_stride % 8 != 0 || filt_row_stride % 8 != 0 || !aligned16(src) ||
        !aligned16(filt))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "tensors must be 16-byte aligned with channel pitch a multiple of 8\n");
    const int Hout = flag ? H : H - 2 * (kh / 2), Wout = flag ? W : W - 2 * (kw / 2);
    if (Hout <= 0 || Wout <= 0) return fail(DECX_HIP_FAIL_DIMS, "kernel larger than the image\n");
    if (src_row_stride < (size_t)W * dpitch || filt_row_stride < (size_t)kw * dpitch ||
        filt_stride < (size_t)(kh - 1) * filt_row_stride + (size_t)kw * dpitch || dst_dpitch < N ||
        dst_row_stride < (size_t)Wout * dst_dpitch)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "stride smaller than the extent it spans\n");
    const long Ml = (long)Hout * Wout, Kl = (long)kh * kw * dpitch;
    if (Ml > 0x7fffffffL || Kl > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large\n");
    const int M = (int)Ml, Kw = (int)(Kl / 2);
    // the loaders address both tensors with 32-bit byte offsets through buffer resources
    const size_t src_bytes = ((size_t)(H - 1) * src_row_stride + (size_t)W * dpitch) * 2;
    const size_t filt_bytes = ((size_t)(N - 1) * filt_stride + (size_t)(kh - 1) * filt_row_stride + (size_t)kw * dpitch) * 2;
    if (src_bytes >= 0x80000000ull || filt_bytes >= 0x80000000ull)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "source tensor and filter bank must each stay below 2 GiB\n");
    const int oy = flag ? kh / 2 : 0, ox = flag ? kw / 2 : 0;
    HalfImage img{src, H, W, kh, kw, oy, ox, Wout, M, dpitch / 2, (int)(src_row_stride / 2), (unsigned)src_bytes};
    HalfFilters fb{filt, N, dpitch / 2, kw, (int)(filt_stride / 2), (int)(filt_row_stride / 2), (unsigned)filt_bytes};
    HalfTensorOut out{reinterpret_cast<_Float16*>(dst), Wout, dst_dpitch, dst_row_stride, reinterpret_cast<const _Float16*>(bias), relu};
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    // the tall tile (half the filter traffic per pixel) once its workgroups cover most of the chip: measured 4 % ahead at
    // 196 tiles on 256 CUs, where the square tile has 392
    const bool tall = (long)cdiv(M, 256) * cdiv(N, 128) >= 3 * cus / 4;
    const int bm = tall ? 256 : 128, tiles_n = cdiv(N, 128);
    const long total = (long)cdiv(M, bm) * tiles_n;
    if (total > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    // a K step of 64 halves inside one tap: the tap walk runs on the scalar unit (hconv_tile.hpp)
    const bool tap_uniform = dpitch % 64 == 0;
    static bool attr_done = false;
    if (!attr_done) {
        auto allow = [](const void* kern, size_t bytes) { return hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes); };
        HIP_TRY(allow(reinterpret_cast<const void*>(hconv_tile_kernel<HconvTall, true>), HconvTall::LDS_BYTES));
        HIP_TRY(allow(reinterpret_cast<const void*>(hconv_tile_kernel<HconvTall, false>), HconvTall::LDS_BYTES));
        HIP_TRY(allow(reinterpret_cast<const void*>(hconv_tile_kernel<HconvSquare, true>), HconvSquare::LDS_BYTES));
        HIP_TRY(allow(reinterpret_cast<const void*>(hconv_tile_kernel<HconvSquare, false>), HconvSquare::LDS_BYTES));
        attr_done = true;
    }
    // small image: few tiles and many K steps -> ranges of K steps as separate workgroups, fp32 partial sums in the
    // workspace, bias / ReLU / rounding in a finishing kernel
    // Measured model, in us: a workgroup walks a K step of 64 halves in 0.75 us (1.3 x that once two workgroups share a
    // CU's LDS bandwidth); the split pays 9 us for fill, finishing kernel and a third launch, and 3.1 ps per atomic add.
    const int all_steps = cdiv(Kw, 32);
    const long square_tiles = (long)cdiv(M, 128) * tiles_n;
    int splits = 1;
    const bool kernel_forced = g_rt.hgemm_variant >= 12 && g_rt.hgemm_variant <= 14;      // experiments and tests: no split
    if (!kernel_forced && !tall && 2 * square_tiles <= cus && all_steps >= 8 && (size_t)M * N <= ((size_t)1 << 26)) {
        const double t_whole = 4.0 + 0.75 * all_steps;
        double best = 0.85 * t_whole;
        const long most = (2 * cus + square_tiles - 1) / square_tiles;
        for (int s = 2; s <= most && s <= all_steps / 2; ++s) {
            const double share = square_tiles * s > cus ? 1.3 : 1.0;
            const double t = 9.0 + 3.1e-6 * M * N * s + 0.75 * share * cdiv(all_steps, s);
            if (t < best) best = t, splits = s;
        }
    }
    if (splits > 1) {
        const int steps_per_split = cdiv(all_steps, splits);
        splits = cdiv(all_steps, steps_per_split);                     // no empty range
        if (int rc = ensure_partial((size_t)M * N * sizeof(float))) return rc;
        static bool split_attr_done = false;
        if (!split_attr_done) {
            HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hconv_tile_kernel<HconvSquare, true, true>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)HconvSquare::LDS_BYTES));
            HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hconv_tile_kernel<HconvSquare, false, true>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)HconvSquare::LDS_BYTES));
            split_attr_done = true;
        }
        const size_t count = (size_t)M * N;
        const unsigned fill_blocks = (unsigned)((count + 255) / 256 < 4096 ? (count + 255) / 256 : 4096);
        hipLaunchKernelGGL(zero_region_kernel, dim3(fill_blocks), dim3(256), 0, g_rt.stream, g_rt.partial, N, M, N);
        const dim3 grid((unsigned)total, (unsigned)splits);
        if (tap_uniform)
            hipLaunchKernelGGL((hconv_tile_kernel<HconvSquare, true, true>), grid, dim3(HconvSquare::NT), HconvSquare::LDS_BYTES,
                               g_rt.stream, img, fb, out, M, N, Kw, tiles_n, g_rt.partial, steps_per_split);
        else
            hipLaunchKernelGGL((hconv_tile_kernel<HconvSquare, false, true>), grid, dim3(HconvSquare::NT), HconvSquare::LDS_BYTES,
                               g_rt.stream, img, fb, out, M, N, Kw, tiles_n, g_rt.partial, steps_per_split);
        hipLaunchKernelGGL(hconv_split_finish_kernel, dim3(fill_blocks), dim3(256), 0, g_rt.stream, g_rt.partial, out, M, N);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    // filters 3, 5 or 7 wide: the LDS-DMA kernel that loads a tap row's pixels once for all of its taps, if a tile's patch
    // fits its 320 rows (255 + kw positions plus kw - 1 per image row the tile touches).  hgemm variant 14 takes it for
    // any image; its tiles are 64 filters wide when there are no more filters than that.
    const int rows_touched = (254 + Wout) / Wout + 1;
    const bool taprow_fits = tap_uniform && (kw == 3 || kw == 5 || kw == 7) && 255 + kw + (kw - 1) * rows_touched <= 320 &&
                             (long)H * W < (1L << 22);
    const bool narrow = N <= 64;
    const bool many_tiles = narrow ? (long)cdiv(M, 256) >= 3 * cus / 4 : tall;
    if (taprow_fits && ((many_tiles && (g_rt.hgemm_variant < 12 || g_rt.hgemm_variant > 13)) || g_rt.hgemm_variant == 14)) {
        auto launch_taprow = [&](auto shape) -> int {
            typedef decltype(shape) S;
            static_assert(S::PATCH_ROWS == 320, "the fit test above is written for this patch");
            static bool attr_done = false;           // one per shape: the lambda's body is instantiated per S
            if (!attr_done) {
                HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hconv_taprow_kernel<S>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                            (int)S::LDS_BYTES));
                attr_done = true;
            }
            const int tn = cdiv(N, S::BN);
            const long tiles = (long)cdiv(M, S::BM) * tn;
            hipLaunchKernelGGL(hconv_taprow_kernel<S>, dim3((unsigned)tiles), dim3(S::NT), S::LDS_BYTES, g_rt.stream, img, fb, out, M, N, tn);
            HIP_TRY(hipGetLastError());
            return 0;
        };
        if (narrow) {      // 8x1 waves of 32 pixels x 64 filters
            if (kw == 3) return launch_taprow(HconvTapRowShape<3, 64, 8, 1>{});
            if (kw == 5) return launch_taprow(HconvTapRowShape<5, 64, 8, 1>{});
            return launch_taprow(HconvTapRowShape<7, 64, 8, 1>{});
        }
        if (kw == 3) return launch_taprow(HconvTapRowShape<3>{});
        if (kw == 5) return launch_taprow(HconvTapRowShape<5>{});
        return launch_taprow(HconvTapRowShape<7>{});
    }
    // at most 64 filters: tiles 64 filters wide (the 128-wide ones would spend half of their MFMAs on filters that do not exist)
    if (narrow && g_rt.hgemm_variant != 13) {
        typedef HconvShape<256, 64, 4, 2, 4> TallNarrow;     // 4x2 waves of 64x32
        typedef HconvShape<128, 64, 2, 2, 4> SquareNarrow;   // 2x2 waves of 64x32
        const bool tall_narrow = many_tiles;
        auto launch_narrow = [&](auto kern, auto shape) -> int {
            typedef decltype(shape) S;
            static bool attr_done = false;           // one per kernel: the lambda's body is instantiated per argument type
            if (!attr_done) {
                HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
                attr_done = true;
            }
            const long tiles = cdiv(M, S::BM);
            hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(S::NT), S::LDS_BYTES, g_rt.stream, img, fb, out, M, N, Kw, 1,
                               static_cast<float*>(nullptr), 0);
            HIP_TRY(hipGetLastError());
            return 0;
        };
        if (tall_narrow && tap_uniform) return launch_narrow(hconv_tile_kernel<TallNarrow, true>, TallNarrow{});
        if (tall_narrow) return launch_narrow(hconv_tile_kernel<TallNarrow, false>, TallNarrow{});
        if (tap_uniform) return launch_narrow(hconv_tile_kernel<SquareNarrow, true>, SquareNarrow{});
        return launch_narrow(hconv_tile_kernel<SquareNarrow, false>, SquareNarrow{});
    }
    // hgemm variant 12 keeps the register-staged kernels, 13 takes the LDS-DMA kernel wherever it can run (experiments)
    if (tap_uniform && g_rt.hgemm_variant != 12 && (tall || g_rt.hgemm_variant == 13)) {
        static bool dma_attr_done = false;
        if (!dma_attr_done) {
            HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hconv_dma_kernel<HconvDma>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)HconvDma::LDS_BYTES));
            dma_attr_done = true;
        }
        const long dma_tiles = (long)cdiv(M, HconvDma::BM) * tiles_n;
        hipLaunchKernelGGL(hconv_dma_kernel<HconvDma>, dim3((unsigned)dma_tiles), dim3(HconvDma::NT), HconvDma::LDS_BYTES, g_rt.stream,
                           img, fb, out, M, N, Kw, tiles_n);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    auto launch = [&](auto kern, auto shape) {
        typedef decltype(shape) S;
        hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(S::NT), S::LDS_BYTES, g_rt.stream, img, fb, out, M, N, Kw, tiles_n,
                           static_cast<float*>(nullptr), 0);
    };
    if (tall && tap_uniform) launch(hconv_tile_kernel<HconvTall, true>, HconvTall{});
    else if (tall) launch(hconv_tile_kernel<HconvTall, false>, HconvTall{});
    else if (tap_uniform) launch(hconv_tile_kernel<HconvSquare, true>, HconvSquare{});
    else launch(hconv_tile_kernel<HconvSquare, false>, HconvSquare{});
    HIP_TRY(hipGetLastError());
    return 0;
}

Batch single_on_library_stream() {
    Batch b;
    b.stream = g_rt.stream;
    return b;
}
Batch batch_on_library_stream(int count, size_t sa, size_t sb, size_t sc, size_t sd) {
    Batch b;
    b.count = count;
    b.stride_a = sa;
    b.stride_b = sb;
    b.stride_c = sc;
    b.stride_d = sd;
    b.stream = g_rt.stream;
    return b;
}

// ---------------------------------------------------------------------------------------------------------------
// Host-resident batches (the MatrixArray GEMM3 of the reference): one matrix triple per pipeline step, two device
// buffer sets, uploads / kernel / downloads on three streams chained by events, so that the copies of steps i+1 and
// i-1 run under the kernel of step i.
// ---------------------------------------------------------------------------------------------------------------
template <typename T, class Enqueue>
int gemm3_host_pipeline(const T* hA, int lda, size_t plane_a, const T* hB, int ldb, size_t plane_b, const T* hC, int ldc,
                        size_t plane_c, T* hD, int ldd, size_t plane_d, int M, int N, int K, int count, Enqueue enqueue) {
    if (!g_rt.is_init) return need_init();
    if (!hA || !hB || !hD) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null matrix pointer\n");
    if (M <= 0 || N <= 0 || K <= 0 || count <= 0) return fail(DECX_HIP_FAIL_DIMS, "Matrix Dims don't match each other");
    if (lda < K || ldb < N || ldd < N || (hC && ldc < N))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "leading dimension smaller than the row length\n");
    const size_t bytes_a = (size_t)M * lda * sizeof(T), bytes_b = (size_t)K * ldb * sizeof(T), bytes_d = (size_t)M * ldd * sizeof(T);
    struct Set { T *a = nullptr, *b = nullptr, *d = nullptr; hipEvent_t up = nullptr, done = nullptr, down = nullptr; } set[2];
    hipStream_t s_up = nullptr, s_down = nullptr;
    int rc = 0;
    auto cleanup = [&] {
        (void)hipDeviceSynchronize();
        for (Set& s : set) {
            if (s.a) (void)hipFree(s.a);
            if (s.b) (void)hipFree(s.b);
            if (s.d) (void)hipFree(s.d);
            if (s.up) (void)hipEventDestroy(s.up);
            if (s.done) (void)hipEventDestroy(s.done);
            if (s.down) (void)hipEventDestroy(s.down);
        }
        if (s_up) (void)hipStreamDestroy(s_up);
        if (s_down) (void)hipStreamDestroy(s_down);
    };
#define PIPE_TRY(expr)                                   \
    do {                                                 \
        hipError_t e_ = (expr);                          \
        if (e_ != hipSuccess) { rc = hip_fail(e_, #expr); cleanup(); return rc; } \
    } while (0)
    for (Set& s : set) {
        if (hipMalloc(&s.a, bytes_a) != hipSuccess || hipMalloc(&s.b, bytes_b) != hipSuccess || hipMalloc(&s.d, bytes_d) != hipSuccess) {
            (void)hipGetLastError();
            cleanup();
            return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
        }
        PIPE_TRY(hipEventCreateWithFlags(&s.up, hipEventDisableTiming));
        PIPE_TRY(hipEventCreateWithFlags(&s.done, hipEventDisableTiming));
        PIPE_TRY(hipEventCreateWithFlags(&s.down, hipEventDisableTiming));
    }
    PIPE_TRY(hipStreamCreateWithFlags(&s_up, hipStreamNonBlocking));
    PIPE_TRY(hipStreamCreateWithFlags(&s_down, hipStreamNonBlocking));
    auto upload = [&](int i) -> hipError_t {
        Set& s = set[i & 1];
        hipError_t e;
        if (i >= 2 && (e = hipStreamWaitEvent(s_up, s.done, 0)) != hipSuccess) return e;    // kernel i-2 has read a, b
        if (hC && i >= 2 && (e = hipStreamWaitEvent(s_up, s.down, 0)) != hipSuccess) return e;   // and d was drained
        if ((e = hipMemcpyAsync(s.a, hA + (size_t)i * plane_a, bytes_a, hipMemcpyHostToDevice, s_up)) != hipSuccess) return e;
        if ((e = hipMemcpyAsync(s.b, hB + (size_t)i * plane_b, bytes_b, hipMemcpyHostToDevice, s_up)) != hipSuccess) return e;
        if (hC && (e = hipMemcpy2DAsync(s.d, (size_t)ldd * sizeof(T), hC + (size_t)i * plane_c, (size_t)ldc * sizeof(T),
                                        (size_t)N * sizeof(T), M, hipMemcpyHostToDevice, s_up)) != hipSuccess) return e;
        return hipEventRecord(s.up, s_up);
    };
    PIPE_TRY(upload(0));
    for (int i = 0; i < count; ++i) {
        Set& s = set[i & 1];
        if (i + 1 < count) PIPE_TRY(upload(i + 1));
        PIPE_TRY(hipStreamWaitEvent(g_rt.stream, s.up, 0));
        if (i >= 2) PIPE_TRY(hipStreamWaitEvent(g_rt.stream, s.down, 0));                   // result i-2 has left d
        Batch one;
        one.stream = g_rt.stream;
        rc = enqueue(s.a, s.b, hC ? s.d : nullptr, s.d, one);
        if (rc) { cleanup(); return rc; }
        PIPE_TRY(hipEventRecord(s.done, g_rt.stream));
        PIPE_TRY(hipStreamWaitEvent(s_down, s.done, 0));
        PIPE_TRY(hipMemcpy2DAsync(hD + (size_t)i * plane_d, (size_t)ldd * sizeof(T), s.d, (size_t)ldd * sizeof(T),
                                  (size_t)N * sizeof(T), M, hipMemcpyDeviceToHost, s_down));
        PIPE_TRY(hipEventRecord(s.down, s_down));
    }
    PIPE_TRY(hipStreamSynchronize(s_down));
    PIPE_TRY(hipStreamSynchronize(g_rt.stream));
#undef PIPE_TRY
    cleanup();
    return 0;
}

// One GEMM on HOST-resident matrices (the Matrix<T> overloads of de::cuda::GEMM, GEMM.h:56-131, :139-228).  The link to
// the host is the bottleneck (8192^3 fp32: 0.54 GB up at 57 GB/s = 9.3 ms against 7.3 ms of kernel), so the uploads never
// pause and the kernel follows them as closely as the data allows: A goes up in row panels, B in column panels, taking
// turns; a new row panel of A is multiplied at once with all column panels of B already there, a new column panel of B
// with all row panels of A already there (one GEMM launch each, on sub-matrices of the device copies), and each finished
// region of the result goes down on a third stream.  Every output is still one whole walk over K: same bits as the
// device-resident call.  Device copies keep the host pitches.  Overlap needs pinned host memory (decx_hip_host_malloc);
// pageable memory works but serialises.
template <typename T, class Enqueue>
int gemm_host_pipeline(const T* hA, int lda, const T* hB, int ldb, const T* hC, int ldc, T* hD, int ldd, int M, int N, int K,
                       Enqueue enqueue) {
    if (!g_rt.is_init) return need_init();
    if (!hA || !hB || !hD) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null matrix pointer\n");
    if (M <= 0 || N <= 0 || K <= 0) return fail(DECX_HIP_FAIL_DIMS, "Matrix Dims don't match each other");
    if (lda < K || ldb < N || ldd < N || (hC && ldc < N))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "leading dimension smaller than the row length\n");
    // panels of whole 256-wide tiles, at least 1024 wide, at most 8 per operand
    constexpr int MAX_PANELS = 8, MAX_STEPS = 2 * MAX_PANELS;
    auto panel_extent = [](int extent) {
        int p = cdiv(cdiv(extent, MAX_PANELS), 256) * 256;
        return p < 1024 ? 1024 : p;
    };
    const int pm = panel_extent(M), pn = panel_extent(N);
    const int panels_a = cdiv(M, pm), panels_b = cdiv(N, pn), steps = panels_a + panels_b;
    T *dA = nullptr, *dB = nullptr, *dD = nullptr;
    hipStream_t s_up = nullptr, s_down = nullptr;
    hipEvent_t up[MAX_STEPS] = {}, done[MAX_STEPS] = {};
    int rc = 0;
    auto cleanup = [&] {
        (void)hipDeviceSynchronize();
        if (dA) (void)hipFree(dA);
        if (dB) (void)hipFree(dB);
        if (dD) (void)hipFree(dD);
        for (int p = 0; p < MAX_STEPS; ++p) {
            if (up[p]) (void)hipEventDestroy(up[p]);
            if (done[p]) (void)hipEventDestroy(done[p]);
        }
        if (s_up) (void)hipStreamDestroy(s_up);
        if (s_down) (void)hipStreamDestroy(s_down);
    };
#define PIPE_TRY(expr)                                   \
    do {                                                 \
        hipError_t e_ = (expr);                          \
        if (e_ != hipSuccess) { rc = hip_fail(e_, #expr); cleanup(); return rc; } \
    } while (0)
    if (hipMalloc(&dA, (size_t)M * lda * sizeof(T)) != hipSuccess || hipMalloc(&dB, (size_t)K * ldb * sizeof(T)) != hipSuccess ||
        hipMalloc(&dD, (size_t)M * ldd * sizeof(T)) != hipSuccess) {
        (void)hipGetLastError();
        cleanup();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    }
    PIPE_TRY(hipStreamCreateWithFlags(&s_up, hipStreamNonBlocking));
    PIPE_TRY(hipStreamCreateWithFlags(&s_down, hipStreamNonBlocking));
    for (int p = 0; p < steps; ++p) {
        PIPE_TRY(hipEventCreateWithFlags(&up[p], hipEventDisableTiming));
        PIPE_TRY(hipEventCreateWithFlags(&done[p], hipEventDisableTiming));
    }
    int a_up = 0, b_up = 0;      // panels of A / B on the device (or on their way, in stream order)
    for (int step = 0; step < steps; ++step) {
        // whichever operand is behind goes next; A first
        const bool next_is_a = b_up == panels_b || (a_up < panels_a && (long)a_up * panels_b <= (long)b_up * panels_a);
        int r0, rows, c0, cols;      // the region of the result that this panel completes the operands of
        if (next_is_a) {
            r0 = a_up * pm, rows = M - r0 < pm ? M - r0 : pm;
            c0 = 0, cols = b_up * pn < N ? b_up * pn : N;
            PIPE_TRY(hipMemcpy2DAsync(dA + (size_t)r0 * lda, (size_t)lda * sizeof(T), hA + (size_t)r0 * lda, (size_t)lda * sizeof(T),
                                      (size_t)K * sizeof(T), rows, hipMemcpyHostToDevice, s_up));
            ++a_up;
        } else {
            c0 = b_up * pn, cols = N - c0 < pn ? N - c0 : pn;
            r0 = 0, rows = a_up * pm < M ? a_up * pm : M;
            PIPE_TRY(hipMemcpy2DAsync(dB + c0, (size_t)ldb * sizeof(T), hB + c0, (size_t)ldb * sizeof(T), (size_t)cols * sizeof(T), K,
                                      hipMemcpyHostToDevice, s_up));
            ++b_up;
        }
        if (rows == 0 || cols == 0) continue;      // the very first panel: its partner is not there yet
        if (hC)   // C goes into the result buffer and is accumulated onto in place, as the reference does (GEMM.h:196-206)
            PIPE_TRY(hipMemcpy2DAsync(dD + (size_t)r0 * ldd + c0, (size_t)ldd * sizeof(T), hC + (size_t)r0 * ldc + c0,
                                      (size_t)ldc * sizeof(T), (size_t)cols * sizeof(T), rows, hipMemcpyHostToDevice, s_up));
        PIPE_TRY(hipEventRecord(up[step], s_up));
        PIPE_TRY(hipStreamWaitEvent(g_rt.stream, up[step], 0));
        Batch one;
        one.stream = g_rt.stream;
        T* d_region = dD + (size_t)r0 * ldd + c0;
        rc = enqueue(dA + (size_t)r0 * lda, dB + c0, hC ? d_region : nullptr, d_region, rows, cols, one);
        if (rc) { cleanup(); return rc; }
        PIPE_TRY(hipEventRecord(done[step], g_rt.stream));
        PIPE_TRY(hipStreamWaitEvent(s_down, done[step], 0));
        PIPE_TRY(hipMemcpy2DAsync(hD + (size_t)r0 * ldd + c0, (size_t)ldd * sizeof(T), d_region, (size_t)ldd * sizeof(T),
                                  (size_t)cols * sizeof(T), rows, hipMemcpyDeviceToHost, s_down));
    }
    PIPE_TRY(hipStreamSynchronize(s_down));
    PIPE_TRY(hipStreamSynchronize(g_rt.stream));
#undef PIPE_TRY
    cleanup();
    return 0;
}

// Plain streaming copy, 16 bytes per lane and iteration: the known-size kernel that hardware traffic counters
// (FETCH_SIZE / WRITE_SIZE) are calibrated against.
__global__ __launch_bounds__(256) void copy_kernel(f32x4* __restrict__ dst, const f32x4* __restrict__ src, size_t quads) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < quads; i += stride) dst[i] = src[i];
}

// Element-wise ReLU family of nn/operators/ReLU.h.  MODE 0: forward; 1: forward + record; 2: backward (dst = src where
// the recorded bit is set, else 0 * src; ReLU.h:131-165).  The bit map has one byte per 8 consecutive floats: bits 4..7
// = the first 16-byte quad's x,y,z,w, bits 0..3 = the second quad's (ReLU.h:86-123).
// One quad per lane, no loop, streaming (non-temporal) accesses: every byte is touched once, consecutive lanes take
// consecutive 16 bytes, and short-lived workgroups keep more loads in flight across the chip than a few long-lived ones
// (measured: 6.7 TB/s against 5.2-5.8 TB/s for grid-stride loops of any unroll depth).  A map byte is assembled from
// the two lanes of a quad pair with one lane exchange; the even lane stores it.
template <int MODE>
__global__ __launch_bounds__(256) void relu_kernel(const f32x4* __restrict__ src, f32x4* __restrict__ dst,
                                                   unsigned char* __restrict__ rec_map, size_t quads) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = i < quads;              // quads is even in modes 1 and 2, so both lanes of a pair are live together
    f32x4 q = {0.f, 0.f, 0.f, 0.f};
    if (live) q = __builtin_nontemporal_load(src + i);
    unsigned nibble = 0;
    if (MODE == 2 && live) {
        const unsigned byte = rec_map[i >> 1];
        nibble = (i & 1) ? (byte & 15u) : (byte >> 4);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (MODE == 2) {
            q[e] = (float)((nibble >> e) & 1u) * q[e];
        } else {
            const unsigned s = (~__float_as_uint(q[e])) >> 31;
            q[e] = (float)s * q[e];
            nibble |= s << e;
        }
    }
    if (MODE == 1) {
        const unsigned other = (unsigned)__shfl_xor((int)nibble, 1);
        if (live && (i & 1) == 0) rec_map[i >> 1] = (unsigned char)((nibble << 4) | other);
    }
    if (live) __builtin_nontemporal_store(q, dst + i);
}
// the last n % 4 floats of the plain forward form
__global__ void relu_tail_kernel(const float* __restrict__ src, float* __restrict__ dst, int n) {
    const int i = threadIdx.x;
    if (i < n) dst[i] = relu_by_sign(src[i]);
}

template <int MODE>
int relu_enqueue(const float* src, float* dst, unsigned char* rec_map, size_t n) {
    if (!g_rt.is_init) return need_init();
    if (!src || !dst || (MODE != 0 && !rec_map)) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null pointer\n");
    if (!aligned16(src) || !aligned16(dst)) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "ReLU needs 16-byte aligned buffers\n");
    if (MODE != 0 && n % 8 != 0)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "the recorded forms work on whole groups of 8 floats (one map byte each)\n");
    const size_t quads = MODE == 0 ? n / 4 : n / 8 * 2;
    if (quads > 0) {
        const size_t blocks = (quads + 255) / 256;
        if (blocks > 0x7fffffffull) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "buffer too large for one launch\n");
        hipLaunchKernelGGL(relu_kernel<MODE>, dim3((unsigned)blocks), dim3(256), 0, g_rt.stream,
                           reinterpret_cast<const f32x4*>(src), reinterpret_cast<f32x4*>(dst), rec_map, quads);
        HIP_TRY(hipGetLastError());
    }
    if (MODE == 0 && n % 4 != 0) {
        hipLaunchKernelGGL(relu_tail_kernel, dim3(1), dim3(64), 0, g_rt.stream, src + quads * 4, dst + quads * 4, (int)(n % 4));
        HIP_TRY(hipGetLastError());
    }
    return 0;
}

int finish(int rc) {
    if (rc != 0) return rc;
    HIP_TRY(hipStreamSynchronize(g_rt.stream));
    return 0;
}

}  // namespace

extern "C" {

int decx_hip_init(int* device) {
    if (!g_rt.is_init) {
        int count = 0;
        HIP_TRY(hipGetDeviceCount(&count));
        if (count <= 0) return fail(DECX_HIP_FAIL_NOT_INIT, "no HIP device visible\n");
        int dev = 0;
        HIP_TRY(hipGetDevice(&dev));
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, dev));
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return fail(DECX_HIP_FAIL_NOT_INIT, "device %d is %s; this library carries gfx950 code only\n", dev,
                        prop.gcnArchName);
        g_rt.device = dev;
        g_rt.compute_units = prop.multiProcessorCount;
        g_rt.clock_khz = prop.clockRate;
        g_rt.hbm_bytes = prop.totalGlobalMem;
        HIP_TRY(hipStreamCreateWithFlags(&g_rt.stream, hipStreamNonBlocking));
        HIP_TRY(hipEventCreate(&g_rt.ev_start));
        HIP_TRY(hipEventCreate(&g_rt.ev_stop));
        if (const char* gm = getenv("DECX_HIP_GROUP_M")) { int v = atoi(gm); if (v > 0) g_rt.group_m = v; }
        g_rt.is_init = true;
    }
    if (device) *device = g_rt.device;
    return 0;
}

int decx_hip_is_init(void) { return g_rt.is_init ? 1 : 0; }

int decx_hip_device_info(int* compute_units, int* clock_khz, size_t* hbm_bytes) {
    if (!g_rt.is_init) return need_init();
    if (compute_units) *compute_units = g_rt.compute_units;
    if (clock_khz) *clock_khz = g_rt.clock_khz;
    if (hbm_bytes) *hbm_bytes = g_rt.hbm_bytes;
    return 0;
}

int decx_hip_malloc(void** dptr, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    if (!dptr) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null output pointer\n");
    *dptr = nullptr;
    if (hipMalloc(dptr, bytes ? bytes : 1) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");   // core/error.h:65
    }
    return 0;
}

int decx_hip_free(void* dptr) {
    if (!dptr) return 0;
    HIP_TRY(hipFree(dptr));
    return 0;
}

int decx_hip_memset(void* dptr, int value, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipMemsetAsync(dptr, value, bytes, g_rt.stream));
    HIP_TRY(hipStreamSynchronize(g_rt.stream));
    return 0;
}

int decx_hip_host_malloc(void** hptr, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    if (!hptr) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null output pointer\n");
    *hptr = nullptr;
    if (hipHostMalloc(hptr, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    }
    return 0;
}

int decx_hip_host_free(void* hptr) {
    if (!hptr) return 0;
    HIP_TRY(hipHostFree(hptr));
    return 0;
}

static hipMemcpyKind copy_kind(int direction) {
    switch (direction) {
        case DECX_HIP_H2D: return hipMemcpyHostToDevice;
        case DECX_HIP_D2H: return hipMemcpyDeviceToHost;
        default: return hipMemcpyDeviceToDevice;
    }
}

int decx_hip_memcpy2d(void* dst, size_t dst_pitch_bytes, const void* src, size_t src_pitch_bytes, size_t width_bytes,
                      size_t rows, int direction) {
    if (!g_rt.is_init) return need_init();
    if (direction < DECX_HIP_H2D || direction > DECX_HIP_D2D) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "bad copy direction\n");
    if (width_bytes == 0 || rows == 0) return 0;
    if (dst_pitch_bytes < width_bytes || src_pitch_bytes < width_bytes)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "pitch smaller than the row width\n");
    HIP_TRY(hipMemcpy2DAsync(dst, dst_pitch_bytes, src, src_pitch_bytes, width_bytes, rows, copy_kind(direction),
                             g_rt.stream));
    HIP_TRY(hipStreamSynchronize(g_rt.stream));
    return 0;
}

int decx_hip_memcpy(void* dst, const void* src, size_t bytes, int direction) {
    if (!g_rt.is_init) return need_init();
    if (direction < DECX_HIP_H2D || direction > DECX_HIP_D2D) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "bad copy direction\n");
    if (bytes == 0) return 0;
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, copy_kind(direction), g_rt.stream));
    HIP_TRY(hipStreamSynchronize(g_rt.stream));
    return 0;
}

int decx_hip_sync(void) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipDeviceSynchronize());
    return 0;
}

int decx_hip_sgemm_async(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd,
                         int M, int N, int K) {
    return sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream());
}
int decx_hip_sgemm(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                   int N, int K) {
    return finish(sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream()));
}
int decx_hip_sgemm_relu(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                        int N, int K) {
    return finish(sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream(), true));
}
int decx_hip_sgemm_splitk(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                          int N, int K, int splits) {
    return finish(sgemm_splitk_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, splits));
}
int decx_hip_sgemm_batched(const float* A, int lda, size_t stride_a, const float* B, int ldb, size_t stride_b,
                           const float* Cin, int ldc, size_t stride_c, float* D, int ldd, size_t stride_d, int M, int N, int K,
                           int batch) {
    return finish(sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K,
                                batch_on_library_stream(batch, stride_a, stride_b, stride_c, stride_d)));
}

int decx_hip_hgemm_f32acc_async(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                uint16_t* D, int ldd, int M, int N, int K) {
    return hgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream());
}
int decx_hip_hgemm_f32acc(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                          int ldd, int M, int N, int K) {
    return finish(hgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream()));
}
int decx_hip_hgemm_f32acc_batched(const uint16_t* A, int lda, size_t stride_a, const uint16_t* B, int ldb, size_t stride_b,
                                  const uint16_t* Cin, int ldc, size_t stride_c, uint16_t* D, int ldd, size_t stride_d, int M,
                                  int N, int K, int batch) {
    return finish(hgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K,
                                batch_on_library_stream(batch, stride_a, stride_b, stride_c, stride_d)));
}

int decx_hip_gemm3_host_f32(const float* hA, int lda, size_t plane_a, const float* hB, int ldb, size_t plane_b,
                            const float* hC, int ldc, size_t plane_c, float* hD, int ldd, size_t plane_d, int M, int N, int K,
                            int count) {
    return gemm3_host_pipeline<float>(hA, lda, plane_a, hB, ldb, plane_b, hC, ldc, plane_c, hD, ldd, plane_d, M, N, K, count,
                                      [&](const float* a, const float* b, const float* c, float* d, const Batch& one) {
                                          return sgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, M, N, K, one);
                                      });
}
int decx_hip_gemm3_host_f16(const uint16_t* hA, int lda, size_t plane_a, const uint16_t* hB, int ldb, size_t plane_b,
                            const uint16_t* hC, int ldc, size_t plane_c, uint16_t* hD, int ldd, size_t plane_d, int M, int N,
                            int K, int count) {
    return gemm3_host_pipeline<uint16_t>(hA, lda, plane_a, hB, ldb, plane_b, hC, ldc, plane_c, hD, ldd, plane_d, M, N, K, count,
                                         [&](const uint16_t* a, const uint16_t* b, const uint16_t* c, uint16_t* d, const Batch& one) {
                                             return hgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, M, N, K, one);
                                         });
}

int decx_hip_gemm_host_f32(const float* hA, int lda, const float* hB, int ldb, const float* hC, int ldc, float* hD, int ldd,
                           int M, int N, int K) {
    return gemm_host_pipeline<float>(hA, lda, hB, ldb, hC, ldc, hD, ldd, M, N, K,
                                     [&](const float* a, const float* b, const float* c, float* d, int rows, int cols, const Batch& one) {
                                         return sgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, rows, cols, K, one);
                                     });
}
int decx_hip_gemm_host_f16(const uint16_t* hA, int lda, const uint16_t* hB, int ldb, const uint16_t* hC, int ldc, uint16_t* hD,
                           int ldd, int M, int N, int K) {
    return gemm_host_pipeline<uint16_t>(hA, lda, hB, ldb, hC, ldc, hD, ldd, M, N, K,
                                        [&](const uint16_t* a, const uint16_t* b, const uint16_t* c, uint16_t* d, int rows, int cols, const Batch& one) {
                                            return hgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, rows, cols, K, one);
                                        });
}

int decx_hip_conv2_im2col_f32_async(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag) {
    return conv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst, dst_dpitch,
                        dst_row_stride, flag);
}
int decx_hip_conv2_im2col_f32(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt, int N,
                              int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst, int dst_dpitch,
                              size_t dst_row_stride, int flag) {
    return finish(conv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst,
                               dst_dpitch, dst_row_stride, flag));
}

int decx_hip_conv2_im2col_f32_fused(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag, const float* bias, int relu) {
    return finish(conv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst,
                               dst_dpitch, dst_row_stride, flag, bias, relu != 0));
}

int decx_hip_conv2_im2col_f16_async(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag, const uint16_t* bias, int relu) {
    return hconv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst, dst_dpitch,
                         dst_row_stride, flag, bias, relu != 0);
}
int decx_hip_conv2_im2col_f16(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt, int N,
                              int kh, int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst, int dst_dpitch,
                              size_t dst_row_stride, int flag, const uint16_t* bias, int relu) {
    return finish(hconv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst,
                                dst_dpitch, dst_row_stride, flag, bias, relu != 0));
}

int decx_hip_relu_f32(const float* src, float* dst, size_t n) { return finish(relu_enqueue<0>(src, dst, nullptr, n)); }
int decx_hip_relu_f32_async(const float* src, float* dst, size_t n) { return relu_enqueue<0>(src, dst, nullptr, n); }
int decx_hip_relu_f32_rec(const float* src, float* dst, unsigned char* rec_map, size_t n) {
    return finish(relu_enqueue<1>(src, dst, rec_map, n));
}
int decx_hip_relu_f32_backward(const float* src, float* dst, const unsigned char* rec_map, size_t n) {
    return finish(relu_enqueue<2>(src, dst, const_cast<unsigned char*>(rec_map), n));
}

int decx_hip_copy_kernel(void* dst, const void* src, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    if (!dst || !src || bytes % 16 != 0 || !aligned16(dst) || !aligned16(src))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "copy needs 16-byte aligned pointers and a multiple of 16 bytes\n");
    if (bytes == 0) return 0;
    const int blocks = g_rt.compute_units > 0 ? g_rt.compute_units * 8 : 2048;
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(256), 0, g_rt.stream, static_cast<f32x4*>(dst),
                       static_cast<const f32x4*>(src), bytes / 16);
    HIP_TRY(hipGetLastError());
    return finish(0);
}

int decx_hip_timer_start(void) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipEventRecord(g_rt.ev_start, g_rt.stream));
    return 0;
}

int decx_hip_timer_stop(float* milliseconds) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipEventRecord(g_rt.ev_stop, g_rt.stream));
    HIP_TRY(hipEventSynchronize(g_rt.ev_stop));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, g_rt.ev_start, g_rt.ev_stop));
    if (milliseconds) *milliseconds = ms;
    return 0;
}

const char* decx_hip_last_error(void) { return g_err; }

int decx_hip_set_sgemm_variant(int variant) {
    int prev = g_rt.sgemm_variant;
    g_rt.sgemm_variant = variant;
    return prev;
}
int decx_hip_set_hgemm_variant(int variant) {
    int prev = g_rt.hgemm_variant;
    g_rt.hgemm_variant = variant;
    return prev;
}

}  // extern "C"
