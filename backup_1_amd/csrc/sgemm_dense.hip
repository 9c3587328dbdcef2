// fp32 dense GEMM: argument checks, kernel choice and launch (sgemm_tile.hpp, sgemm_chain16.hpp), split-K.
#include "sgemm_launch.hpp"
#include "sgemm_chain16.hpp"

namespace decx_hip {

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
        enqueue_zero_region(D, ldd, M, N, g_rt.stream);
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

int sgemm_enqueue(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                  int N, int K, const Batch& batch, bool relu) {
    if (int rc = check_gemm_args(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch)) return rc;
    const bool vec_a = aligned16(A) && lda % 4 == 0 && batch.stride_a % 4 == 0;
    const bool vec_b = aligned16(B) && ldb % 4 == 0 && ldb >= 4 && batch.stride_b % 4 == 0;
    DenseOut out{ldd, relu, aligned16(D) && ldd % 4 == 0 && batch.stride_d % 4 == 0};
    const bool one_launch = g_rt.sgemm_variant == 34;
    const ShapeForThisCall shape_for_this_call(one_launch ? 0 : g_rt.sgemm_variant);
    const int plan = plan_sgemm(M, N, K, batch.count, vec_a, vec_b, lda, ldb);
    if (!one_launch && plan != 0) {
        const WholeRoundsSplit split = plan_whole_rounds_split(M, N, K, batch.count, lda, ldb);
        if (split.shape && !split.by_columns) {
            if (int rc = launch_sgemm_dma_shape(split.shape, A, lda, B, ldb, Cin, ldc, D, ldd, split.first, N, K, batch, relu)) return rc;
            return sgemm_enqueue(A + (size_t)split.first * lda, lda, B, ldb, Cin ? Cin + (size_t)split.first * ldc : nullptr, ldc,
                                 D + (size_t)split.first * ldd, ldd, M - split.first, N, K, batch, relu);
        }
        if (split.shape) {
            if (int rc = launch_sgemm_dma_shape(split.shape, A, lda, B, ldb, Cin, ldc, D, ldd, M, split.first, K, batch, relu)) return rc;
            return sgemm_enqueue(A, lda, B + split.first, ldb, Cin ? Cin + split.first : nullptr, ldc, D + split.first, ldd, M,
                                 N - split.first, K, batch, relu);
        }
    }
    if (plan == 0) {     // unaligned operands: element-wise loaders, one tile shape only
        DenseA<false> a{A, lda, M, K, batch.stride_a};
        DenseB<false> b{B, ldb, N, K, batch.stride_b};
        return launch_sgemm_tile<SShapeSmall>(a, b, Cin, ldc, D, out, M, N, K, batch);
    }
    if ((plan >= 18 && plan <= 22) || (plan >= 24 && plan <= 28)) return launch_sgemm_dma_shape(plan, A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (plan == 11) return launch_sgemm_chain16<Chain16<2, 1, 4, 4>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (plan == 12) return launch_sgemm_chain16<Chain16<1, 1, 8, 2>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (plan == 13) return launch_sgemm_chain16<Chain16<4, 2, 2, 3>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (plan == 23) return launch_sgemm_chain16<Chain16Rect<1, 2, 1, 6, 2>>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    DenseA<true> a{A, lda, M, K, batch.stride_a};
    DenseB<true> b{B, ldb, N, K, batch.stride_b};
    if (plan == 14) return launch_sgemm_tile<SShape192>(a, b, Cin, ldc, D, out, M, N, K, batch);
    return dispatch_sgemm(plan, a, b, Cin, ldc, D, out, M, N, K, batch);
}

// host-only: the choice above for a product described by its sizes and pitches (decx_hip_sgemm_plan)
int sgemm_plan(int M, int N, int K, int batch, long lda, long ldb, bool aligned) {
    const ShapeForThisCall shape_for_this_call(g_rt.sgemm_variant == 34 ? 0 : g_rt.sgemm_variant);
    return plan_sgemm(M, N, K, batch, aligned && lda % 4 == 0, aligned && ldb % 4 == 0 && ldb >= 4, lda, ldb);
}

// host-only: the two-launch plan of plan_whole_rounds_split for a product (decx_hip_sgemm_plan_split)
int sgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, bool aligned, int* shape, int* by_columns) {
    WholeRoundsSplit split;
    if (aligned && lda % 4 == 0 && ldb % 4 == 0 && ldb >= 4) split = plan_whole_rounds_split(M, N, K, batch, lda, ldb);
    if (shape) *shape = split.shape;
    if (by_columns) *by_columns = split.by_columns ? 1 : 0;
    return split.shape ? split.first : 0;
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

}  // namespace decx_hip
