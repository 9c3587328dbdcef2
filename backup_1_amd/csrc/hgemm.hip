// fp16 GEMM with fp32 accumulation: kernel choice and launch (hgemm_dma_tile.hpp, hgemm_tile.hpp), split-K.
#include "runtime.hpp"
#include "hgemm_dma_tile.hpp"
#include "hgemm_tile.hpp"
#include "hgemm_mfma16_tile.hpp"

namespace decx_hip {

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
//   7: as 4 with 2x4 waves of 128x64 (two waves per SIMD) -- the best of the 32x32x16 shapes: the chip is power-capped on
//      them (MFMA busy x clock stays ~1.27 GHz-equivalents whatever the schedule), and this one is 1 % ahead
//  15: 256x256x64, 2x4 waves of 128x64 on v_mfma_f32_16x16x32_f16, 2-stage LDS-DMA pipeline, result written through LDS in
//      16-byte pieces (hgemm_mfma16_tile.hpp) -- the default for large problems: 8 % faster than 7 at 8192^3, because
//      this instruction draws less power per flop on real-valued data
//  16: as 15 with 4 LDS stages of 32 k instead of 2 of 64 (three K steps in flight instead of one): measured equal to 15 at
//      8192^3 (1381 vs 1396 TFLOP/s), and so were 5 stages and a refill spread over the following step -- the wait for the
//      loads is not what the kernel loses time to (4 waves of 128x128, a quarter fewer LDS reads, measured 1387 too: on
//      uniform[-1,1] data every arrangement ends at the same power-limited rate); kept as the second instantiation of
//      the kernel's stage arithmetic
//  17: as 15 with one workgroup per compute unit that walks its tiles as one stream of K steps (no prologue after the
//      first tile, the epilogue under the next tile's loads); products of whole tiles only, others fall back to 15
//  11: split-K on shape 8 through an fp32 workspace (hgemm_splitk_enqueue) -- few tiles and a long K
// and, for the fp16 convolution only: 12 keeps its register-staged kernels, 13 takes its LDS-DMA kernel for any image
// whose channel pitch allows it, 14 its tap-row kernel, 18 its kernel on 16x16x32 matrix instructions with patch-shaped
// tiles (hconv_mfma16.hpp); each switches its split over K off.  19 keeps kernel 18 out of the automatic choice.
// 20: the automatic choice, every product in one launch (plan_hgemm_whole_rounds_split switched off).
// (experiments and tests)
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

typedef Hgemm16Shape<256, 256, 64, 2, 4, 2> HShape16;            // 8 waves, 128x64 each, 16x16x32 MFMAs, 2 stages of 64 k
typedef Hgemm16Shape<256, 256, 32, 2, 4, 4> HShape16K32S4;       // 4 stages of 32 k

template <class S>
int launch_hgemm_mfma16(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                        int ldd, int M, int N, int K, const Batch& batch) {
    auto kern = Cin ? hgemm_mfma16_kernel<S, true> : hgemm_mfma16_kernel<S, false>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_mfma16_kernel<S, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_mfma16_kernel<S, false>),
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
                       tiles_m, tiles_n, group_m, batch.stride_a, batch.stride_b, batch.stride_c, batch.stride_d);
    HIP_TRY(hipGetLastError());
    return 0;
}

// The same tile as one workgroup per compute unit that walks its tiles as one stream of K steps (PERSIST build of the
// kernel): whole tiles only, one problem per launch.
template <class S>
bool hgemm_mfma16_persistent_fits(int M, int N, int K, const Batch& batch) {
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    return batch.count == 1 && M % S::BM == 0 && N % S::BN == 0 && K % (S::BK * S::WALK) == 0 && K >= S::BK * S::STAGES &&
           (long)(M / S::BM) * (N / S::BN) > cus;                  // with at most one tile per CU there is nothing to chain
}

template <class S>
int launch_hgemm_mfma16_persistent(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                                   int ldd, int M, int N, int K, const Batch& batch) {
    auto kern = Cin ? hgemm_mfma16_kernel<S, true, 0, true> : hgemm_mfma16_kernel<S, false, 0, true>;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_mfma16_kernel<S, true, 0, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::PERSIST_LDS_BYTES));
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_mfma16_kernel<S, false, 0, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::PERSIST_LDS_BYTES));
        attr_done = true;
    }
    const int tiles_m = M / S::BM, tiles_n = N / S::BN;
    const long total = (long)tiles_m * tiles_n;
    if (total > 0x7fffffffL) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "problem too large for one launch\n");
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)(total < cus ? total : cus)), dim3(S::NT), S::PERSIST_LDS_BYTES, batch.stream,
                       reinterpret_cast<const _Float16*>(A), lda, reinterpret_cast<const _Float16*>(B), ldb,
                       reinterpret_cast<const _Float16*>(Cin), ldc, reinterpret_cast<_Float16*>(D), ldd, M, N, K,
                       tiles_m, tiles_n, group_m, (size_t)0, (size_t)0, (size_t)0, (size_t)0);
    HIP_TRY(hipGetLastError());
    return 0;
}

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
                       static_cast<float*>(nullptr), 0, (size_t)0);
    HIP_TRY(hipGetLastError());
    return 0;
}

// fp16 GEMM whose result has too few tiles to fill the chip while K is long: K is cut into ranges that run as separate
// workgroups (blockIdx.z).  Each range stores its fp32 partial sums into a plane of its own in a workspace, and a second
// kernel adds the planes in range order, adds C and rounds to binary16 once: the same bits on every run.  In the atomic
// mode (decx_hip_set_splitk_mode(1)) all ranges add into one zeroed plane in whatever order they arrive, so the last
// bit can differ between runs.  (fp32 GEMM never splits K by itself: its results are bit-exact chains.)
struct SplitPlan {
    int splits, k_split_len;
};
static SplitPlan plan_hgemm_split(int K, int splits) {
    typedef HShapeDmaSmall S;
    const int k_split_len = cdiv(cdiv(K, splits), S::BK) * S::BK;
    return SplitPlan{cdiv(K, k_split_len), k_split_len};                 // no empty range
}

// the automatic number of K ranges for an M x N x K product (0: do not split) -- the choice of hgemm_enqueue.
// Measured, in us: a tile walks K at 6.7 ns per k (1.6 times that when two workgroups share a CU); a launch costs about
// 4, the finishing kernel and its launch 5.5, a partial sum stored and read back (or an atomic add) about 3 ps.
static int auto_hgemm_splits(int M, int N, int K) {
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long tiles = (long)cdiv(M, 128) * cdiv(N, 128);
    // ranges for two workgroups per CU with atomics; one per CU when every range writes and the finishing kernel reads a
    // plane of its own (measured: 64x65536x1024 49 us with 32 ranges, 52 with 64; 128x16384x2048 38 with 16, 42 with 32)
    long splits = ((g_rt.splitk_atomic ? 2 : 1) * cus + tiles - 1) / tiles;
    if (splits > K / 512) splits = K / 512;                        // at least 8 K steps per range
    if (splits < 2 || (size_t)M * N > ((size_t)1 << 26)) return 0;
    const double t_whole = 4.0 + 0.0067 * K * (double)((tiles + cus - 1) / cus);
    const double share = tiles * splits > cus ? 1.6 : 1.0;
    const double t_split = (g_rt.splitk_atomic ? 9.0 : 5.5) + 3.1e-6 * M * N * splits +
                           0.0067 * ((double)K / splits) * share * (double)((tiles * splits + 2 * cus - 1) / (2 * cus));
    return t_split < 0.85 * t_whole ? (int)splits : 0;
}

static int hgemm_splitk_launch(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                               int ldd, int M, int N, int K, const SplitPlan& plan, float* workspace, bool ordered,
                               hipStream_t stream) {
    typedef HShapeDmaSmall S;                      // 128x128x64, LDS-DMA staged, two workgroups per CU
    auto kern = hgemm_dma_kernel<S, false, true>;
    const size_t total = (size_t)M * N;
    const unsigned fill_blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    if (!ordered) enqueue_zero_region(workspace, N, M, N, stream);
    const int tiles_m = cdiv(M, S::BM), tiles_n = cdiv(N, S::BN);
    const int group_m = tiles_m < g_rt.group_m ? tiles_m : g_rt.group_m;
    hipLaunchKernelGGL(kern, dim3((unsigned)(tiles_m * tiles_n), 1, (unsigned)plan.splits), dim3(S::NT), S::LDS_BYTES, stream,
                       reinterpret_cast<const _Float16*>(A), lda, reinterpret_cast<const _Float16*>(B), ldb,
                       static_cast<const _Float16*>(nullptr), 0, reinterpret_cast<_Float16*>(D), ldd, M, N, K, tiles_m, tiles_n,
                       group_m, (size_t)0, (size_t)0, (size_t)0, (size_t)0, workspace, plan.k_split_len, ordered ? total : (size_t)0);
    hipLaunchKernelGGL(hgemm_split_finish_kernel, dim3(fill_blocks), dim3(256), 0, stream, workspace, ordered ? plan.splits : 1,
                       total, reinterpret_cast<const _Float16*>(Cin), ldc, reinterpret_cast<_Float16*>(D), ldd, M, N);
    HIP_TRY(hipGetLastError());
    return 0;
}

static int allow_split_kernel_lds() {
    typedef HShapeDmaSmall S;
    static bool attr_done = false;
    if (!attr_done) {
        HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hgemm_dma_kernel<S, false, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::LDS_BYTES));
        attr_done = true;
    }
    return 0;
}

int hgemm_splitk_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                         int ldd, int M, int N, int K, int splits, hipStream_t stream) {
    const SplitPlan plan = plan_hgemm_split(K, splits);
    const bool ordered = !g_rt.splitk_atomic;
    if (int rc = ensure_partial((size_t)M * N * sizeof(float) * (ordered ? plan.splits : 1))) return rc;
    if (int rc = allow_split_kernel_lds()) return rc;
    return hgemm_splitk_launch(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, plan, g_rt.partial, ordered, stream);
}

// the LDS-DMA tiles address a tile's rows with 32-bit byte offsets from the tile's first row: 256 rows of A, 64 of B
static bool hgemm_pitches_fit(long lda, long ldb) {
    return lda % 8 == 0 && ldb % 8 == 0 && ldb >= 8 && (size_t)lda * 256 * sizeof(uint16_t) < ((size_t)1 << 32) &&
           (size_t)ldb * 64 * sizeof(uint16_t) < ((size_t)1 << 32);
}
static bool hgemm_vector_path(const uint16_t* A, int lda, const uint16_t* B, int ldb, const Batch& batch) {
    return aligned16(A) && aligned16(B) && batch.stride_a % 8 == 0 && batch.stride_b % 8 == 0 && hgemm_pitches_fit(lda, ldb);
}

// The kernel decx_hip_hgemm_f32acc takes for a product, as the number decx_hip_set_hgemm_variant would force it with
// (the table at the top of this file); 0 = operands the vector loaders cannot take (the 128x128 tile with element-wise
// loaders); 11 = split over K, *splits ranges.
static int plan_hgemm(int M, int N, int K, int batch_count, bool vec, int* splits_out) {
    if (splits_out) *splits_out = 0;
    if (!vec) return 0;
    int variant = g_rt.hgemm_variant == 20 ? 0 : g_rt.hgemm_variant;
    // few 128x128 tiles and a long K: split K (variant 11 forces it, any other fixed variant switches it off)
    if (batch_count == 1 && (variant < 1 || variant > 10) && (variant < 15 || variant > 17)) {
        int splits = auto_hgemm_splits(M, N, K);
        if (variant == 11 && splits == 0 && K >= 1024 && (size_t)M * N <= ((size_t)1 << 26)) {
            const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
            const long tiles = (long)cdiv(M, 128) * cdiv(N, 128);
            long s = (2 * cus + tiles - 1) / tiles;
            if (s > K / 512) s = K / 512;
            splits = s >= 2 ? (int)s : 0;
        }
        if (splits >= 2) {
            if (splits_out) *splits_out = splits;
            return 11;
        }
    }
    if (variant == 11) variant = 0;
    if (variant < 1 || (variant > 10 && (variant < 15 || variant > 17))) {
        // same cost model as the fp32 picker: rounds of tiles per CU x tile area / measured shape efficiency
        const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
        const long big = (long)cdiv(M, 256) * cdiv(N, 256) * batch_count, small = (long)cdiv(M, 128) * cdiv(N, 128) * batch_count;
        const double cost_big = (double)((big + cus - 1) / cus) * 65536.0;
        const double cost_small = (double)((small + cus - 1) / cus) * 16384.0 / 0.75;
        // the small tile with three LDS stages holds one workgroup per CU: only worth it when there is at most one to hold
        variant = cost_big <= cost_small ? 15 : (small <= cus ? 9 : 8);
        // several rounds of whole 256x256 tiles on a K of 128 .. 3072 (the measured range; the walk needs K >= 128): one workgroup per CU that walks its tiles as one
        // stream of K steps (17) has no prologue after the first tile and stores under the next tile's loads, which a
        // short K walk cannot hide otherwise -- 8192x128x8192 49.4 -> 40.2 us, x256 58.7 -> 50.2, 16384x256x8192 105.2 -> 84.9, 8192x512x8192 85.0 -> 75.2, x1024 126.8 -> 117.9, x2048 215.8 -> 210.7,
        // x3072 307.2 -> 300.7, 6144x1024x8192 93.8 -> 87.4; level at 8192^3 (770.1 against 772.7), behind by 1 % on a
        // single round (4096x1024x4096), where hgemm_mfma16_persistent_fits says no anyway
        if (variant == 15 && batch_count == 1 && K <= 3072 && hgemm_mfma16_persistent_fits<HShape16>(M, N, K, Batch())) variant = 17;
    }
    return variant;
}

// A result whose 256x256 tiles come in whole rounds plus a part of one (a round = one tile per CU) pays a whole round
// for the part, and five rounds of 128x128 tiles where four and a bit would do.  The rows -- or columns -- that fill
// whole rounds of the 256x256 tile go to one launch of it, the rest to a second launch that picks its own kernel
// (4352^2: 289 tiles; 3840 rows in one round, 512 rows on 136 tiles of 128x128): taken where whole rounds plus the
// one-launch cost of the rest plus 4 us for the second launch stay under 96 % of the one-launch cost of the whole.
// Costs in tile area per CU / efficiency, the unit of plan_hgemm; 5.5e6 of it per microsecond and k.  Variant 20 keeps
// every product in one launch (experiments and tests).
struct HgemmWholeRoundsSplit {
    bool by_columns = false;
    int first = 0;          // rows (columns) of the first launch; 0 = one launch
};
static double hgemm_one_launch_cost(int M, int N) {
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long big = (long)cdiv(M, 256) * cdiv(N, 256), small = (long)cdiv(M, 128) * cdiv(N, 128);
    return std::min((double)((big + cus - 1) / cus) * 65536.0, (double)((small + cus - 1) / cus) * 16384.0 / 0.75);
}
static HgemmWholeRoundsSplit plan_hgemm_whole_rounds_split(int M, int N, int K, int batch_count, bool vec) {
    HgemmWholeRoundsSplit plan;
    if (!vec || g_rt.hgemm_variant != 0 || batch_count != 1 || K < 512) return plan;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long tiles_m = cdiv(M, 256), tiles_n = cdiv(N, 256), whole = tiles_m * tiles_n / cus;
    if (whole < 1 || tiles_m * tiles_n % cus == 0) return plan;
    double best = 0.96 * hgemm_one_launch_cost(M, N);
    const double second_launch = 4.0 * 5.5e6 / (2.0 * K);
    for (int by_columns = 0; by_columns < 2; ++by_columns) {
        const long lines = whole * cus / (by_columns ? tiles_m : tiles_n);          // whole tile rows (columns) in the whole rounds
        if (lines < 1 || lines >= (by_columns ? tiles_n : tiles_m)) continue;
        const int first = (int)lines * 256;
        const double cost = (double)whole * 65536.0 + (by_columns ? hgemm_one_launch_cost(M, N - first) : hgemm_one_launch_cost(M - first, N)) + second_launch;
        if (cost < best) {
            best = cost;
            plan.by_columns = by_columns != 0, plan.first = first;
        }
    }
    return plan;
}

// host-only: the two-launch plan for a product (decx_hip_hgemm_plan_split)
int hgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, bool aligned, int* by_columns) {
    const HgemmWholeRoundsSplit split = plan_hgemm_whole_rounds_split(M, N, K, batch, aligned && hgemm_pitches_fit(lda, ldb));
    if (by_columns) *by_columns = split.by_columns ? 1 : 0;
    return split.first;
}

// host-only: the choice above for a product described by its sizes and pitches (decx_hip_hgemm_plan)
int hgemm_plan(int M, int N, int K, int batch, long lda, long ldb, bool aligned, int* splits) {
    return plan_hgemm(M, N, K, batch, aligned && hgemm_pitches_fit(lda, ldb), splits);
}

int hgemm_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                  int ldd, int M, int N, int K, const Batch& batch) {
    if (int rc = check_gemm_args(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch)) return rc;
    int splits = 0;
    const bool vec = hgemm_vector_path(A, lda, B, ldb, batch);
    const HgemmWholeRoundsSplit split = plan_hgemm_whole_rounds_split(M, N, K, batch.count, vec);
    // the first launch of a split: whole rounds of the 256x256 tile, as the stream of K steps where plan_hgemm would take that
    auto whole_rounds = [&](int rows, int cols) -> int {
        if (K <= 3072 && hgemm_mfma16_persistent_fits<HShape16>(rows, cols, K, batch))
            return launch_hgemm_mfma16_persistent<HShape16>(A, lda, B, ldb, Cin, ldc, D, ldd, rows, cols, K, batch);
        return launch_hgemm_mfma16<HShape16>(A, lda, B, ldb, Cin, ldc, D, ldd, rows, cols, K, batch);
    };
    if (split.first > 0 && !split.by_columns) {
        if (int rc = whole_rounds(split.first, N)) return rc;
        return hgemm_enqueue(A + (size_t)split.first * lda, lda, B, ldb, Cin ? Cin + (size_t)split.first * ldc : nullptr, ldc,
                             D + (size_t)split.first * ldd, ldd, M - split.first, N, K, batch);
    }
    if (split.first > 0) {
        if (int rc = whole_rounds(M, split.first)) return rc;
        return hgemm_enqueue(A, lda, B + split.first, ldb, Cin ? Cin + split.first : nullptr, ldc, D + split.first, ldd, M,
                             N - split.first, K, batch);
    }
    int variant = plan_hgemm(M, N, K, batch.count, vec, &splits);
    if (variant == 0) return launch_hgemm_tile<HShapeSmall, false>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 11) return hgemm_splitk_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, splits, batch.stream);
    if (variant == 17) {
        if (hgemm_mfma16_persistent_fits<HShape16>(M, N, K, batch))
            return launch_hgemm_mfma16_persistent<HShape16>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
        variant = 15;
    }
    if (variant == 15) return launch_hgemm_mfma16<HShape16>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
    if (variant == 16) return launch_hgemm_mfma16<HShape16K32S4>(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch);
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

// ---------------------------------------------------------------------------------------------------------------
// The K-range route on a workspace that is part of the library's code object instead of an allocation: for callers
// that must not allocate device memory (serving loops, harnesses that forbid it).  Every GPU
// the library is loaded on holds its own copy of the array until the process ends; host code reaches it only through
// the address hipGetSymbolAddress returns for the current device.
// ---------------------------------------------------------------------------------------------------------------
constexpr size_t kScratchBytes = DECX_HIP_STATIC_WORKSPACE_BYTES;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kMaxDevices = 64;
static float* g_scratch_ptr[kMaxDevices] = {};

int hgemm_static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "device ordinal out of range\n");
    if (g_scratch_ptr[device]) return 0;
    void* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));     // the current device's copy
    if (!ptr) return fail(DECX_HIP_FAIL_ALLOCATION, "the static workspace has no device address\n");
    if (int rc = allow_split_kernel_lds()) return rc;            // done here so that the entry point only launches
    g_scratch_ptr[device] = static_cast<float*>(ptr);
    return 0;
}

int hgemm_splitk_static_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                uint16_t* D, int ldd, int M, int N, int K, int splits) {
    Batch one;
    one.stream = g_rt.stream;
    if (int rc = check_gemm_args(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, one)) return rc;
    float* workspace = g_rt.device >= 0 && g_rt.device < kMaxDevices ? g_scratch_ptr[g_rt.device] : nullptr;
    if (!workspace) return fail(DECX_HIP_FAIL_NOT_INIT, "CUDA should be initialized first\n");
    if (!hgemm_vector_path(A, lda, B, ldb, one))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "the allocation-free entry point needs 16-byte aligned A, B with lda, ldb multiples of 8\n");
    if (splits <= 0) splits = auto_hgemm_splits(M, N, K);
    if (splits < 1) splits = 1;                                  // one range: still through the workspace, no allocation
    if (splits > (K + 63) / 64) splits = (K + 63) / 64;
    const SplitPlan plan = plan_hgemm_split(K, splits);
    const size_t need = (size_t)M * N * sizeof(float) * plan.splits;
    if (need > kScratchBytes)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS,
                    "M*N*4 bytes times %d K ranges = %zu bytes exceed the static workspace of %zu bytes; use decx_hip_hgemm_f32acc\n",
                    plan.splits, need, kScratchBytes);
    // always one plane per range, added in range order: nothing in the workspace has to start at zero
    return hgemm_splitk_launch(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, plan, workspace, true, g_rt.stream);
}

}  // namespace decx_hip
