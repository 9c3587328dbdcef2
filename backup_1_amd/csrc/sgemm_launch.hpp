// fp32 tile launchers, the table of tile shapes and the shape choosers, shared by the dense GEMM and the convolution
// translation units (each instantiates the kernels for its own operand sources).
#pragma once
#include "runtime.hpp"
#include "sgemm_tile.hpp"

namespace decx_hip {

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
//  16: shape 2 compiled for one wave per SIMD (two staging sets, one workgroup per CU): ahead of shape 2 wherever the
//         cost model picks 128x128 tiles (2048^3: 0.140 -> 0.126 ms; 2048x2048x4096, two rounds: 0.259 -> 0.247 ms)
//  15: 224x128x16, 2x4 waves of 128x32 (upper row) and 96x32 (lower row) -- shape 6 on two waves per SIMD: each SIMD
//         carries a 4-block and a 3-block wave
//  17: 208x128x16, 2x4 waves of 112x32 (three 32-row blocks and one of 16 rows on v_mfma_f32_16x16x4_f32) and 96x32:
//         convolution only (filter-bank B); 6 1/2 blocks per SIMD for results whose rows fill the CUs badly in steps of 32
// the one-wave-per-16x16-block kernel of sgemm_chain16.hpp (dense GEMM and small-image convolutions):
//  11:  32x32x64,  2x2 computing + 4 moving waves, two workgroups per CU -- results too small to fill the chip with tiles
//  12:  16x16x64,  1 computing + 2 moving waves -- at most one 16x16 block per CU: the fastest a single chain can walk K
//  13:  64x64x64,  8 computing waves of two blocks each + 4 moving waves -- results of about one such tile per CU (1024^2)
//  23:  16x32x64,  2 computing + 2 moving waves, one per SIMD -- at most one such tile per CU
// and, for dense GEMM only, the tiles fed by LDS-DMA loads of sgemm_dma_tile.hpp (2x2 waves, one per SIMD):
//  18:  64x64, K steps of 32 in 4 LDS buffers     19:  64x64, K steps of 64 in 3 buffers
//  20: 128x128 on 4x2 waves of 32x64 (two per SIMD), K steps of 16 in 2 buffers; 21: 64x128, 22: 128x64 (four waves), K steps of 32 in 4 buffers
//  24:  32x32 on 16x16 blocks (v_mfma_f32_16x16x4_f32), K steps of 64 in 3 buffers     25: 64x32, two blocks per wave
//  26: 256x256 on 4x2 waves of 64x128 (two per SIMD), K steps of 16 in 2 buffers -- the large-problem default
//  27: 256x224 on 8x1 waves of 32x224 -- for results that 224 columns tile better than 256     28: 256x192, likewise
// and, for convolutions with a channel pitch that is a multiple of 32 and filters in fours, the LDS-DMA kernel on 16x16
// blocks of sconv_dma.hpp (K steps of 32 in 2 buffers, eight waves, two per SIMD):
//  29: 208x128 (a patch of 16 x 13 pixels) on 1x8 waves of 13x1 blocks -- 6 1/2 block rows of 32 for results of 196 rows per CU (224x224 pixels)
//  30: 256x256 (16 x 16 pixels) on 2x4 waves of 8x4 blocks -- measured behind shape 7 (512x512x256 under 256 filters: 148.1 against 149 TFLOP/s), not chosen by itself
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
typedef SgemmShape<208, 128, 16, 2, 4, 2, 2, true, true> SShape208Split;   // 8 waves, 3 1/2 + 3 row blocks per SIMD (filter-bank B only)
typedef SgemmShape<128, 128, 16, 2, 2, 1> SShapeSmallSolo;
typedef SgemmShape<64, 64, 16, 2, 2, 4> SShapeTiny;      // 2x2 waves of 32x32
typedef SgemmShape<128, 64, 16, 2, 2, 4> SShapeTiny2;    // 2x2 waves of 64x32

// Tile shape by a small cost model: a CU works through ceil(tiles / CUs) tiles one after another (tiles that share a CU
// share its matrix pipe, so residency does not change this), a tile costs its area divided by how well that shape keeps
// the pipe busy (measured on large squares, relative to shape 7).  The 256x128 and 224x128 shapes come in a
// two-workgroups-per-CU build, better on short K walks where one tile's prologue and epilogue overlap the other's loop,
// and a one-workgroup-per-CU build with deeper prefetch, better on long ones (224x128: shape 15, which measured 5-6 %
// ahead of shape 6 on the 224x224x64 convolution under 128 filters; the same split of the 224x256 tile, and 256x128 on
// 8 waves of 128x32, measured no better than shapes 10 and 5 and are not built).
inline int pick_sgemm_variant(int M, int N, int K, int batch, bool dense = false, double* cost_out = nullptr) {
    if ((g_rt.sgemm_variant >= 1 && g_rt.sgemm_variant <= 10) || (g_rt.sgemm_variant >= 15 && g_rt.sgemm_variant <= 17)) return g_rt.sgemm_variant;
    if (g_rt.sgemm_variant == 14) return dense ? 14 : 2;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    // At most 8 K steps and several rounds of tiles: the launch is bound by writing the result, and two small workgroups
    // per CU overlap one tile's stores with the other's K walk (8192x64x8192: 0.100 -> 0.091 ms, 4096x128x4096: 0.0430
    // -> 0.0417 ms against the big tiles).
    // (a result at most 64 wide: 128x64 tiles -- 400000x32x64: 52.1 -> 29.3 us, 500000x64x48: 52.8 us against 64.7 on the
    // 64x64 LDS-DMA tiles)
    if (K <= 128 && (long)cdiv(M, 128) * cdiv(N, 128) * batch >= 2 * cus) return N <= 64 ? 9 : 2;
    struct Cand { int variant, bm, bn; double eff; };
    const Cand cands[] = {{7, 256, 256, 1.00}, {10, 224, 256, 0.96}, {3, 256, 128, 0.95}, {4, 224, 128, 0.94}, {2, 128, 128, 0.92},
                          {9, 128, 64, 0.83}, {8, 64, 64, 0.78}, {14, 192, 192, 0.93}, {17, 208, 128, 0.90}};
    int best = 7;
    double best_cost = 0.0;
    for (const Cand& c : cands) {
        if (c.variant == 14 && !dense) continue;
        // 208 rows (a block of 16 among them): filter-bank B only, and only as the single round of a launch that 224-row
        // tiles would leave an eighth of the chip idle in (224x224x64 under 128 filters: 242 tiles, 65.0 -> 63.0 us)
        if (c.variant == 17 && (dense || (long)cdiv(M, c.bm) * cdiv(N, c.bn) * batch > cus)) continue;
        const long tiles = (long)cdiv(M, c.bm) * cdiv(N, c.bn) * batch;
        const double cost = (double)((tiles + cus - 1) / cus) * c.bm * c.bn / c.eff;
        if (best_cost == 0.0 || cost < best_cost) {
            best_cost = cost;
            const bool one_per_cu = tiles <= cus || K >= 1024;
            best = one_per_cu && c.variant == 3 ? 5 : one_per_cu && c.variant == 4 ? 15 : c.variant == 2 ? 16 : c.variant;
        }
    }
    if (cost_out) *cost_out = best_cost;
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
        case 16: return launch_sgemm_tile<SShapeSmallSolo>(a, b, Cin, ldc, D, out, M, N, K, batch);
        case 17:
            if constexpr (!BSrc::ROW_MAJOR_LDS) return launch_sgemm_tile<SShape208Split>(a, b, Cin, ldc, D, out, M, N, K, batch);
            else return launch_sgemm_tile<SShape224Split>(a, b, Cin, ldc, D, out, M, N, K, batch);
        default: return launch_sgemm_tile<SShapeSmall>(a, b, Cin, ldc, D, out, M, N, K, batch);
    }
}

// Which shape of the one-wave-per-block kernel (sgemm_chain16.hpp) a result of M x N takes, or 0 for the tiles.
// Measured: ahead of the tiles up to about ten 32x32 tiles per CU -- 1536x1536 on 256 CUs -- 1.7x at 1024x8192x1024, 9x at
// 64x65536x1024.  All paths give the same bits, so this is a choice of speed only.
inline int pick_chain_shape(int M, int N, int K, int batch) {
    if ((g_rt.sgemm_variant >= 11 && g_rt.sgemm_variant <= 13) || g_rt.sgemm_variant == 23) return g_rt.sgemm_variant;
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
    // At most one 16x16 block per CU: shape 12.  More, but at most one 16x32 tile per CU: shape 23, whose chains run as
    // undisturbed (128x16384x1024: 98.6 -> 59.5 us, 196x4608x512: 29.9 -> 18.9 us, 64x65536x2048: 389 -> 319 us).
    if (blocks16 <= cus) return 12;
    if ((long)cdiv(M, 16) * cdiv(N, 32) * batch <= cus) return 23;
    return tiles32 > tile_limit ? 0 : cost64 < cost32 ? 13 : 11;
}

// The tiles fed by LDS-DMA loads (sgemm_dma_tile.hpp) address a tile's rows with 32-bit byte offsets from the tile's
// first row: 255 rows (the tallest tile has 256) of a pitch below 2^21 floats stay below 2^31 bytes.
constexpr int kDmaMaxPitch = 1 << 21;

// The shapes of the LDS-DMA kernel are instantiated in four translation units (sgemm_dma_small.hip, sgemm_dma_blocks16.hip,
// sgemm_dma_large.hip, sgemm_dma_wide.hip).
int launch_sgemm_dma_small(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu);
int launch_sgemm_dma_blocks16(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu);
int launch_sgemm_dma_large(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu);
int launch_sgemm_dma_wide(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu);
inline int launch_sgemm_dma_shape(int shape, const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N, int K, const Batch& batch, bool relu) {
    if (shape >= 28) return launch_sgemm_dma_wide(shape, A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape >= 26) return launch_sgemm_dma_large(shape, A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    if (shape == 20 || shape >= 24) return launch_sgemm_dma_blocks16(shape, A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
    return launch_sgemm_dma_small(shape, A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, batch, relu);
}

// Which shape of the LDS-DMA kernel a result of M x N takes, or 0 for the other kernels.  Measured on 256 CUs against
// the automatic choice among the others: ahead from about half a 64x64 tile per CU (768^2: 16.1 -> 14.5 us) to about six
// (2560^2: 270 -> 266 us), by most around one per CU (1024^3: 23.3 -> 18.3 us, 1024x8192x1024: 158 -> 122 us); below, the
// block-chain kernels fill more of the chip, above, the big tiles re-use their operands better.  Steps of 64 k in three
// buffers (96 KiB: one workgroup per CU) are ahead on a long K with at most one tile per CU, steps of 32 k in four
// buffers (64 KiB: two workgroups share a CU) everywhere else.  Shapes 20 - 22 are 128x128, 64x128 and 128x64 tiles of
// the same kernel, 24 and 25 tiles of 32x32 and 64x32 on 16x16 blocks, 26, 27 and 28 the 256x256, 256x224 and 256x192 tiles on eight waves; all but 21 and 22
// are chosen automatically.  All paths give the same bits.
inline int pick_dma_shape(int M, int N, int K, int batch) {
    if ((g_rt.sgemm_variant >= 18 && g_rt.sgemm_variant <= 22) || (g_rt.sgemm_variant >= 24 && g_rt.sgemm_variant <= 28)) return g_rt.sgemm_variant;
    if (g_rt.sgemm_variant != 0) return 0;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long tiles64 = (long)cdiv(M, 64) * cdiv(N, 64) * batch, tiles128 = (long)cdiv(M, 128) * cdiv(N, 128) * batch;
    const long tiles32 = (long)cdiv(M, 32) * cdiv(N, 32) * batch;
    // 128x128 tiles on eight waves (4 x 2 of 32x64, two per SIMD) in one or two rounds whose last is at least 7/8 full:
    // 2048^3 128.5 -> 118.2 us (145 TFLOP/s), 2048x8192x2048 501 -> 456 us (151 TFLOP/s), 1920^2 x 4096 245 -> 231 us,
    // 2816^2 x 4096 482 -> 459 us
    {
        const long last = tiles128 % cus == 0 ? cus : tiles128 % cus;
        // ... and whose tiles are at least 85 % result (30000x512x48: a tile 128 wide is 5/8 padding, 32.7 us against 19.6
        // on 64x64 tiles)
        const bool mostly_result = 100.0 * M * N * batch >= 85.0 * 16384.0 * tiles128;
        if (tiles128 <= 2 * cus && 8 * last >= 7 * cus && mostly_result) return 20;     // (1920^2: 225 tiles of 256)
    }
    // Cycles per k of a launch, measured over squares of 384 .. 1792 at K = 1024 and 8192: a round of 64x64 tiles (one
    // per CU) walks K at 34.2, a round of 32x32 tiles of 16x16 blocks at 9.7.  The small tiles win where the 64x64 ones
    // fill their last round badly (1152^2: 324 tiles = 2 rounds against 1296 = 6 rounds: 235 -> 193 us at K = 8192;
    // 768^2: 117 -> 95 us; 1536^2: 359 -> 311 us) and below half a 64x64 tile per CU (512x8192x512: 51 -> 36 us).
    const double walk64 = 34.2 * (double)((tiles64 + cus - 1) / cus), walk32 = 9.7 * (double)((tiles32 + cus - 1) / cus);
    // where the register-staged kernel would run its 256x256 tiles on two waves per SIMD (shape 7), the same tile fed by
    // LDS-DMA loads is 0.6 - 1 % ahead (8192^3: 150.5 -> 151.9 TFLOP/s, 4096^3: 148.9 -> 150.0, 8192x2048x8192: 147.9 -> 148.9):
    // MFMA busy 98.3 % against 97.5 %
    if (4 * tiles64 > 25 * cus) {
        double cost = 0.0;
        const int tiled = pick_sgemm_variant(M, N, K, batch, true, &cost);
        if (K >= 512) {
            // the 256x224 tile of the same kernel (eight waves of 32x224) in that cost model: 3000x1500x4500 (252 tiles either
            // way) 311 -> 305 us against the register-staged 224x256 tile, 8192x8192x7168 6612 -> 6350 us
            const long tiles224 = (long)cdiv(M, 256) * cdiv(N, 224) * batch, tiles192 = (long)cdiv(M, 256) * cdiv(N, 192) * batch;
            const double cost224 = (double)((tiles224 + cus - 1) / cus) * 256 * 224 / 0.975;
            // and the 256x192 tile (eight waves of 32x192): 6144^3 is 768 of them, three whole rounds: 3186 -> 3075 us (150.8 TFLOP/s)
            const double cost192 = (double)((tiles192 + cus - 1) / cus) * 256 * 192 / 0.975;
            if (cost > 0.0 && cost192 < cost && cost192 < cost224) return 28;
            if (cost > 0.0 && cost224 < cost) return 27;
            if (tiled == 7) return 26;
        }
        // A tall result at most 32 wide: the 64x32 tiles of 16x16 blocks are the only ones that do not pad it to 64 columns
        // (200000x1024x32: 271 -> 172 us, 150000x2304x32: 407 -> 269, 400000x128x32: 128 -> 54, 600000x576x16: 401 -> 285)
        if (N <= 32) return 25;
        if (N <= 256) {
            // At most 256 wide on a short K: bound by the epilogue.  Up to 64 columns the register-staged 128x64 tiles
            // (pick_sgemm_variant) up to K = 128, the 64x64 LDS-DMA tiles from there (200000x256x64: 68.1 -> 65.7 us);
            // beyond 64 columns the 128x128 LDS-DMA tiles (200000x128x128: 67.4 -> 62.9 us, 200000x96x96: 60.3 -> 49.7,
            // 60000x256x100: 45.6 -> 35.4)
            if (K <= 128 && N <= 64) return 0;
            if (K <= 256) return N <= 64 ? 18 : 20;
            // On a longer K, in microseconds: the tile cost at one CU's matrix peak after 8 us, against
            //  - the 64x32 tiles of 16x16 blocks, which every SIMD walks at 8 cycles per k and block, at 0.93 K / (K + 280)
            //    of the matrix pipe's pace, but at most 0.75 (launches of several hundred microseconds on real-valued data
            //    run into the power limit, where the small tiles' extra LDS traffic costs clock: 100000x4096x128 runs at
            //    0.88 on zeros and 0.77 on uniform data), after 4 us: ahead where the wide tiles pad the columns heavily
            //    (82944x864x96: 165.6 -> 134.5 us; 64 rows per tile are ahead of 32 in this many rounds: 144.7 -> 134.5).
            //    The tile model's efficiencies are those of a long K; against these tiles the big tiles' prologue and
            //    epilogue weigh 150 k more (82944x864x224 on 224x128 tiles: 358 us against the model's 265);
            //  - the 64x64 tiles fed by LDS-DMA loads, at 85 % in the tile model, for one or two of them across: ahead of
            //    the register-staged 128x64 and 64x64 ones (409600x576x64: 301.7 -> 291.5 us, 200704x288x64: 79.7 -> 74.9);
            //  - the 128x128 tiles fed by LDS-DMA loads where at least 85 % of them is result, at 96 % in the tile model
            //    (147456x1152x128: 352 us on the 64x64 tiles -> 340, 150000x2048x256: 1219 on the 256x128 tile -> 1167).
            const double us_per_cost = K * 2.0 / 614.5e3;
            const double t_tiles = cost > 0.0 ? 8.0 + cost * us_per_cost : 1e30;
            const double small_pace = std::min(0.75, 0.93 * K / (K + 280.0));
            const double t_small = K >= 512 ? 4.0 + (double)tiles32 / cus * K * 8.0 / 2400.0 / small_pace : 1e30;
            const double t_64 = N <= 128 ? 8.0 + (double)((tiles64 + cus - 1) / cus) * 4096.0 / 0.85 * us_per_cost : 1e30;
            const bool mostly_result128 = 100.0 * M * N * batch >= 85.0 * 16384.0 * tiles128;
            const double t_128 = mostly_result128 ? 8.0 + (double)((tiles128 + cus - 1) / cus) * 16384.0 / 0.96 * us_per_cost : 1e30;
            if (t_small < t_tiles * (K + 150.0) / K && t_small < t_64 && t_small < t_128) return 25;
            if (t_128 < t_tiles && t_128 < t_64) return 20;
            if (t_64 < t_tiles) return 18;
        }
    }
    if (2 * tiles64 >= cus && 4 * tiles64 <= 25 * cus) {
        if (walk32 < 1.05 * walk64) return 24;      // (a tie goes to the small tiles: 1280^2 237 -> 230 us, 1664^2 379 -> 366 us)
        return tiles64 <= cus && K >= 1024 ? 19 : 18;
    }
    // fewer tiles than that: the block-chain shapes 12 and 23 (pick_chain_shape) keep their results -- one chain per
    // CU walks a very long K with less trouble from pitches of a power of two -- the 32x32 tiles take the rest
    if (2 * tiles64 < cus && (long)cdiv(M, 16) * cdiv(N, 32) * batch > cus) return 24;
    return 0;
}

// The kernel decx_hip_sgemm takes for a product, as the number decx_hip_set_sgemm_variant would force it with: a shape
// of the LDS-DMA tiles (18 - 22, 24 - 28) where both pitches leave a tile's byte offsets in 32 bits, else a shape of the
// one-wave-per-block kernel (11 - 13, 23), else a register-staged tile (1 - 10, 14 - 17); 0 = operands that the vector
// loaders cannot take (not 16-byte aligned, pitch not in fours): the 128x128 tile with element-wise loaders.
inline int plan_sgemm(int M, int N, int K, int batch, bool vec_a, bool vec_b, long lda, long ldb) {
    if (!(vec_a && vec_b)) return 0;
    if (lda < kDmaMaxPitch && ldb < kDmaMaxPitch) {
        const int dma = pick_dma_shape(M, N, K, batch);
        if (dma) return dma;
    }
    const int chain = pick_chain_shape(M, N, K, batch);
    if (chain) return chain;
    return pick_sgemm_variant(M, N, K, batch, true);
}

// What one launch of the automatic choice costs, in the tile model's unit (tile area per CU / efficiency; times
// 2 K / 614.5e3 it is microseconds), or 0 where the model has no figure (the block-chain kernels).  It prices the kernel
// plan_sgemm answers, with the pickers' own figures; the planner below compares such prices, it picks no kernel.
inline double sgemm_one_launch_cost(int M, int N, int K, int batch, long lda, long ldb) {
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long tiles64 = (long)cdiv(M, 64) * cdiv(N, 64) * batch, tiles32 = (long)cdiv(M, 32) * cdiv(N, 32) * batch;
    auto rounds = [cus](long tiles) { return (double)((tiles + cus - 1) / cus); };
    // cycles per k of the small LDS-DMA tiles (pick_dma_shape) in the model's unit: 614.5e3 / 2 / 2400 per cycle
    const double per_cycle = 128.0;
    const int plan = plan_sgemm(M, N, K, batch, true, true, lda, ldb);
    switch (plan) {
        case 26: return rounds((long)cdiv(M, 256) * cdiv(N, 256) * batch) * 65536.0 / 0.975;
        case 27: return rounds((long)cdiv(M, 256) * cdiv(N, 224) * batch) * 57344.0 / 0.975;
        case 28: return rounds((long)cdiv(M, 256) * cdiv(N, 192) * batch) * 49152.0 / 0.975;
        case 20: return rounds((long)cdiv(M, 128) * cdiv(N, 128) * batch) * 16384.0 / 0.96;
        case 18: case 19: return rounds(tiles64) * 34.2 * per_cycle;
        case 24: case 25:
            if (4 * tiles64 > 25 * cus) return (double)tiles32 / cus * 1024.0 / std::min(0.75, 0.93 * K / (K + 280.0));
            return rounds(tiles32) * 9.7 * per_cycle;
        case 11: case 12: case 13: case 23: return 0.0;
        default: break;
    }
    double cost = 0.0;
    pick_sgemm_variant(M, N, K, batch, true, &cost);
    return cost;
}

// A result whose 256-row tiles come in whole rounds plus a part of one (a round = one tile per CU) pays a whole round for
// the part.  Every element's sum is the same chain of products whatever tile computes it, so the rows -- or columns --
// that fill whole rounds can go to one launch of such tiles and the rest to a second launch, which picks its own tiles
// (4096x4608: 288 tiles of 256x256; 4096 columns in one round, the other 512 on 128 tiles of 128x128, against two rounds
// of 256x192).  The plan: for each of the three 256-row LDS-DMA tiles, whole rounds of it plus the one-launch cost of the
// rest plus 4 us for the second launch; taken where the cheapest is under 96 % of the one-launch cost of the whole.
struct WholeRoundsSplit {
    int shape = 0;          // 26 - 28: the tile of the first launch; 0 = one launch
    bool by_columns = false;
    int first = 0;          // rows (columns) of the first launch
};
inline WholeRoundsSplit plan_whole_rounds_split(int M, int N, int K, int batch, long lda, long ldb) {
    WholeRoundsSplit plan;
    if (g_rt.sgemm_variant != 0 || batch != 1 || K < 512 || lda >= kDmaMaxPitch || ldb >= kDmaMaxPitch) return plan;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    if (4 * (long)cdiv(M, 64) * cdiv(N, 64) <= 25 * cus) return plan;
    const double whole_cost = sgemm_one_launch_cost(M, N, K, 1, lda, ldb);
    if (whole_cost == 0.0) return plan;
    double best = 0.96 * whole_cost;
    const double second_launch = 4.0 * 614.5e3 / (2.0 * K);
    const int shapes[3] = {26, 27, 28}, widths[3] = {256, 224, 192};
    for (int i = 0; i < 3; ++i) {
        const long tiles_m = cdiv(M, 256), tiles_n = cdiv(N, widths[i]), whole = tiles_m * tiles_n / cus;
        if (whole < 1 || tiles_m * tiles_n % cus == 0) continue;
        const double first_cost = (double)whole * 256.0 * widths[i] / 0.975;
        for (int by_columns = 0; by_columns < 2; ++by_columns) {
            const long lines = whole * cus / (by_columns ? tiles_m : tiles_n);          // whole tile rows (columns) in the whole rounds
            if (lines < 1 || lines >= (by_columns ? tiles_n : tiles_m)) continue;
            const int first = (int)lines * (by_columns ? widths[i] : 256);
            const double rest = by_columns ? sgemm_one_launch_cost(M, N - first, K, 1, lda, ldb) : sgemm_one_launch_cost(M - first, N, K, 1, lda, ldb);
            if (rest == 0.0) continue;
            const double cost = first_cost + rest + second_launch;
            if (cost < best) {
                best = cost;
                plan.shape = shapes[i], plan.by_columns = by_columns != 0, plan.first = first;
            }
        }
    }
    return plan;
}

// shape 33 (convolution: the automatic choice with the small-image kernel kept out of it) and shape 34 (dense products:
// the automatic choice in one launch, plan_whole_rounds_split switched off) are for experiments and tests: the rest of
// the call sees shape 0
struct ShapeForThisCall {
    int saved;
    explicit ShapeForThisCall(int shape) : saved(g_rt.sgemm_variant) { g_rt.sgemm_variant = shape; }
    ~ShapeForThisCall() { g_rt.sgemm_variant = saved; }
};

}  // namespace decx_hip
