// fp16 fused im2col convolution with fp32 accumulation: kernel choice and launch (hconv_mfma16.hpp for images that give
// at least a quarter of the CUs a tile and have a channel pitch in 64s, else hconv_taprow.hpp, hconv_dma.hpp,
// hconv_tile.hpp), split over K for small images.
#include "runtime.hpp"
#include "hconv_tile.hpp"
#include "hconv_dma.hpp"
#include "hconv_taprow.hpp"
#include "hconv_mfma16.hpp"

namespace decx_hip {

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
    // a K step of 64 halves inside one tap: the kernel on v_mfma_f32_16x16x32_f16 with patch-shaped tiles (hconv_mfma16.hpp).
    // Its column test adds 2^31 to an offset, which must throw it out of the tensor's range even from the apron's negative
    // offsets, and its patches reach up to 15 rows and 15 columns past the output: those offsets must stay below 2^31 as
    // well.  hgemm variant 18 takes it for any image it can run on; by itself it takes the images whose patches give at
    // least a sixth of the CUs a tile (56x56x256 under 256 filters: 64 tiles of 64 filters 17.2 us, split over K 22.8;
    // 112x112x64 under 64 filters: 49 tiles 6.9 us against 7.9), and then before the split over K is considered.
    const bool kernel_forced = (g_rt.hgemm_variant >= 12 && g_rt.hgemm_variant <= 14) || g_rt.hgemm_variant == 18;      // experiments and tests: no split
    const bool fits16 = tap_uniform && conv_patch_offsets_fit(src_bytes, src_row_stride, (size_t)dpitch, kh, kw, oy, ox, 2);
    const long patches = (long)cdiv(Hout, 16) * cdiv(Wout, 16);
    // tiles 256 filters wide (half the image traffic per filter) where they still give half of the CUs a tile (measured:
    // 224x224x64 under 256 filters, 196 patches, 18.6 us against 21.1 on 392 tiles of 128 filters; 112x112x128 under
    // 256, 49 patches, 24.9 against 15.6), 64 wide for at most 64 filters (the wider ones would spend their matrix
    // instructions on filters that do not exist: 1024x512x64 under 64 filters 65.9 -> 49.1 us against the tap-row kernel)
    const bool wide = N > 128 && 2 * patches * cdiv(N, 256) >= cus;
    // ... and also where tiles of 128 filters would leave half of the CUs without one (measured: 112x112x128 under 256
    // filters 15.0 -> 11.6 us, 128x128x128 under 128 filters 14.9 -> 10.8 us; at 196 patches under 128 filters 10.5 -> 14.5)
    const bool slim = N <= 64 || 2 * patches * cdiv(N, 128) <= cus;
    const long tiles16 = patches * cdiv(N, wide ? 256 : slim ? 64 : 128);
    bool take16 = fits16 && tiles16 <= 0x7fffffffL &&
                  (g_rt.hgemm_variant == 18 || (!kernel_forced && 6 * tiles16 >= cus && g_rt.hgemm_variant != 19));
    // small image: few tiles and many K steps -> ranges of K steps as separate workgroups, fp32 partial sums in the
    // workspace, bias / ReLU / rounding in a finishing kernel
    // Measured model, in us: a workgroup walks a K step of 64 halves in 0.75 us (1.3 x that once two workgroups share a
    // CU's LDS bandwidth); the split pays 9 us for fill, finishing kernel and a third launch, and 3.1 ps per atomic add.
    const int all_steps = cdiv(Kw, 32);
    const long square_tiles = (long)cdiv(M, 128) * tiles_n;
    int splits = 1;
    if (!kernel_forced && !take16 && !tall && 2 * square_tiles <= cus && all_steps >= 8 && (size_t)M * N <= ((size_t)1 << 26)) {
        const double t_whole = 4.0 + 0.75 * all_steps;
        double best = 0.85 * t_whole;
        const long most = (2 * cus + square_tiles - 1) / square_tiles;
        for (int s = 2; s <= most && s <= all_steps / 2; ++s) {
            const double share = square_tiles * s > cus ? 1.3 : 1.0;
            const double t = 9.0 + 3.1e-6 * M * N * s + 0.75 * share * cdiv(all_steps, s);
            if (t < best) best = t, splits = s;
        }
        // the 16x16x32 kernel on a single round of tiles, in the same model: 5 us fixed + 0.34 us per K step (measured at
        // 16 - 64 tiles: 64x64x256 under 128 filters 17.1 us against 20.0 for the split, 28x28x512 under 512 30.8 against 21.7)
        if (fits16 && tiles16 <= cus && g_rt.hgemm_variant != 19 && 5.0 + 0.34 * all_steps < best) {
            take16 = true;
            splits = 1;
        }
    }
    if (splits > 1) {
        const int steps_per_split = cdiv(all_steps, splits);
        splits = cdiv(all_steps, steps_per_split);                     // no empty range
        const bool ordered = !g_rt.splitk_atomic;             // one workspace plane per range, added in range order
        if (int rc = ensure_partial((size_t)M * N * sizeof(float) * (ordered ? splits : 1))) return rc;
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
        if (!ordered) enqueue_zero_region(g_rt.partial, N, M, N, g_rt.stream);
        const size_t plane = ordered ? count : (size_t)0;
        const dim3 grid((unsigned)total, (unsigned)splits);
        if (tap_uniform)
            hipLaunchKernelGGL((hconv_tile_kernel<HconvSquare, true, true>), grid, dim3(HconvSquare::NT), HconvSquare::LDS_BYTES,
                               g_rt.stream, img, fb, out, M, N, Kw, tiles_n, g_rt.partial, steps_per_split, plane);
        else
            hipLaunchKernelGGL((hconv_tile_kernel<HconvSquare, false, true>), grid, dim3(HconvSquare::NT), HconvSquare::LDS_BYTES,
                               g_rt.stream, img, fb, out, M, N, Kw, tiles_n, g_rt.partial, steps_per_split, plane);
        hipLaunchKernelGGL(hconv_split_finish_kernel, dim3(fill_blocks), dim3(256), 0, g_rt.stream, g_rt.partial, ordered ? splits : 1, count,
                           out, M, N);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    {
        if (take16) {
            // on output rows row0 .. row0 + rows - 1: the kernel places output row y of the part at image row y - (oy - row0),
            // so a part further down is the same launch with oy moved and dst advanced
            auto launch16 = [&](auto shape, int row0, int rows) -> int {
                typedef decltype(shape) S;
                static bool attr_done = false;           // one per shape: the lambda's body is instantiated per S
                if (!attr_done) {
                    HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(hconv_mfma16_kernel<S>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                (int)S::LDS_BYTES));
                    attr_done = true;
                }
                HalfImage part_img = img;
                part_img.oy = oy - row0, part_img.Mtot = rows * Wout;
                HalfTensorOut part_out = out;
                part_out.dst = out.dst + (size_t)row0 * dst_row_stride;
                const int tn = cdiv(N, S::BN), tx = cdiv(Wout, S::PATCH_X);
                const long part_patches = (long)cdiv(rows, S::PATCH_Y) * tx;
                hipLaunchKernelGGL(hconv_mfma16_kernel<S>, dim3((unsigned)(part_patches * tn)), dim3(S::NT), S::LDS_BYTES, g_rt.stream, part_img, fb,
                                   part_out, rows, N, tx, (int)part_patches, tn);
                HIP_TRY(hipGetLastError());
                return 0;
            };
            auto launch_rows = [&](int row0, int rows) -> int {
                const long part_patches = (long)cdiv(rows, 16) * cdiv(Wout, 16);
                if (N > 128 && 2 * part_patches * cdiv(N, 256) >= cus) return launch16(Hconv16Shape<256, 2, 4>{}, row0, rows);      // 2x4 waves of 128 pixels x 64 filters
                if (N <= 64 || 2 * part_patches * cdiv(N, 128) <= cus) return launch16(Hconv16Shape<64, 8, 1>{}, row0, rows);      // 8x1 waves of 32 pixels x 64 filters
                return launch16(Hconv16Shape<128, 4, 2>{}, row0, rows);                // 4x2 waves of 64 pixels x 64 filters
            };
            // The tiles run one per CU: tiles beyond whole rounds of them pay a round of their own (268x268x128 under 256
            // filters, 289 tiles: 58.4 us where 256 tiles take 35.7), and a nearly empty round still costs two thirds of
            // a full one.  With the 256-filter tiles, while the part is at most a quarter of a round, the image rows that
            // fill the whole rounds go to one launch and the rows below to a second one on narrower tiles, which spread
            // them over the chip (hgemm variant 20 keeps one launch).  Not with the narrower tiles: measured, under 128
            // filters the second launch gains 0 - 2 %, and under 64, where it has no narrower tile to go to, loses 4 - 22 %.
            if (wide && g_rt.hgemm_variant == 0) {
                const long row_tiles = (long)cdiv(Wout, 16) * cdiv(N, 256), whole = tiles16 / cus, part = tiles16 % cus;
                const long first = whole * cus / row_tiles * 16;          // image rows whose tiles fit the whole rounds
                if (whole >= 1 && part > 0 && 4 * part <= cus && first >= 16 && first < Hout) {
                    if (int rc = launch_rows(0, (int)first)) return rc;
                    return launch_rows((int)first, Hout - (int)first);
                }
            }
            return launch_rows(0, Hout);
        }
    }
    // filters 3, 5 or 7 wide: the LDS-DMA kernel that loads a tap row's pixels once for all of its taps, if a tile's patch
    // fits its 320 rows (255 + kw positions plus kw - 1 per image row the tile touches).  hgemm variant 14 takes it for
    // any image; its tiles are 64 filters wide when there are no more filters than that.
    const int rows_touched = (254 + Wout) / Wout + 1;
    const bool taprow_fits = tap_uniform && (kw == 3 || kw == 5 || kw == 7) && 255 + kw + (kw - 1) * rows_touched <= 320 &&
                             (long)H * W < (1L << 22);
    const bool narrow = N <= 64;
    const bool many_tiles = narrow ? (long)cdiv(M, 256) >= 3 * cus / 4 : tall;
    // measured in steady state against the other kernels' best: ahead from a quarter of the CUs holding a tile (64 tiles:
    // 128x128x128 under 128 5x5 filters 36.3 -> 34.1 us; 98 tiles: 112x112x128 under 256 3x3 filters 17.4 -> 16.8 us),
    // behind at 26 tiles (56x56x256 under 256 filters, where the split over K wins)
    const bool taprow_tiles = (long)cdiv(M, 256) * (narrow ? 1 : cdiv(N, 128)) >= cus / 4;
    if (taprow_fits && ((taprow_tiles && (g_rt.hgemm_variant < 12 || g_rt.hgemm_variant > 13)) || g_rt.hgemm_variant == 14)) {
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
                               static_cast<float*>(nullptr), 0, (size_t)0);
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
                           static_cast<float*>(nullptr), 0, (size_t)0);
    };
    if (tall && tap_uniform) launch(hconv_tile_kernel<HconvTall, true>, HconvTall{});
    else if (tall) launch(hconv_tile_kernel<HconvTall, false>, HconvTall{});
    else if (tap_uniform) launch(hconv_tile_kernel<HconvSquare, true>, HconvSquare{});
    else launch(hconv_tile_kernel<HconvSquare, false>, HconvSquare{});
    HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace decx_hip
