// fp32 fused im2col convolution: argument checks, loader and kernel choice, launch (sgemm_tile.hpp, conv_chain16.hpp).
#include "sgemm_launch.hpp"
#include "sgemm_chain16.hpp"
#include "conv_chain16.hpp"

namespace decx_hip {

// One translation unit per loader build instantiates the tile kernels for it (sgemm_conv_uniform.hip,
// sgemm_conv_paired.hip, sgemm_conv_plain.hip): they compile side by side.
int conv_dispatch_uniform(int variant, const Im2colAUniform& a, const FilterBUniform& b, const float* bias, float* dst,
                          const TensorOut& out, int M, int N, int K, const Batch& batch);
int conv_dispatch_paired(int variant, const Im2colA<true>& a, const FilterB<true>& b, const float* bias, float* dst,
                         const TensorOut& out, int M, int N, int K, const Batch& batch);
int conv_dispatch_plain(int variant, const Im2colA<false>& a, const FilterB<false>& b, const float* bias, float* dst,
                        const TensorOut& out, int M, int N, int K, const Batch& batch);

// the convolution on LDS-DMA loads and 16x16 blocks (sconv_dma.hpp), instantiated in sconv_dma.hip
int launch_sconv_dma_shape(int shape, const Im2colA<true>& img, const FilterB<true>& fb, const float* bias, float* dst,
                           const TensorOut& out, int M, int N, int K);
// the convolution of small images on tiles of 32 x 32 fed by LDS-DMA loads (sconv_small.hpp), instantiated in sconv_small.hip
int launch_sconv_small_shape(const Im2colA<true>& img, const FilterB<true>& fb, const float* bias, float* dst, const TensorOut& out,
                             int M, int N, int K);

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

namespace {
// see conv_enqueue: image rows of the first of two launches, on the 256x256 tile (shape 7, one workgroup per CU), or
// rows = 0 for one launch.  Only where one launch would take one of the big tiles, whose rounds the model counts right
// (the 128x128 tile runs several workgroups per CU and does not come in rounds: measured, its products lose 1 - 2 %
// when split); first launches on the 256x128 and 224x128 tiles lost 3 - 10 % on four shapes of five and are not planned.
struct ConvRowsSplit {
    int rows = 0, shape = 0;
};
ConvRowsSplit plan_conv_rows_split(int Hout, int Wout, int N, int K) {
    ConvRowsSplit plan;
    const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
    const long M = (long)Hout * Wout;
    if (K < 512 || M > 0x7fffffffL) return plan;
    double whole_cost = 0.0;
    const int whole_shape = pick_sgemm_variant((int)M, N, K, 1, false, &whole_cost);
    if (whole_cost == 0.0 || !(whole_shape == 7 || whole_shape == 10 || (whole_shape >= 3 && whole_shape <= 5) || whole_shape == 15)) return plan;
    const long tiles_m = cdiv((int)M, 256), tiles_n = cdiv(N, 256), whole = tiles_m * tiles_n / cus;
    if (whole < 1 || tiles_m * tiles_n % cus == 0) return plan;
    const long rows = whole * cus / tiles_n * 256 / Wout;          // image rows whose tiles fit the whole rounds
    if (rows < 1 || rows >= Hout) return plan;
    double rest = 0.0;
    (void)pick_sgemm_variant((int)((Hout - rows) * Wout), N, K, 1, false, &rest);
    if (rest == 0.0) return plan;
    if ((double)whole * 65536.0 + rest + 4.0 * 614.5e3 / (2.0 * K) < 0.96 * whole_cost) plan.rows = (int)rows, plan.shape = 7;
    return plan;
}
}  // namespace

int conv_enqueue(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt, int N, int kh,
                 int kw, size_t filt_stride, size_t filt_row_stride, float* dst, int dst_dpitch, size_t dst_row_stride,
                 int flag, const float* bias, bool relu) {
    if (!g_rt.is_init) return need_init();
    const bool small_kept_out = g_rt.sgemm_variant == 33, one_launch = g_rt.sgemm_variant == 34;
    const ShapeForThisCall shape_for_this_call(small_kept_out || g_rt.sgemm_variant == 34 ? 0 : g_rt.sgemm_variant);
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
    // (its 64x64 shape walks a convolution 14 % slower than a dense product of the same size -- the moving waves do the
    // im2col addressing -- so once 128x64 tiles cover three quarters of the CUs the tiles are ahead: 112x112x128 under 128
    // filters 57.1 -> 50.6 us)
    // Small images with a channel pitch in 32s (a K step inside one tap): tiles of 32 pixels x 32 filters on 16x16 blocks fed
    // by LDS-DMA loads (sconv_small.hpp; forced by shape 31).  Taken where a measured model of its time is below that of
    // the kernel the rest of this function would take (microseconds; fitted on 48 layer shapes from 7x7x512 to
    // 1024x1024x32, on which the choice is within 2 % of the better kernel everywhere): every SIMD walks K once per
    // 16x16 block it owns, at 8 cycles per k and 72 % of the matrix pipe's pace, after 4 us of launch, first loads and
    // stores; the patch kernel's single round takes 7 us + 2.93 us per 32 k; the register-staged tiles 8 us + their
    // tile cost at the matrix peak of one CU.
    if (!small_kept_out && (g_rt.sgemm_variant == 0 || g_rt.sgemm_variant == 31) && dpitch % 32 == 0 &&
        conv_patch_offsets_fit(src_bytes, src_row_stride, (size_t)dpitch, kh, kw, oy, ox, sizeof(float))) {
        bool take = g_rt.sgemm_variant == 31;
        if (!take) {
            const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
            const double blocks = 4.0 * (double)cdiv(Hout, 8) * cdiv(Wout, 4) * cdiv(N, 32);
            const double rounds = blocks / (4.0 * cus) > 1.0 ? blocks / (4.0 * cus) : 1.0;
            const double t_small = 4.0 + rounds * K * 8.0 / 2400.0 / 0.72;
            const long patches = (long)cdiv(Hout, 16) * cdiv(Wout, 13) * cdiv(N, 128);
            const bool patch_kernel = N % 4 == 0 && aligned16(dst) && dst_dpitch % 4 == 0 && dst_row_stride % 4 == 0 &&
                                      patches <= cus && 4 * patches >= 3 * cus;
            double tile_cost = 0.0;
            (void)pick_sgemm_variant(M, N, K, 1, false, &tile_cost);
            // (the tile model is optimistic where its tiles come in at most two rounds -- they do not fill the chip and
            // their prologue and epilogue lie open: there it counts for a tenth more)
            const bool few_rounds = (long)cdiv(M, 128) * cdiv(N, 128) <= 2 * cus;
            const double t_other = patch_kernel ? 7.0 + K / 32 * 2.93 : (8.0 + tile_cost * K * 2.0 / 614.5e3) * (few_rounds ? 1.0 / 0.9 : 1.0);
            take = t_small < t_other;
        }
        if (take) {
            Im2colA<true> a{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes};
            FilterB<true> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
            return launch_sconv_small_shape(a, b, bias, dst, out, M, N, K);
        }
    }
    int chain = pick_chain_shape(M, N, K, 1);
    if (chain == 13 && g_rt.sgemm_variant == 0 && (long)cdiv(M, 128) * cdiv(N, 64) >= 3 * (g_rt.compute_units > 0 ? g_rt.compute_units : 256) / 4)
        chain = 0;
    if (chain) {
        Im2colA<false> a{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes};
        FilterB<false> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
        if (chain == 11) return launch_conv_chain16<Chain16<2, 1, 4, 4>>(a, b, bias, dst, out, M, N, K);
        if (chain == 12) return launch_conv_chain16<Chain16<1, 1, 8, 2>>(a, b, bias, dst, out, M, N, K);
        if (chain == 23) return launch_conv_chain16<Chain16Rect<1, 2, 1, 6, 2>>(a, b, bias, dst, out, M, N, K);
        return launch_conv_chain16<Chain16<4, 2, 2, 3>>(a, b, bias, dst, out, M, N, K);
    }
    // a K step of 32 inside one tap, results leaving as 16-byte units: the LDS-DMA kernel on 16x16 blocks.  Its column
    // test adds 2^31 to an offset, which must throw it out of the tensor's range even from the apron's negative offsets,
    // and its patches reach up to 15 rows and 12 columns past the output: those offsets must stay below 2^31 as well.
    // Forced by shapes 29 and 30; by itself it takes a result that its patches of 16 x 13 pixels x 128 filters cover in
    // one round that fills at least three quarters of the CUs
    if (dpitch % 32 == 0 && N % 4 == 0 && aligned16(dst) && dst_dpitch % 4 == 0 && dst_row_stride % 4 == 0 &&
        conv_patch_offsets_fit(src_bytes, src_row_stride, (size_t)dpitch, kh, kw, oy, ox, sizeof(float))) {
        const long cus = g_rt.compute_units > 0 ? g_rt.compute_units : 256;
        const long patches = (long)cdiv(Hout, 16) * cdiv(Wout, 13) * cdiv(N, 128);
        int shape = g_rt.sgemm_variant >= 29 && g_rt.sgemm_variant <= 30 ? g_rt.sgemm_variant : 0;
        if (g_rt.sgemm_variant == 0 && patches <= cus && 4 * patches >= 3 * cus) shape = 29;
        if (shape) {
            Im2colA<true> a{src, H, W, dpitch, kh, kw, oy, ox, Wout, M, K, (int)src_row_stride, (unsigned)src_bytes};
            FilterB<true> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
            return launch_sconv_dma_shape(shape, a, b, bias, dst, out, M, N, K);
        }
    }
    // The register-staged tiles, on output rows row0 .. row0 + rows - 1: the loaders place output pixel m of the part at
    // image row m / Wout - (oy - row0), so a part further down is the same launch with oy moved and dst advanced.
    auto tiles_on_rows = [&](int shape, int row0, int rows) -> int {
        const int part_m = rows * Wout, part_oy = oy - row0;
        float* part_dst = dst + (size_t)row0 * dst_row_stride;
        if (dpitch % 16 == 0) {      // a whole K step inside one tap: the tap walk runs on the scalar unit
            Im2colAUniform a{{src, H, W, dpitch, kh, kw, part_oy, ox, Wout, part_m, K, (int)src_row_stride, (unsigned)src_bytes}};
            FilterBUniform b{{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes}};
            return conv_dispatch_uniform(shape, a, b, bias, part_dst, out, part_m, N, K, one);
        }
        if (dpitch % 8 == 0) {       // the 8 consecutive k of a staging task never straddle a tap
            Im2colA<true> a{src, H, W, dpitch, kh, kw, part_oy, ox, Wout, part_m, K, (int)src_row_stride, (unsigned)src_bytes};
            FilterB<true> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
            return conv_dispatch_paired(shape, a, b, bias, part_dst, out, part_m, N, K, one);
        }
        Im2colA<false> a{src, H, W, dpitch, kh, kw, part_oy, ox, Wout, part_m, K, (int)src_row_stride, (unsigned)src_bytes};
        FilterB<false> b{filt, N, K, dpitch, kw, (int)filt_stride, (int)filt_row_stride, (unsigned)filt_bytes};
        return conv_dispatch_plain(shape, a, b, bias, part_dst, out, part_m, N, K, one);
    };
    // Tiles that come in whole rounds plus a part of one (a round = one tile per CU) pay a whole round for the part.
    // Every output element is the same chain of products whatever tile computes it, so the image rows that fill whole
    // rounds of the 256x256 tile go to one launch and the rows below to a second one on the tile that is cheapest for
    // them: taken where that costs under 96 % of the one launch, in the tile model's unit, 4 us for the second launch
    // included (300x300x128 under 256 filters: 418 -> 383 us, 348x348x256 under 512: 2061 -> 1944).  Shape 34 keeps
    // every convolution in one launch.
    if (g_rt.sgemm_variant == 0 && !one_launch) {
        const ConvRowsSplit split = plan_conv_rows_split(Hout, Wout, N, K);
        if (split.rows > 0) {
            if (int rc = tiles_on_rows(split.shape, 0, split.rows)) return rc;
            return tiles_on_rows(pick_sgemm_variant((Hout - split.rows) * Wout, N, K, 1), split.rows, Hout - split.rows);
        }
    }
    return tiles_on_rows(variant, 0, Hout);
}

// host-only: the two-launch plan above for an output of Hout x Wout pixels under N filters (decx_hip_conv_plan_split)
int conv_plan_split(int Hout, int Wout, int N, int K, int* shape) {
    const ConvRowsSplit split = g_rt.sgemm_variant == 0 ? plan_conv_rows_split(Hout, Wout, N, K) : ConvRowsSplit();
    if (shape) *shape = split.shape;
    return split.rows;
}

}  // namespace decx_hip
