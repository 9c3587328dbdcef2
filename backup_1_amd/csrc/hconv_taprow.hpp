// fp16 convolution (fp32 accumulate), LDS-DMA fed like hconv_dma.hpp, that loads the pixels of a tap ROW once for all
// of its kw taps.
//
// The taps (ki, 0) .. (ki, kw-1) of a block of 64 channels read the same pixels, one position apart: tap kj of output
// pixel (y, x) is input pixel (y + ki - oy, x + kj - ox).  So per (ki, channel block) -- a "row step" -- the kernel puts a
// PATCH of input pixels into LDS once, one 128-byte row per pixel, and the kw K steps of that row step read their pixel
// fragments from it with the row index shifted by kj.  The filters still arrive per K step.  Per three K steps of a 3x3
// convolution that is 40 + 3 x 16 KB instead of 3 x 48 KB.
//
// Patch rows.  Image rows are laid end to end with kw - 1 rows of zeros between them (Wp = W + 2 ox positions per image
// row; without zero compensation ox = 0 and an output row is simply shorter than an input row): output pixel (y, x) of a
// tile whose first pixel is (y0, x0) reads patch row  q + kj,  q = (y - y0) Wp + x - x0,  for every tap of the row step,
// and what it finds at a position outside the image's columns is the zeros that the loads put there (out-of-range
// buffer offsets, which the hardware answers with zeros; rows above and below the image fall out of the buffer by
// themselves).  q is a per-lane constant for the whole K walk; so are the swizzled addresses q + kj gives.  A tile of 256
// pixels spans 255 + kw + 2 (rows it touches) positions: the patch has 320 rows, the host checks that this is enough.
//
// K is walked in the order (ki, channel block, kj) -- not the order of the other kernels, which for binary16 results
// (no reference bits to match, fp32 accumulation, one rounding) changes nothing but the last bit of a sum.
//
// Pipeline: two patch buffers (80 KB) and a ring of four filter buffers (64 KB).  Step t = kw s + j (row step s, tap j)
// computes from patch s % 2 and filter buffer t % 4; its barrier sits inside its last block of MFMAs, after it the filter
// loads of step t + 4 go out and, when j = kw - 1, the patch loads of row step s + 2.  Loads past the end ask for
// out-of-range offsets, so the number of loads in flight at each wait only depends on j:
//   program order of a wave's loads ... B(t+1) | B(t+2) | A(s+1) B(t+3) ...   with A(s+1) issued after the last tap of row step s-1
//   j = 0: B(t+1), B(t+2), A(s+1), B(t+3)      need B(t+1)          -> at most 2 + 5 + 2 younger loads outstanding
//   j = 1: B(t+1), A(s+1), B(t+2), B(t+3)      need B(t+1)          -> 5 + 2 + 2
//   j > 1: A(s+1) .. B(t+1), B(t+2), B(t+3)    need B(t+1), and A(s+1) after the last tap -> 2 + 2
// (kw = 3, 5 and 7 are built; the patch, the tap and the filter buffer of a step repeat with period 4 kw.)
#pragma once
#include "hconv_dma.hpp"

namespace decx_hip {

template <int KW_, int BN_ = 128, int WAVES_M_ = 4, int WAVES_N_ = 2>
struct HconvTapRowShape {
    static constexpr int BM = 256, BN = BN_, BK = 64, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KW = KW_;
    static_assert(KW >= 3 && KW % 2 == 1, "the wait counts of the kernel are derived for odd widths from 3 on");
    static constexpr int NWAVES = WAVES_M * WAVES_N, NT = NWAVES * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int U = 8;
    static constexpr int PATCH_ROWS = 320;                     // >= 255 + KW + 2 * (image rows a tile touches)
    static constexpr int A_BYTES = PATCH_ROWS * 128, B_BYTES = BN * 128;
    static constexpr int A_LOADS = PATCH_ROWS / 8 / NWAVES, B_LOADS = BN / 8 / NWAVES;   // per wave: 5 per row step, 2 per K step
    static constexpr int A_BUFFERS = 2, B_BUFFERS = 4;
    static constexpr int OUT_ROW = BN + 4;
    static constexpr size_t OUT_BYTES = (size_t)BM * OUT_ROW * 2 + (size_t)BN * 4;
    static constexpr size_t LDS_BYTES = (size_t)A_BUFFERS * A_BYTES + (size_t)B_BUFFERS * B_BYTES;
    static_assert(PATCH_ROWS % (8 * NWAVES) == 0 && BN % (8 * NWAVES) == 0, "chunks of 8 rows must divide over the waves");
    static_assert(LDS_BYTES >= OUT_BYTES, "the result tile reuses the operand buffers");
    static_assert(NWAVES == 8, "256 threads would leave a SIMD with one wave and nothing to overlap its waits with");
};

template <class S>
__global__ __launch_bounds__(S::NT) void hconv_taprow_kernel(HalfImage img, HalfFilters fb, HalfTensorOut out, int M, int N,
                                                             int tiles_n) {
    constexpr int BM = S::BM, BN = S::BN, MI = S::MI, NI = S::NI, KW = S::KW;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw;
    constexpr int B_BASE = S::A_BUFFERS * S::A_BYTES;          // the filter ring starts behind the patches

    const TileCoord tc = xcd_grouped_tile((int)blockIdx.x, (int)gridDim.x / tiles_n, tiles_n, 8);
    const int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;
    const bool small_m = M < (1 << 22);
    const float rcp_wout = 1.0f / (float)img.Wout;
    auto pixel_of = [&](int m, int& y, int& x) {
        if (small_m) small_divmod(m, img.Wout, rcp_wout, y, x);
        else { y = m / img.Wout; x = m - y * img.Wout; }
    };
    const int channel_blocks = img.dpitch_w / 32;              // K steps per tap
    const int row_steps = img.kh * channel_blocks, steps = row_steps * KW;
    const int Wp = img.W + 2 * img.ox;

    // the tile's first and last pixel: where the patch starts, and how many of its rows are ever read
    int y0, x0, y_last, x_last;
    pixel_of(bm0, y0, x0);
    pixel_of(bm0 + BM - 1 < M ? bm0 + BM - 1 : M - 1, y_last, x_last);
    y0 = __builtin_amdgcn_readfirstlane(y0);
    x0 = __builtin_amdgcn_readfirstlane(x0);
    const int extent = __builtin_amdgcn_readfirstlane((y_last - y0) * Wp + x_last - x0 + KW);

    // ---- sources of this wave's loads.  Chunk c of a buffer is rows 8c .. 8c+7; lane L moves, for row 8c + L/8, the unit
    // whose slot in the row is L%8 (slot = unit ^ ((row/2) % 8)).  Patch row r holds position p = r + x0 of the image
    // rows laid end to end from row y0 - oy (+ ki): image row p / Wp, column p % Wp - ox.
    const i32x4 img_rsrc = raw_buffer_words(img.src, img.bytes), filt_rsrc = raw_buffer_words(fb.filt, fb.bytes);
    const float rcp_wp = 1.0f / (float)Wp;
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int r = (wave * S::A_LOADS + j) * 8 + lane / 8;
        const int unit = (lane % 8) ^ ((r / 2) % 8);
        int yy, xp;
        small_divmod(r + x0, Wp, rcp_wp, yy, xp);               // r + x0 < 320 + W
        const int xx = xp - img.ox;
        const bool wanted = r < extent && (unsigned)xx < (unsigned)img.W;
        a_off[j] = wanted ? (uint32_t)(4 * ((y0 - img.oy + yy) * img.row_stride_w + xx * img.dpitch_w) + 16 * unit) : kOutOfRange;
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int r = (wave * S::B_LOADS + j) * 8 + lane / 8;
        const int unit = (lane % 8) ^ ((r / 2) % 8);
        int n = bn0 + r;
        if (n >= N) n = N - 1;
        b_off[j] = (uint32_t)(4 * n * fb.filt_stride_w + 16 * unit);
    }
    // what to fetch next: the row step of the next patch, the K step of the next filter slice (all wave-uniform)
    int fa_s = 0, fa_ki = 0, fa_cb = 0;
    int fb_t = 0, fb_ki = 0, fb_cb = 0, fb_kj = 0;
    auto issue_patch_load = [&](int buffer, int j) {
        // an out-of-range a_off stays out of range: the step offset is far below 2^31
        const uint32_t step_off = (uint32_t)(4 * (fa_ki * img.row_stride_w + fa_cb * 32));
        dma_buffer_load16(img_rsrc, fa_s < row_steps ? a_off[j] + step_off : kOutOfRange, 0u,
                          lds_base + (uint32_t)buffer * S::A_BYTES + (uint32_t)(wave * S::A_LOADS + j) * 1024u);
        if (j == S::A_LOADS - 1) {
            ++fa_s;
            if (++fa_cb == channel_blocks) { fa_cb = 0; ++fa_ki; }
        }
    };
    auto issue_filter_load = [&](int buffer, int j) {
        const uint32_t step_off = (uint32_t)(4 * (fb_ki * fb.row_stride_w + fb_kj * fb.dpitch_w + fb_cb * 32));
        dma_buffer_load16(filt_rsrc, fb_t < steps ? b_off[j] : kOutOfRange, step_off,
                          lds_base + (uint32_t)B_BASE + (uint32_t)buffer * S::B_BYTES + (uint32_t)(wave * S::B_LOADS + j) * 1024u);
        if (j == S::B_LOADS - 1) {
            ++fb_t;
            if (++fb_kj == KW) {
                fb_kj = 0;
                if (++fb_cb == channel_blocks) { fb_cb = 0; ++fb_ki; }
            }
        }
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    // prologue, in the order the waits below count on: A(0) B(0) | B(1) B(2) A(1) B(3)
    static_for<0, S::A_LOADS>([&](auto j) { issue_patch_load(0, decltype(j)::value); });
    static_for<0, S::B_LOADS>([&](auto j) { issue_filter_load(0, decltype(j)::value); });
    static_for<0, S::B_LOADS>([&](auto j) { issue_filter_load(1, decltype(j)::value); });
    static_for<0, S::B_LOADS>([&](auto j) { issue_filter_load(2, decltype(j)::value); });
    static_for<0, S::A_LOADS>([&](auto j) { issue_patch_load(1, decltype(j)::value); });
    static_for<0, S::B_LOADS>([&](auto j) { issue_filter_load(3, decltype(j)::value); });

    // ---- fragment reads.  Pixel fragments: per lane, block mi and tap kj a patch row, and per k-block of the step its
    // swizzled unit -- 24 loop-invariant byte offsets.  Filter fragments as in hconv_dma.hpp.
    constexpr int KS = S::BK / 16, BLK = MI * NI, FRAG_READS = MI + NI;
    uint32_t pix_frag[MI][KW][KS], filt_frag[KS];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi) {
        int m = bm0 + wm0 + mi * 32 + li;
        if (m >= M) m = M - 1;                                       // computed, never stored
        int y, x;
        pixel_of(m, y, x);
        const int q = (y - y0) * Wp + x - x0;
#pragma unroll
        for (int kj = 0; kj < KW; ++kj)
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                pix_frag[mi][kj][ks] = (uint32_t)((q + kj) * 128 + ((2 * ks + lh) ^ (((q + kj) / 2) % 8)) * 16);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        filt_frag[ks] = (uint32_t)(B_BASE + (wn0 + li) * 128 + ((2 * ks + lh) ^ ((li / 2) % 8)) * 16);
    struct Frags {
        f16x8 p[MI], f[NI];
    };
    // read r of k-block ks of a step that uses patch buffer A_BUF with tap KJ and filter buffer B_BUF
    auto read_one = [&](Frags& fr, auto a_buf, auto kj, auto b_buf, int ks, int r) {
        constexpr int A_BUF = decltype(a_buf)::value, KJ = decltype(kj)::value, B_BUF = decltype(b_buf)::value;
        if (r < MI) fr.p[r] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(lds_raw + A_BUF * S::A_BYTES + pix_frag[r][KJ][ks]));
        else fr.f[r - MI] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(lds_raw + B_BUF * S::B_BYTES + (r - MI) * (32 * 128) + filt_frag[ks]));
    };
    auto mfma_one = [&](const Frags& fr, int i) {
        const int mi = i / NI, ni = i % NI;
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr.f[ni], fr.p[mi], acc[mi][ni], 0, 0, 0);
    };
#define DECX_PIN() __builtin_amdgcn_sched_barrier(0)
    Frags f0, f1;
    static_assert(KS % 2 == 0, "fragment sets must line up across K steps (block 0 always in f0)");

    // Step I of a run of 4 kw (patch buffer, tap and filter buffer repeat with that period).  f0 holds the fragments of its first
    // k-block on entry and those of the next step's first k-block on exit.
    auto k_step = [&](auto step_tag, bool has_next) {
        constexpr int I = decltype(step_tag)::value, J = I % KW;
        typedef std::integral_constant<int, (I / KW) % 2> ABuf;
        typedef std::integral_constant<int, J> Tap;
        typedef std::integral_constant<int, I % 4> BBuf;
        typedef std::integral_constant<int, ((I + 1) / KW) % 2> NextABuf;
        typedef std::integral_constant<int, (I + 1) % KW> NextTap;
        typedef std::integral_constant<int, (I + 1) % 4> NextBBuf;
        // k-blocks 0 .. KS-2: MFMA i of block b rides with the reads of block b+1 (fragment sets alternate f0, f1)
        constexpr int RPS = (FRAG_READS + BLK - 1) / BLK;      // reads per MFMA slot, front-loaded
#pragma unroll
        for (int b = 0; b + 1 < KS; ++b) {
#pragma unroll
            for (int i = 0; i < BLK; ++i) {
#pragma unroll
                for (int r = i * RPS; r < (i + 1) * RPS && r < FRAG_READS; ++r) read_one((b & 1) ? f0 : f1, ABuf{}, Tap{}, BBuf{}, b + 1, r);
                mfma_one((b & 1) ? f1 : f0, i);
                DECX_PIN();
            }
        }
        Frags& fl = ((KS - 1) & 1) ? f1 : f0;
        Frags& fn = ((KS - 1) & 1) ? f0 : f1;
        constexpr int PRE = BLK / 4 > 0 ? BLK / 4 : 1;
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            mfma_one(fl, i);
            DECX_PIN();
        }
        // what the next step reads has landed (see the table at the top), my reads of this step's buffers are done
        wait_dma_then_barrier<(J >= 2 ? 2 * S::B_LOADS : S::A_LOADS + 2 * S::B_LOADS)>();
        DECX_PIN();
        // between the MFMAs that are left: the refills -- the patch of row step s + 2 after the last tap, then the filters
        // of step t + 4, in this order -- and the next step's first fragments
        constexpr int SLOTS = BLK - PRE, REFILLS = (J == KW - 1 ? S::A_LOADS : 0) + S::B_LOADS;
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
#pragma unroll
            for (int l = (i * REFILLS) / SLOTS; l < ((i + 1) * REFILLS) / SLOTS; ++l) {
                if (l < REFILLS - S::B_LOADS) issue_patch_load(ABuf::value, l);
                else issue_filter_load(BBuf::value, l - (REFILLS - S::B_LOADS));
            }
            if (has_next) {
#pragma unroll
                for (int r = (i * FRAG_READS) / SLOTS; r < ((i + 1) * FRAG_READS) / SLOTS; ++r) read_one(fn, NextABuf{}, NextTap{}, NextBBuf{}, 0, r);
            }
            mfma_one(fl, PRE + i);
            DECX_PIN();
        }
    };
    static_assert(BLK >= 2, "the barrier sits between two MFMAs of the last k-block");

    // A(0) and B(0) have landed: everything younger (B(1), B(2), A(1), B(3)) may still fly
    wait_dma_then_barrier<S::A_LOADS + 3 * S::B_LOADS>();
    {
        typedef std::integral_constant<int, 0> Z;
        static_for<0, FRAG_READS>([&](auto r) { read_one(f0, Z{}, Z{}, Z{}, 0, decltype(r)::value); });
    }
    DECX_PIN();
    for (int t0 = 0; t0 < steps; t0 += 4 * KW)
        static_for<0, 4 * KW>([&](auto i) {
            if (t0 + decltype(i)::value < steps) k_step(i, t0 + decltype(i)::value + 1 < steps);
        });
#undef DECX_PIN
    // the loads past the end of K still write (zeros) when they land: wait for them before LDS becomes the result tile
    wait_dma_then_barrier<0>();
    hconv_store_tile<S>(acc, lds_raw, out, M, N, bm0, bn0, wm0, wn0, tid, pixel_of);
}

}  // namespace decx_hip
