// fp16 convolution (fp32 accumulate) with the operands moved global -> LDS by the gfx950 LDS-DMA loads: the kernel of
// hconv_tile.hpp (same lowering, same LDS layout, same fragment reads, same epilogue) without its trip through registers.
//
// For a channel pitch that is a multiple of the K step (64 halves) a K step lies inside one tap, and the image side of a
// step is, per pixel, 128 contiguous bytes -- eight 16-byte units.  buffer_load_dwordx4 ... lds moves one unit per lane
// straight into LDS (lane L of an instruction lands at M0 + 16 L; measured), takes its address as a 32-bit offset into a
// buffer resource and answers an offset outside the buffer with zeros, which it writes to LDS like any other data
// (measured): the same out-of-range trick that zero-fills the apron in the register-staged kernel.  The XOR swizzle of
// the LDS layout is applied on the global side: lane L of a 64-unit chunk (8 rows) fetches the unit whose slot is L.
// What this saves: the staging registers, the LDS store instructions (a 16-byte store of a wave holds the LDS pipe for
// 13 cycles; the 48 KB of a step took more of that pipe than the fragment reads), and all but three vector instructions
// per image load (add the tap's offset, test the column, select).
//
// Pipeline as in hgemm_dma_tile.hpp: STAGES LDS buffers, one barrier per K step placed inside the step's last block of
// MFMAs -- before it a wave waits until its own loads of step t+1 have landed, after it nobody reads step t's buffer any
// more and the loads of step t+STAGES go out, between the remaining MFMAs.  Every step refills its buffer, past the end
// of K with out-of-range offsets (zeros, no memory traffic), so the count of loads in flight is the same at every wait.
#pragma once
#include "hconv_tile.hpp"
#include "hgemm_dma_tile.hpp"

namespace decx_hip {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_>
struct HconvDmaShape {
    static constexpr int BM = BM_, BN = BN_, BK = 64, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = STAGES_;
    static constexpr int NWAVES = WAVES_M * WAVES_N, NT = NWAVES * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int U = BK / 8;                          // 16-byte units per row and K step
    static constexpr int A_UNITS = BM * U, B_UNITS = BN * U;
    static constexpr int A_LOADS = A_UNITS / 64 / NWAVES, B_LOADS = B_UNITS / 64 / NWAVES, LOADS = A_LOADS + B_LOADS;   // per wave and step
    static constexpr int STAGE_BYTES = (A_UNITS + B_UNITS) * 16;
    static constexpr int OUT_ROW = BN + 4;                    // as HconvShape
    static constexpr size_t OUT_BYTES = (size_t)BM * OUT_ROW * 2 + (size_t)BN * 4;
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_BYTES > OUT_BYTES ? (size_t)STAGES * STAGE_BYTES : OUT_BYTES;
    static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(A_UNITS % (64 * NWAVES) == 0 && B_UNITS % (64 * NWAVES) == 0, "chunks of 64 units must divide over the waves");
    static_assert(STAGES >= 2 && LOADS * (STAGES - 1) <= 63, "vmcnt is a 6-bit counter");
    static_assert(BN % 8 == 0 && (BM * (BN / 8)) % NT == 0, "the result tile leaves in whole 16-byte units");
};

template <class S>
__global__ __launch_bounds__(S::NT) void hconv_dma_kernel(HalfImage img, HalfFilters fb, HalfTensorOut out, int M, int N,
                                                          int Kw /* K in words, a multiple of 32 */, int tiles_n) {
    constexpr int BM = S::BM, BN = S::BN, U = S::U, MI = S::MI, NI = S::NI, STAGES = S::STAGES;
    static_assert(U == 8, "the swizzle below is written for 8 units per row");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw;

    const TileCoord tc = xcd_grouped_tile((int)blockIdx.x, (int)gridDim.x / tiles_n, tiles_n, 8);
    const int steps = Kw / (S::BK / 2);
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

    // ---- sources of this wave's loads.  Chunk c of an operand is rows 8c .. 8c+7; lane L moves, for row 8c + L/8, the
    // unit whose slot in the row is L%8 (slot = unit ^ ((row/2) % 8), a_unit_slot).
    const i32x4 img_rsrc = raw_buffer_words(img.src, img.bytes), filt_rsrc = raw_buffer_words(fb.filt, fb.bytes);
    int a_x[S::A_LOADS];
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int r = (wave * S::A_LOADS + j) * 8 + lane / 8;
        const int unit = (lane % 8) ^ ((r / 2) % 8);
        int m = bm0 + r;
        if (m >= M) m = M - 1;                                       // rows past the end are computed and never stored
        int y, x;
        pixel_of(m, y, x);
        a_x[j] = x - img.ox;
        a_off[j] = (uint32_t)(4 * ((y - img.oy) * img.row_stride_w + a_x[j] * img.dpitch_w) + 16 * unit);
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int r = (wave * S::B_LOADS + j) * 8 + lane / 8;
        const int unit = (lane % 8) ^ ((r / 2) % 8);
        int n = bn0 + r;
        if (n >= N) n = N - 1;
        b_off[j] = (uint32_t)(4 * n * fb.filt_stride_w + 16 * unit);
    }
    // the walk over (tap row, tap column, channel block): wave-uniform
    TapWalk wa, wb;
    wa.init(0, img.dpitch_w, img.kw, img.row_stride_w);
    wb.init(0, fb.dpitch_w, fb.kw, fb.row_stride_w);
    const TapStep sa = TapStep::make(S::BK / 2, img.dpitch_w, img.kw, img.row_stride_w);
    const TapStep sb = TapStep::make(S::BK / 2, fb.dpitch_w, fb.kw, fb.row_stride_w);
    int fetch_step = 0;                                        // the K step the next loads belong to

    // load number j (image loads first, then filters) of step fetch_step into LDS buffer `stage`.  Rows above and below the
    // image need no test: their offsets are negative or past the end of the tensor.
    auto issue_one = [&](int stage, int j) {
        const uint32_t base = lds_base + (uint32_t)stage * S::STAGE_BYTES;
        const bool live = fetch_step < steps;
        if (j < S::A_LOADS) {
            const bool inside = live && (unsigned)(a_x[j] + wa.kj) < (unsigned)img.W;
            dma_buffer_load16(img_rsrc, inside ? a_off[j] + (uint32_t)wa.off : kOutOfRange, 0u,
                              base + (uint32_t)(wave * S::A_LOADS + j) * 1024u);
        } else {
            const int jb = j - S::A_LOADS;
            dma_buffer_load16(filt_rsrc, live ? b_off[jb] : kOutOfRange, (uint32_t)wb.off,
                              base + (uint32_t)(S::A_UNITS * 16) + (uint32_t)(wave * S::B_LOADS + jb) * 1024u);
        }
        if (j == S::LOADS - 1) {
            wa.advance(sa, img.dpitch_w, img.kw);
            wb.advance(sb, fb.dpitch_w, fb.kw);
            ++fetch_step;
        }
    };

    // acc[mi][ni]: rows of the MFMA result are filters, columns are pixels (see hconv_tile.hpp)
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

#pragma unroll
    for (int s = 0; s < STAGES; ++s)
#pragma unroll
        for (int j = 0; j < S::LOADS; ++j) issue_one(s, j);

    // ---- fragment reads: per lane one swizzled byte offset per k-block, everything else is an immediate
    constexpr int KS = S::BK / 16, BLK = MI * NI, FRAG_READS = MI + NI;
    uint32_t frag_x[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) frag_x[ks] = (uint32_t)(((2 * ks + lh) ^ ((li / 2) % U)) * 16);
    const uint32_t a_frag_row = (uint32_t)((wm0 + li) * U * 16), b_frag_row = (uint32_t)(S::A_UNITS * 16 + (wn0 + li) * U * 16);
    struct Frags {
        f16x8 p[MI], f[NI];
    };
    auto read_one = [&](Frags& fr, int stage, int ks, int r) {
        const unsigned char* buf = lds_raw + (size_t)stage * S::STAGE_BYTES;
        if (r < MI) fr.p[r] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(buf + a_frag_row + r * (32 * U * 16) + frag_x[ks]));
        else fr.f[r - MI] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(buf + b_frag_row + (r - MI) * (32 * U * 16) + frag_x[ks]));
    };
    auto mfma_one = [&](const Frags& fr, int i) {
        const int mi = i / NI, ni = i % NI;
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr.f[ni], fr.p[mi], acc[mi][ni], 0, 0, 0);
    };
#define DECX_PIN() __builtin_amdgcn_sched_barrier(0)
    Frags f0, f1;
    static_assert(KS % 2 == 0, "fragment sets must line up across K steps (block 0 always in f0)");

    // One K step.  f0 holds the fragments of its first k-block on entry and those of the next step's first k-block on exit.
    auto k_step = [&](int stg, int next, bool has_next) {
#pragma unroll
        for (int b = 0; b + 1 < KS; ++b) {
#pragma unroll
            for (int i = 0; i < BLK; ++i) {
                constexpr int RPS = (FRAG_READS + BLK - 1) / BLK;
#pragma unroll
                for (int r = i * RPS; r < (i + 1) * RPS && r < FRAG_READS; ++r) read_one((b & 1) ? f0 : f1, stg, b + 1, r);
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
        // my loads of step t+1 have landed (those of t+2 .. t+STAGES-1 may still fly), my reads of this buffer are done
        wait_dma_then_barrier<S::LOADS*(STAGES - 2)>();
        DECX_PIN();
        constexpr int SLOTS = BLK - PRE;
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
#pragma unroll
            for (int j = (i * S::LOADS) / SLOTS; j < ((i + 1) * S::LOADS) / SLOTS; ++j) issue_one(stg, j);
            if (has_next) {
#pragma unroll
                for (int r = (i * FRAG_READS) / SLOTS; r < ((i + 1) * FRAG_READS) / SLOTS; ++r) read_one(fn, next, 0, r);
            }
            mfma_one(fl, PRE + i);
            DECX_PIN();
        }
    };

    wait_dma_then_barrier<S::LOADS*(STAGES - 1)>();            // step 0 has landed
#pragma unroll
    for (int r = 0; r < FRAG_READS; ++r) read_one(f0, 0, 0, r);
    DECX_PIN();
    // unrolled over the LDS buffers: the buffer of a step is then a compile-time constant and folds into the offset fields
    // of its fragment reads
    for (int t0 = 0; t0 < steps; t0 += STAGES)
        static_for<0, STAGES>([&](auto d) {
            constexpr int STG = decltype(d)::value;
            if (t0 + STG < steps) k_step(STG, (STG + 1) % STAGES, t0 + STG + 1 < steps);
        });
#undef DECX_PIN
    // the loads past the end of K still write (zeros) when they land: wait for them before LDS becomes the result tile
    wait_dma_then_barrier<0>();
    hconv_store_tile<S>(acc, lds_raw, out, M, N, bm0, bn0, wm0, wn0, tid, pixel_of);
}

}  // namespace decx_hip
