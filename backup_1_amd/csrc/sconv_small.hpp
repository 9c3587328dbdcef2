// fp32 fused im2col convolution for SMALL images (CNN layers of 7x7 .. 112x112 pixels): tiles of 32x32 or 64x64 on 16x16
// blocks (v_mfma_f32_16x16x4_f32), both operands moved global -> LDS by the gfx950 LDS-DMA loads.
//
// The lowered product of a small image has few outputs and a long K (56x56x256 under 256 filters: 3136 x 256 outputs,
// K = 2304), the class for which the dense kernel runs its tiles of 16x16 blocks (sgemm_dma_tile.hpp: four waves, one
// per SIMD, a wave's blocks chained over K, nothing on the computing waves but matrix instructions and their operand
// reads).  This kernel is that K walk -- STAGES LDS buffers, one barrier per K step, the step computed in two halves from
// two fragment sets, the refill of a buffer and the first fragments of the next step between the matrix instructions of
// the second half -- with the operand sources of the patch convolution (sconv_dma.hpp):
//   * a tile's rows are a PATCH of 8 output rows x BM / 8 columns, column by column: row 8 bx + yy of the lowered
//     product is pixel (y0 + yy, x0 + bx).  A K step lies inside one tap (channel pitch a multiple of the step), and per
//     pixel it is BK contiguous floats of the image: a row of A as in the dense kernel.  A load instruction moves 64
//     16-byte units = 8 rows (steps of 32 k) or 4 rows (steps of 64 k), pixels of ONE image column: whether its tap lies
//     left or right of the image is the same for all lanes, so the scalar unit decides it and adds 2^31 to the load's
//     offset, which throws every lane out of the buffer's range (buffer_load_dwordx4 ... lds answers such an offset with
//     zeros, written to LDS like data); image rows above and below the tensor fall out of range by themselves.
//   * the filter bank holds filter n's taps channel-innermost: its side of a K step is BK contiguous floats per filter,
//     B^T in the layout of A.  Both fragments are ds_read_b32: lane (i, s) takes float s of unit j of row i of its block
//     for the matrix instruction that covers k = 4j .. 4j+3 (unit j of row r in slot j ^ (r % 8) of the row).
//   * the tap walk runs on the scalar unit; an image load costs the vector unit one addition per step.
// Arithmetic: per output one fused multiply-add chain over ascending k = (ki kw + kj) dpitch + c, as every fp32 path
// (conv2_mk_im2col.h:167-274, eq_GEMM.cuh:109-209); bias and ReLU join the finished sum.
// Needs a channel pitch that is a multiple of BK, 16-byte aligned tensors below 2 GiB less the patch's reach
// (conv_patch_offsets_fit), like sconv_dma_kernel.
#pragma once
#include "sconv_dma.hpp"

namespace decx_hip {

template <int MI_, int NI_, int BK_, int STAGES_>
struct SconvSmallShape {
    static constexpr int MI = MI_, NI = NI_, BK = BK_, STAGES = STAGES_;
    static constexpr int WAVES_M = 2, WAVES_N = 2, NWAVES = 4, NT = 64 * NWAVES;
    static constexpr int WM = 16 * MI, WN = 16 * NI, BM = WM * WAVES_M, BN = WN * WAVES_N;
    static constexpr int PY = 8, PX = BM / PY;                          // the patch: PY output rows x PX columns
    static constexpr int UA = BK / 4, ROWS_PER_LOAD = 64 / UA;          // 16-byte units per row and step; rows a load moves
    static constexpr int A_LOADS = BM * UA / 64 / NWAVES, B_LOADS = BN * UA / 64 / NWAVES, LOADS = A_LOADS + B_LOADS;
    static constexpr int A_BYTES = BM * UA * 16, B_BYTES = BN * UA * 16, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_BYTES;
    static constexpr int HALF = BK / 4 / 2;                             // k-groups (matrix instructions per block) in half a step
    static constexpr int MFMAS = HALF * MI * NI, READS = HALF * (MI + NI);              // per half step and wave
    static_assert((BK == 32 || BK == 64) && PY % ROWS_PER_LOAD == 0, "a load's rows are pixels of one image column");
    static_assert(BM * UA % (64 * NWAVES) == 0 && BN * UA % (64 * NWAVES) == 0, "loads divide over the waves");
    static_assert(STAGES >= 2 && LOADS * (STAGES - 1) <= 63, "vmcnt is a 6-bit counter");
    static_assert(LOADS <= MFMAS - 1, "the loads go out behind the matrix instructions of half a step");
};

template <class S>
__global__ __launch_bounds__(S::NT) void sconv_small_kernel(Im2colA<true> img, FilterB<true> fb, const float* __restrict__ bias,
                                                            float* __restrict__ dst, TensorOut out, int Hout, int N, int K,
                                                            int tiles_x, int tiles_m, int tiles_n) {
    constexpr int MI = S::MI, NI = S::NI, UA = S::UA, STAGES = S::STAGES, HALF = S::HALF, MFMAS = S::MFMAS, READS = S::READS;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];   // [STAGES][A: BM rows x UA units | B: BN rows x UA units]
    const uint32_t lds_base = lds_byte_address(lds_raw);

    const TileCoord tc = xcd_grouped_tile((int)blockIdx.x, tiles_m, tiles_n, 8);
    const int tile_y = tc.tm / tiles_x, tile_x = tc.tm - tile_y * tiles_x;
    const int y0 = S::PY * tile_y, x0 = S::PX * tile_x, bn0 = tc.tn * S::BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane % 16, ls = lane / 16;
    const int steps = K / S::BK;

    // ---- sources of this wave's loads.  A load moves 64 units = ROWS_PER_LOAD rows; lane L moves, for row
    // ROWS_PER_LOAD chunk + L / UA, the unit whose slot in the row is L % UA (slot = unit ^ (row % 8)).
    const i32x4 img_rsrc = raw_buffer_words(img.src, img.bytes), filt_rsrc = raw_buffer_words(fb.filt, fb.bytes);
    int a_x[S::A_LOADS];                                   // image column of tap column 0 of the load's pixels: the same for all lanes
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int chunk = wave * S::A_LOADS + j;
        const int row = chunk * S::ROWS_PER_LOAD + lane / UA;
        const int unit = (lane % UA) ^ (row & 7);
        const int bx = (chunk * S::ROWS_PER_LOAD) / S::PY;                   // wave-uniform: the load's rows share their column
        const int y = y0 + row % S::PY, x = x0 + bx;
        // pixels below or right of the output are computed and never stored; what they load is range-checked like the rest
        a_x[j] = x - img.ox;
        a_off[j] = (uint32_t)(4 * ((y - img.oy) * img.row_stride + (x - img.ox) * img.dpitch) + 16 * unit);
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int row = (wave * S::B_LOADS + j) * S::ROWS_PER_LOAD + lane / UA;
        const int unit = (lane % UA) ^ (row & 7);
        int n = bn0 + row;
        if (n >= N) n = N - 1;                              // such filters are computed and never stored
        b_off[j] = (uint32_t)(4 * n * fb.filt_stride + 16 * unit);
    }
    // ---- the walk over (tap column, channel block) of the steps to fetch: wave-uniform, on the scalar unit.  Taps of one
    // row are contiguous in both tensors; from the last tap of a row to the first of the next the offsets jump by the rest
    // of the tensors' rows.  (The tap row itself is never needed: image rows outside the tensor fall out of range.)
    int walk_c = 0, walk_kj = 0, fetch_step = 0;
    uint32_t walk_off_a = 0, walk_off_b = 0;              // byte offsets of the step to fetch: in the image from tap (0,0), in a filter
    uint32_t walk_w = steps > 0 ? (uint32_t)img.W : 0u;   // the image width while there are steps to fetch, then 0: every column "outside"
    const uint32_t wrap_a = 4u * (uint32_t)(img.row_stride - img.kw * img.dpitch), wrap_b = 4u * (uint32_t)(fb.filt_row_stride - fb.kw * fb.dpitch);
    uint32_t a_next[S::A_LOADS], b_soff_next = 0;
    auto prepare_load = [&](auto j_tag) {                 // offsets of load J of the next batch (one scalar select, one vector addition)
        constexpr int J = decltype(j_tag)::value;
        const uint32_t add = (uint32_t)(a_x[J] + walk_kj) < walk_w ? walk_off_a : walk_off_a + kOutOfRange;
        a_next[J] = a_off[J] + add;
        if constexpr (J == 0) b_soff_next = walk_w != 0u ? walk_off_b : 0u;     // past the end of K: the first step again (never read)
    };
    auto advance_walk = [&] {
        walk_c += S::BK;
        ++fetch_step;
        const bool carry_c = walk_c >= img.dpitch;
        walk_c = carry_c ? 0 : walk_c;
        walk_kj += carry_c ? 1 : 0;
        walk_w = fetch_step < steps ? walk_w : 0u;
        const bool carry_kj = walk_kj >= img.kw;
        walk_kj = carry_kj ? 0 : walk_kj;
        walk_off_a += 4u * S::BK + (carry_kj ? wrap_a : 0u);
        walk_off_b += 4u * S::BK + (carry_kj ? wrap_b : 0u);
    };
    auto issue_one = [&](auto stage_tag, auto j_tag, auto site_tag) {     // site_tag: a number of its own for every place of call
        constexpr int ST = decltype(stage_tag)::value, J = decltype(j_tag)::value, TAG = decltype(site_tag)::value * 64 + J;
        if constexpr (J < S::A_LOADS) {
            dma_buffer_load16_tagged<TAG>(img_rsrc, a_next[J], 0u, lds_base + (uint32_t)(ST * S::STAGE_BYTES) + (uint32_t)(wave * S::A_LOADS + J) * 1024u);
        } else {
            constexpr int JB = J - S::A_LOADS;
            dma_buffer_load16_tagged<TAG>(filt_rsrc, b_off[JB], b_soff_next,
                                          lds_base + (uint32_t)(ST * S::STAGE_BYTES + S::A_BYTES) + (uint32_t)(wave * S::B_LOADS + JB) * 1024u);
        }
    };

    // the first STAGES steps go out before anything else is set up
    static_for<0, STAGES>([&](auto s_tag) {
        static_for<0, S::A_LOADS>([&](auto j) { prepare_load(j); });
        static_for<0, S::LOADS>([&](auto j) { issue_one(s_tag, j, std::integral_constant<int, 2 * STAGES + decltype(s_tag)::value>{}); });
        advance_walk();
    });
    __builtin_amdgcn_sched_barrier(0);

    // ---- where this lane's operands lie: float ls of unit q of row li of a block; the swizzle looks at the low bits of
    // the row only, which blocks and waves do not change, so block and buffer are whole rows further: an offset the
    // read carries
    const float* pa[UA];
    const float* pb[UA];
#pragma unroll
    for (int q = 0; q < UA; ++q) {
        pa[q] = reinterpret_cast<const float*>(lds_raw) + ((wm0 + li) * UA + (q ^ (li & 7))) * 4 + ls;
        pb[q] = reinterpret_cast<const float*>(lds_raw) + S::A_BYTES / 4 + ((wn0 + li) * UA + (q ^ (li & 7))) * 4 + ls;
    }

    // accumulators: lane holds D[4 ls + r][li], r = 0 .. 3, of each of its blocks (row = pixel, column = filter)
    f32x4 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};

    float af[2][HALF][MI], bf[2][HALF][NI];      // fragment sets: set 0 feeds the first half of a step, set 1 the second
    // read number n (0 .. READS-1) of half H of the step in buffer ST: k-group n / (MI + NI) of the half, filters first
    auto read_one = [&](auto st_tag, auto h_tag, auto n_tag) {
        constexpr int ST = decltype(st_tag)::value, H = decltype(h_tag)::value, NR = decltype(n_tag)::value;
        constexpr int G = NR / (MI + NI), W = NR % (MI + NI), Q = H * HALF + G;
        if constexpr (W < NI) bf[H][G][W] = pb[Q][(ST * S::STAGE_BYTES) / 4 + W * 16 * UA * 4];
        else af[H][G][W - NI] = pa[Q][(ST * S::STAGE_BYTES) / 4 + (W - NI) * 16 * UA * 4];
    };
    // matrix instruction m (0 .. MFMAS-1) of half H: k-group m / (MI NI) of the half, blocks in turn
    auto mfma_one = [&](auto h_tag, auto m_tag) {
        constexpr int H = decltype(h_tag)::value, MM = decltype(m_tag)::value;
        constexpr int G = MM / (MI * NI), BMI = (MM / NI) % MI, BNI = MM % NI;
        acc[BMI][BNI] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[H][G][BMI], bf[H][G][BNI], acc[BMI][BNI], 0, 0, 0);
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    wait_dma_then_barrier<S::LOADS*(STAGES - 1)>();                      // step 0 has landed
    static_for<0, READS>([&](auto n) { read_one(I0{}, I0{}, n); });     // its first half

    auto k_step = [&](auto st_tag, auto copy_tag) {
        constexpr int ST = decltype(st_tag)::value, SITE = decltype(copy_tag)::value * STAGES + ST;
        typedef std::integral_constant<int, (ST + 1) % STAGES> NextStage;
        // first half: read n of the second half goes out behind matrix instruction n MFMAS / READS; the offsets of the
        // loads to come are worked out behind the first instructions
        static_for<0, MFMAS>([&](auto m_tag) {
            constexpr int MM = decltype(m_tag)::value;
            mfma_one(I0{}, m_tag);
            static_for<0, READS>([&](auto n_tag) {
                if constexpr (decltype(n_tag)::value * MFMAS / READS == MM) read_one(st_tag, I1{}, n_tag);
            });
            if constexpr (MM < S::A_LOADS) prepare_load(m_tag);
            __builtin_amdgcn_sched_barrier(0);
        });
        // second half: the barrier behind its first instruction, then the loads of step t + STAGES behind instructions
        // 1, 2, ..., the walk's move to the step after behind the last load, and read n of the next step's first half
        // behind instruction 1 + n (MFMAS - 1) / READS
        static_for<0, MFMAS>([&](auto m_tag) {
            constexpr int MM = decltype(m_tag)::value;
            mfma_one(I1{}, m_tag);
            if constexpr (MM == 0) {
                __builtin_amdgcn_sched_barrier(0);
                wait_dma_then_barrier<S::LOADS*(STAGES - 2)>();          // step t+1 has landed; step t's buffer is free
            } else {
                if constexpr (MM - 1 < S::LOADS) issue_one(st_tag, std::integral_constant<int, MM - 1>{}, std::integral_constant<int, SITE>{});
                if constexpr (MM == S::LOADS) advance_walk();
                static_for<0, READS>([&](auto n_tag) {
                    if constexpr (1 + decltype(n_tag)::value * (MFMAS - 1) / READS == MM) read_one(NextStage{}, I0{}, n_tag);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    static_assert(S::A_LOADS <= MFMAS, "the offsets of the image loads are worked out during the first half");
    // whole passes over the buffers, free of branches, then the steps that are left
    int t0 = 0;
    for (; t0 + STAGES <= steps; t0 += STAGES) static_for<0, STAGES>([&](auto st) { k_step(st, I0{}); });
    static_for<0, STAGES - 1>([&](auto st) {
        if (t0 + decltype(st)::value < steps) k_step(st, I1{});
    });
    // the refills past the end of K still write when they land
    wait_dma_then_barrier<0>();

    // ---- epilogue: a lane's accumulator r of block (mi, ni) is pixel row wm0 + 16 mi + 4 ls + r of the tile under filter
    // bn0 + wn0 + 16 ni + li; 16 lanes store 16 consecutive filters of a pixel (64 contiguous bytes)
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int n = bn0 + wn0 + 16 * ni + li;
        const float bv = bias != nullptr && n < N ? bias[n] : 0.f;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = wm0 + 16 * mi + 4 * ls + r;
                const int y = y0 + row % S::PY, x = x0 + row / S::PY;
                if (y < Hout && x < out.Wout && n < N) {
                    float v = acc[mi][ni][r];
                    if (bias != nullptr) v += bv;                 // (adding 0 would turn -0 into +0)
                    dst[(size_t)y * out.row_stride + (size_t)x * out.dpitch + n] = out.finish(v);
                }
            }
    }
}

}  // namespace decx_hip
