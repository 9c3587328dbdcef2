// fp32 fused im2col convolution with both operands moved global -> LDS by the gfx950 LDS-DMA loads, on blocks of 16x16
// (v_mfma_f32_16x16x4_f32), for a channel pitch that is a multiple of the K step (32 floats).
//
// Why blocks of 16: 224x224 output pixels are 196 rows of the lowered product per CU.  Tiles of whole 32x32 blocks cover
// them with 224 rows on 224 CUs or with 208 rows by mixing block sizes; on 16x16 blocks a tile of 208 rows x 128 filters
// is 13 x 8 blocks -- 6 1/2 block rows of 32 where 6 1/8 is all the work there is -- on eight waves, two per SIMD, each
// wave owning all 13 row blocks of one 16-filter column.  Both instructions retire 32 multiply-adds per cycle.
// The 208 rows are a patch of 16 output rows x 13 columns, column by column: a block of 16 rows is 16 pixels of one image
// column, and so is each group of 8 rows that one load instruction fetches (224x224: 14 x 18 = 252 patches, one round).
//
// Why LDS-DMA: with the im2col lowering a K step lies inside one tap, and per output pixel it is 128 contiguous bytes of
// the image -- eight 16-byte units -- exactly as a row of A in the dense kernel (sgemm_dma_tile.hpp).  The filter bank
// holds filter n's taps channel-innermost, so its side of the step is 128 contiguous bytes per filter as well: B lies in
// LDS as B^T, in the same layout as A, and both fragments are one ds_read_b32 per MFMA and block (lane (i, s), i = 0..15,
// s = 0..3, reads float s of unit g of row i for the MFMA that covers k = 4g .. 4g+3).  Unit g of row r sits in slot
// g ^ (r % 8) of its row, and every other group of 8 rows starts 8 bytes off the 16-byte grid (the LDS-DMA loads take
// such a destination): the lower 32 lanes of a read -- 16 rows, floats 0 and 1 of their units -- then cover all 32 banks
// once, and so do the upper 32 (counted bank conflicts: half of the LDS cycles without the 8 bytes, none with them).
// The swizzle is applied on the global side (the lane whose place is slot t of row r fetches unit t ^ (r % 8)).
// buffer_load_dwordx4 ... lds takes a 32-bit offset into a buffer resource and answers an offset outside the buffer
// with zeros, written to LDS like data: image rows above and below the tensor fall out of range by themselves (negative
// or past the end).  Whether a tap lies left or right of the image is the same for all pixels of a load -- they share
// their column -- so the scalar unit decides it and adds 2^31 to the load's offset, which throws every lane out of range.
//
// Pipeline: two LDS buffers, one barrier per K step (eight k-groups of MI x NI MFMAs per wave).  Fragments are read one
// k-group ahead into the other of two register sets, between the MFMAs.  The barrier sits behind the first MFMA of the
// last k-group: before it the wave waits for its own loads of step t+1, after it nobody reads step t's buffer any
// more; the loads of step t+2 into that buffer and the reads of step t+1's first k-group follow between the remaining
// MFMAs.  The walk is whole passes over the two buffers, then one more step if the count is odd; the loads of every
// copy carry their own tag in the instruction text (dma_load16_tagged explains why).
// A 16x16x4 MFMA lasts 32 cycles, half of a 32x32x2, and what a wave issues between two of them shows: a vector
// instruction takes the matrix pipe's issue slot (probed: one v_add_u32 behind every 16x16x4 MFMA, two waves per SIMD,
// 152.6 -> 126 TFLOP/s; scalar instructions cost a tenth of that), a chain of dependent ones its latency besides.  Per
// step a wave therefore issues, beside its 104 MFMAs, 112 LDS reads and 6 loads, four vector instructions (one
// addition per image load) and the tap walk on the scalar unit, in pieces spread over the step.  With the pixels of a
// tile in raster order (a compare and a select per lane and image load, 14 vector instructions per step) the same kernel
// took 61.1 us on 224x224x64 under 128 filters; as patches 59.7 us: 18 K steps at 2.93 us where the 208 MFMAs of a SIMD
// take 2.77 us at 2.4 GHz, plus 7 us of launch, first loads and 25.7 MB of stores.
//
// Arithmetic: per output one fused multiply-add chain over ascending k = (ki*kw + kj)*dpitch + c, taps outside the image
// and padding channels entering as zeros -- the chain of sgemm_tile_kernel's convolution and of the reference
// (conv2_mk_im2col.h:167-274, eq_GEMM.cuh:109-209).  Bias and ReLU join the finished sum.
// The result tile leaves through LDS, up to four block rows at a time, as 16-byte non-temporal stores of whole output
// rows (the 25.7 MB of the 224x224x128 result, written by all CUs at once when the single round ends, take about 4 us).
#pragma once
#include "sgemm_tile.hpp"

namespace decx_hip {

template <int MI_, int NI_, int WAVES_M_, int WAVES_N_, int STAGES_ = 2>
struct SconvDmaShape {
    static constexpr int MI = MI_, NI = NI_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NWAVES = WAVES_M * WAVES_N, NT = 64 * NWAVES;
    static constexpr int BK = 32, U = BK / 4, STAGES = STAGES_, GROUPS = BK / 4;      // 16-byte units per row and step; k-groups per step
    static constexpr int WM = 16 * MI, WN = 16 * NI, BM = WM * WAVES_M, BN = WN * WAVES_N;
    static constexpr int A_LOADS = (BM * U + 64 * NWAVES - 1) / (64 * NWAVES), B_LOADS = BN * U / (64 * NWAVES), LOADS = A_LOADS + B_LOADS;
    static constexpr int A_ROWS = A_LOADS * NWAVES * 8;       // rows of A a buffer holds: BM rounded up to whole loads per wave (the surplus fetches nothing)
    // a load's 8 rows (1 KiB) are CHUNK bytes apart: every other group of 8 rows starts 8 bytes off the 16-byte grid, so
    // that the two floats per unit which the lower 32 lanes of a fragment read want lie on banks 0, 1 (mod 4) for rows
    // 0 - 7 of a block and on banks 2, 3 for rows 8 - 15: all 32 banks once
    static constexpr int CHUNK = 1024 + 8, BLOCK_BYTES = 2 * CHUNK;
    static constexpr int A_BYTES = A_ROWS / 8 * CHUNK, B_BYTES = BN / 8 * CHUNK;
    static_assert(A_BYTES % 16 == 0 && B_BYTES % 16 == 0, "buffers start on the 16-byte grid");
    static constexpr int MFMAS = MI * NI, READS = MI + NI;    // per k-group and wave
    static constexpr int OUT_ROW = BN + 4, OUT_FLOATS = 16 * WAVES_M * OUT_ROW;     // one block row of the result tile in LDS
    static constexpr size_t LDS_BYTES = (size_t)STAGES * (A_BYTES + B_BYTES);
    static_assert(BN * U % (64 * NWAVES) == 0, "filter loads divide over the waves");
    static_assert(MI * BLOCK_BYTES <= 65536 && NI * BLOCK_BYTES <= 65536, "a fragment read reaches every block and buffer by its offset field");
    static_assert(LOADS <= MFMAS - 1 && LOADS * (STAGES - 1) <= 63, "loads go out behind the MFMAs of a k-group; vmcnt is a 6-bit counter");
    static_assert(2 * OUT_FLOATS * 4 <= LDS_BYTES && BN % 4 == 0, "two block rows of the result fit the operand buffers");
    // block rows of the result that go through LDS between two barriers (two such groups lie in LDS side by side)
    static constexpr int OUT_GROUP = LDS_BYTES / (2 * OUT_FLOATS * 4) >= 4 ? 4 : LDS_BYTES / (2 * OUT_FLOATS * 4) >= 2 ? 2 : 1;
};

template <class S>
__global__ __launch_bounds__(S::NT) void sconv_dma_kernel(Im2colA<true> img, FilterB<true> fb, const float* __restrict__ bias,
                                                          float* __restrict__ dst, TensorOut out, int Hout, int N, int K,
                                                          int tiles_x, int tiles_m, int tiles_n) {
    constexpr int MI = S::MI, NI = S::NI, U = S::U, STAGES = S::STAGES, GROUPS = S::GROUPS, MFMAS = S::MFMAS, READS = S::READS;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];   // [STAGES][A_ROWS x U units] [STAGES][BN x U units]
    const uint32_t lds_base = lds_byte_address(lds_raw);

    const TileCoord tc = xcd_grouped_tile((int)blockIdx.x, tiles_m, tiles_n, 8);
    // a tile is a patch of 16 output rows x TILE_X columns: row 16 bx + yy of the lowered product is pixel (y0 + yy, x0 + bx),
    // so a block of 16 rows -- and each of the two loads that fetch it -- lies in one image column
    constexpr int TILE_X = S::BM / 16;
    const int tile_y = tc.tm / tiles_x, tile_x = tc.tm - tile_y * tiles_x;
    const int y0 = 16 * tile_y, x0 = TILE_X * tile_x, bn0 = tc.tn * S::BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane % 16, ls = lane / 16;
    const int steps = K / S::BK;

    // ---- sources of this wave's loads.  A load moves 64 units = 8 rows; lane L moves, for row 8c + L/8, the unit whose
    // slot in the row is L%8.
    const i32x4 img_rsrc = raw_buffer_words(img.src, img.bytes), filt_rsrc = raw_buffer_words(fb.filt, fb.bytes);
    int a_x[S::A_LOADS];                                   // image column of tap column 0 of the load's pixels: the same for all lanes
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int chunk = wave * S::A_LOADS + j;             // rows 8 chunk .. 8 chunk + 7: column x0 + chunk / 2, rows y0 + 8 (chunk % 2) ...
        const int unit = (lane % 8) ^ (lane / 8);
        const int y = y0 + 8 * (chunk % 2) + lane / 8, x = x0 + chunk / 2;
        // pixels below or right of the output are computed and never stored; what they load is range-checked like everything else
        a_x[j] = chunk < 2 * TILE_X ? x - img.ox : -(1 << 30);      // rows past the tile: every tap "outside"
        a_off[j] = (uint32_t)(4 * ((y - img.oy) * img.row_stride + (x - img.ox) * img.dpitch) + 16 * unit);
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int r = (wave * S::B_LOADS + j) * 8 + lane / 8;
        const int unit = (lane % 8) ^ (lane / 8);
        int n = bn0 + r;
        if (n >= N) n = N - 1;
        b_off[j] = (uint32_t)(4 * n * fb.filt_stride + 16 * unit);
    }
    // ---- the walk over (tap column, channel block) of the steps to fetch: wave-uniform, on the scalar unit.  A step of 32
    // channels stays inside a tap; taps of one row are contiguous in both tensors; from the last tap of a row to the first of
    // the next the offsets jump by the rest of the tensors' rows.  (The tap row itself is never needed: image rows above
    // and below the tensor fall out of the buffer's range.)
    int walk_c = 0, walk_kj = 0, fetch_step = 0;          // channel and tap column of the step to fetch; its number
    uint32_t walk_off_a = 0, walk_off_b = 0;              // byte offsets of that position in the image (from tap (0,0)) and in a filter
    uint32_t walk_w = steps > 0 ? (uint32_t)img.W : 0u;   // the image width while there are steps to fetch, then 0: every column "outside"
    const uint32_t wrap_a = 4u * (uint32_t)(img.row_stride - img.kw * img.dpitch), wrap_b = 4u * (uint32_t)(fb.filt_row_stride - fb.kw * fb.dpitch);
    // Offsets of the next batch of loads, worked out ahead of time in pieces that are spread between the MFMAs of a step:
    // every instruction a wave issues between two MFMAs delays its next MFMA by its own latency when it depends on the one
    // before (measured: 12 dependent additions per step cost 0.11 us of 2.8), and a vector instruction takes the matrix
    // pipe's issue slot besides.  An image load's pixels share their column, so whether the tap lies beside the image is
    // the scalar unit's to decide: it adds 2^31 to the walk's offset of such a load, which throws every lane out of the
    // buffer's range (tensors stay below 2 GiB less the apron, checked by the launcher).  That leaves one vector addition
    // per image load and step.  A filter load needs none: the walk is its scalar offset, and past the end of K it
    // fetches the filter's first step again (never read).
    uint32_t a_next[S::A_LOADS], a_add[S::A_LOADS], b_soff_next = 0;
    constexpr int PREPARE_PIECES = 2 * S::A_LOADS, ADVANCE_PIECES = 3;
    auto prepare_piece = [&](auto p_tag) {
        constexpr int P = decltype(p_tag)::value, J = P / 2;
        if constexpr (P % 2 == 0) {
            a_add[J] = (uint32_t)(a_x[J] + walk_kj) < walk_w ? walk_off_a : walk_off_a + kOutOfRange;
            if constexpr (P == 0) b_soff_next = walk_w != 0u ? walk_off_b : 0u;
        } else {
            a_next[J] = a_off[J] + a_add[J];
        }
    };
    auto advance_piece = [&](auto q_tag) {
        constexpr int Q = decltype(q_tag)::value;
        if constexpr (Q == 0) {
            walk_c += S::BK;
            ++fetch_step;
        } else if constexpr (Q == 1) {
            const bool carry_c = walk_c >= img.dpitch;
            walk_c = carry_c ? 0 : walk_c;
            walk_kj += carry_c ? 1 : 0;
            walk_w = fetch_step < steps ? walk_w : 0u;
        } else {
            const bool carry_kj = walk_kj >= img.kw;
            walk_kj = carry_kj ? 0 : walk_kj;
            walk_off_a += 4u * S::BK + (carry_kj ? wrap_a : 0u);
            walk_off_b += 4u * S::BK + (carry_kj ? wrap_b : 0u);
        }
    };
    auto issue_one = [&](auto stage_tag, auto j_tag, auto site_tag) {     // site_tag: a number of its own for every place of call
        constexpr int ST = decltype(stage_tag)::value, J = decltype(j_tag)::value, TAG = decltype(site_tag)::value * 64 + J;
        if constexpr (J < S::A_LOADS) {
            dma_buffer_load16_tagged<TAG>(img_rsrc, a_next[J], 0u, lds_base + (uint32_t)(ST * S::A_BYTES) + (uint32_t)((wave * S::A_LOADS + J) * S::CHUNK));
        } else {
            constexpr int JB = J - S::A_LOADS;
            dma_buffer_load16_tagged<TAG>(filt_rsrc, b_off[JB], b_soff_next,
                                          lds_base + (uint32_t)(STAGES * S::A_BYTES + ST * S::B_BYTES) + (uint32_t)((wave * S::B_LOADS + JB) * S::CHUNK));
        }
    };

    // the first STAGES steps go out before anything else is set up: the rest of the preparation runs under their latency
    if (steps > 0) {
        static_for<0, STAGES>([&](auto s_tag) {
            static_for<0, PREPARE_PIECES>([&](auto p) { prepare_piece(p); });
            static_for<0, S::LOADS>([&](auto j) { issue_one(s_tag, j, std::integral_constant<int, 2 * STAGES + decltype(s_tag)::value>{}); });
            static_for<0, ADVANCE_PIECES>([&](auto q) { advance_piece(q); });
        });
        __builtin_amdgcn_sched_barrier(0);
    }

    // ---- where this lane's operands lie: float ls of unit g of row li of a block, one register per unit and operand;
    // block and buffer are whole rows further, in the offset field of the read
    const float* pa[STAGES][GROUPS];
    const float* pb[STAGES][GROUPS];
#pragma unroll
    for (int st = 0; st < STAGES; ++st)
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            const int in_block = (li / 8) * (S::CHUNK / 4) + (li % 8) * (U * 4) + (g ^ (li & 7)) * 4 + ls;
            pa[st][g] = reinterpret_cast<const float*>(lds_raw) + st * (S::A_BYTES / 4) + (wm0 / 16) * (S::BLOCK_BYTES / 4) + in_block;
            pb[st][g] = reinterpret_cast<const float*>(lds_raw) + STAGES * (S::A_BYTES / 4) + st * (S::B_BYTES / 4) + (wn0 / 16) * (S::BLOCK_BYTES / 4) + in_block;
        }

    // accumulators: lane holds D[4 ls + r][li], r = 0 .. 3, of each of its blocks
    f32x4 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4{0.f, 0.f, 0.f, 0.f};

    float af[2][MI], bf[2][NI];      // fragment sets: k-group g computes from set g % 2
    // read number n (0 .. READS-1) of k-group G of the step in buffer ST, into set G % 2
    auto read_one = [&](auto st_tag, auto g_tag, auto n_tag) {
        constexpr int ST = decltype(st_tag)::value, G = decltype(g_tag)::value, NR = decltype(n_tag)::value;
        // filters first: the first MFMA of the k-group waits for them, the last row block is needed last
        if constexpr (NR < NI) bf[G % 2][NR] = pb[ST][G][NR * (S::BLOCK_BYTES / 4)];
        else af[G % 2][NR - NI] = pa[ST][G][(NR - NI) * (S::BLOCK_BYTES / 4)];
    };
    auto mfma_one = [&](auto g_tag, auto m_tag) {
        constexpr int G = decltype(g_tag)::value, MM = decltype(m_tag)::value, BMI = MM / NI, BNI = MM % NI;
        acc[BMI][BNI] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[G % 2][BMI], bf[G % 2][BNI], acc[BMI][BNI], 0, 0, 0);
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    if (steps > 0) {
        wait_dma_then_barrier<S::LOADS*(STAGES - 1)>();                      // step 0 has landed
        static_for<0, READS>([&](auto n) { read_one(I0{}, I0{}, n); });     // its first k-group

        // One K step.  Between the MFMAs of k-groups 0 .. GROUPS-2: the reads of the next k-group and, PIECE_EVERY MFMAs
        // apart, the pieces that prepare this step's loads.  In the last k-group: the barrier behind its first MFMA, then
        // the loads, then the pieces that move the walk on, and the reads of the next step's first k-group.
        constexpr int PIECE_EVERY = (GROUPS - 1) * MFMAS / (PREPARE_PIECES + 1);
        static_assert(PIECE_EVERY >= 1 && 1 + S::LOADS + ADVANCE_PIECES <= MFMAS, "the pieces fit between the MFMAs");
        auto k_step = [&](auto st_tag, auto copy_tag) {
            constexpr int ST = decltype(st_tag)::value, SITE = decltype(copy_tag)::value * STAGES + ST;
            typedef std::integral_constant<int, (ST + 1) % STAGES> NextStage;
            static_for<0, GROUPS>([&](auto g_tag) {
                constexpr int G = decltype(g_tag)::value;
                static_for<0, MFMAS>([&](auto m_tag) {
                    constexpr int MM = decltype(m_tag)::value, SLOT = G * MFMAS + MM;
                    mfma_one(g_tag, m_tag);
                    if constexpr (G + 1 < GROUPS) {
                        // the next k-group's operands: read n goes out behind MFMA n MFMAS / READS
                        static_for<0, READS>([&](auto n_tag) {
                            if constexpr (decltype(n_tag)::value * MFMAS / READS == MM) read_one(st_tag, std::integral_constant<int, G + 1>{}, n_tag);
                        });
                        if constexpr (SLOT % PIECE_EVERY == PIECE_EVERY - 1 && SLOT / PIECE_EVERY < PREPARE_PIECES) prepare_piece(std::integral_constant<int, SLOT / PIECE_EVERY>{});
                    } else if constexpr (MM == 0) {
                        __builtin_amdgcn_sched_barrier(0);
                        wait_dma_then_barrier<S::LOADS*(STAGES - 2)>();      // step t+1 has landed; step t's buffer is free
                    } else {
                        if constexpr (MM - 1 < S::LOADS) issue_one(st_tag, std::integral_constant<int, MM - 1>{}, std::integral_constant<int, SITE>{});
                        else if constexpr (MM - 1 - S::LOADS < ADVANCE_PIECES) advance_piece(std::integral_constant<int, MM - 1 - S::LOADS>{});
                        static_for<0, READS>([&](auto n_tag) {
                            if constexpr (1 + decltype(n_tag)::value * (MFMAS - 1) / READS == MM) read_one(NextStage{}, I0{}, n_tag);
                        });
                    }
                    __builtin_amdgcn_sched_barrier(0);
                });
            });
        };
        static_assert(GROUPS % 2 == 0, "k-group 0 always computes from set 0");
        int t0 = 0;
        for (; t0 + STAGES <= steps; t0 += STAGES) static_for<0, STAGES>([&](auto st) { k_step(st, I0{}); });
        static_for<0, STAGES - 1>([&](auto st) {
            if (t0 + decltype(st)::value < steps) k_step(st, I1{});
        });
    }
    // the refills past the end of K still write (zeros) when they land: wait for them before LDS becomes the result tile
    wait_dma_then_barrier<0>();

    // ---- result: OUT_GROUP block rows of every wave go to LDS (bias and ReLU applied), then leave as whole rows of
    // 16-byte stores; two such LDS tiles in turn, so one barrier per group
    // (bias and ReLU are the same for the whole launch: one instance of the loop per combination, chosen by scalar
    // branches, instead of selects per element -- vector instructions here are time with nothing behind them to hide in)
    float bv[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int n = bn0 + wn0 + 16 * ni + li;
        bv[ni] = bias != nullptr && n < N ? bias[n] : 0.f;
    }
    float* out_lds = reinterpret_cast<float*>(lds_raw);
    const int wave_m = wave / S::WAVES_N;
    constexpr int UNITS = 16 * S::WAVES_M * (S::BN / 4);
    static_assert(UNITS % S::NT == 0, "the stores of a block row divide over the threads");
    // where this thread's 16-byte units of a block row go: row `srow` of the LDS tile = output row sy of column sx0 (+ 1
    // per block row)
    int srow[UNITS / S::NT], sy[UNITS / S::NT], sx0[UNITS / S::NT], sc4[UNITS / S::NT];
#pragma unroll
    for (int it = 0; it < UNITS / S::NT; ++it) {
        const int id = tid + it * S::NT;
        srow[it] = id / (S::BN / 4);
        sc4[it] = id % (S::BN / 4);
        sy[it] = y0 + srow[it] % 16;
        sx0[it] = x0 + (srow[it] / 16) * MI;
    }
    auto store_tile = [&](auto bias_tag, auto relu_tag) {
        constexpr bool BIAS = decltype(bias_tag)::value, RELU = decltype(relu_tag)::value;
#pragma unroll
        for (int p0 = 0; p0 < MI; p0 += S::OUT_GROUP) {
            float* ot = out_lds + ((p0 / S::OUT_GROUP) & 1) * (S::OUT_GROUP * S::OUT_FLOATS);
#pragma unroll
            for (int pp = 0; pp < S::OUT_GROUP && p0 + pp < MI; ++pp)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float v = BIAS ? acc[p0 + pp][ni][r] + bv[ni] : acc[p0 + pp][ni][r];      // (adding 0 would turn -0 into +0)
                        ot[pp * S::OUT_FLOATS + (wave_m * 16 + 4 * ls + r) * S::OUT_ROW + wn0 + 16 * ni + li] = RELU ? relu_by_sign(v) : v;
                    }
            lds_sync();
#pragma unroll
            for (int pp = 0; pp < S::OUT_GROUP && p0 + pp < MI; ++pp)
#pragma unroll
                for (int it = 0; it < UNITS / S::NT; ++it) {
                    const int x = sx0[it] + p0 + pp, n = bn0 + 4 * sc4[it];
                    if (sy[it] < Hout && x < out.Wout && n < N) {      // N is a multiple of 4: a quad is inside or outside as a whole
                        const f32x4 v = *reinterpret_cast<const f32x4*>(ot + pp * S::OUT_FLOATS + srow[it] * S::OUT_ROW + 4 * sc4[it]);
                        __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(dst + (size_t)sy[it] * out.row_stride + (size_t)x * out.dpitch + n));
                    }
                }
        }
    };
    typedef std::integral_constant<bool, false> No;
    typedef std::integral_constant<bool, true> Yes;
    if (bias != nullptr) {
        if (out.relu) store_tile(Yes{}, Yes{});
        else store_tile(Yes{}, No{});
    } else {
        if (out.relu) store_tile(No{}, Yes{});
        else store_tile(No{}, No{});
    }
}

}  // namespace decx_hip
