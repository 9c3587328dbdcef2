// fp16 fused im2col convolution (fp32 accumulate) on v_mfma_f32_16x16x32_f16, both operands moved global -> LDS by the
// gfx950 LDS-DMA loads, for a channel pitch that is a multiple of the K step (64 halves).
//
// The K walk is the one of the large fp16 GEMM tile (hgemm_mfma16_tile.hpp): two LDS stages of 64 k, a K step cut into
// four units (k-block x half of the wave's row blocks) whose fragments are fetched during the unit before, the barrier
// inside the last unit, the refill of the stage a step leaves between that unit's remaining matrix instructions, stage,
// k-block and block of every fragment read folded into the instruction's offset field, the matrix instructions of a unit
// ordered so that one operand changes at a time.  What differs is where the operands come from:
//   * a tile's 256 rows are a PATCH of 16 output rows x 16 columns, column by column: row 16 bx + yy of the lowered
//     product is pixel (y0 + yy, x0 + bx).  A K step lies inside one tap, and per pixel it is 128 contiguous bytes of the
//     image -- eight 16-byte units, a row of A as in the dense kernel.  A load instruction moves 8 rows, i.e. 8 pixels of
//     ONE image column: whether its tap lies left or right of the image is the same for all its lanes, so the scalar
//     unit decides it and adds 2^31 to the load's offset, which throws every lane out of the buffer's range
//     (buffer_load_dwordx4 ... lds answers an offset outside the buffer with zeros, written to LDS like data); image rows
//     above and below the tensor fall out of range by themselves.  That leaves one vector addition per image load and
//     K step; the tap walk itself runs on the scalar unit, in pieces spread between the matrix instructions.
//   * the filter bank holds filter n's taps channel-innermost: its side of a K step is 128 contiguous bytes per filter,
//     B^T in the layout of A.  Both fragments are ds_read_b128 (no transposing reads), from rows swizzled alike.
//   * the filter fragment is the matrix instruction's first operand: a lane then owns 4 consecutive filters of one
//     pixel; bias, ReLU and the one rounding to binary16 are applied to them, the wave's piece is parked in LDS and
//     leaves as 16-byte stores, 128 contiguous bytes per pixel and wave.
// K is walked in ascending k = (ki kw + kj) dpitch + c, the order of the reference's lowering (im2col.cuh:146-153).
#pragma once
#include "hconv_dma.hpp"
#include "hgemm_mfma16_tile.hpp"

namespace decx_hip {

template <int BN_, int WAVES_M_, int WAVES_N_>
struct Hconv16Shape {
    static constexpr int PATCH_Y = 16, PATCH_X = 16;
    static constexpr int BM = PATCH_Y * PATCH_X, BN = BN_, BK = 64, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = 2;
    static constexpr int NWAVES = WAVES_M * WAVES_N, NT = NWAVES * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 16, NI = WN / 16;            // 16 x 16 accumulator blocks of a wave
    static constexpr int MH = 2, UM = MI / MH;                  // a unit = one k-block x UM row blocks
    static constexpr int KS = BK / 32, UNITS = KS * MH;
    static constexpr int ROW_BYTES = BK * 2, BLOCK_BYTES = 16 * ROW_BYTES;         // a row of either operand in LDS; 16 of them
    static constexpr int A_BYTES = BM * ROW_BYTES, B_BYTES = BN * ROW_BYTES;
    static constexpr int A_LOADS = BM / 8 / NWAVES, B_LOADS = BN / 8 / NWAVES, LOADS = A_LOADS + B_LOADS;   // 8 rows per load
    static constexpr size_t LDS_BYTES = (size_t)STAGES * (A_BYTES + B_BYTES);
    static_assert(MI % MH == 0 && NI % MH == 0 && WM % 16 == 0 && WN % 16 == 0, "units of whole blocks");
    static_assert(BM % (8 * NWAVES) == 0 && BN % (8 * NWAVES) == 0, "loads must divide over the waves");
    static_assert((size_t)NWAVES * WM * WN * 2 <= LDS_BYTES, "the epilogue parks every wave's piece in LDS");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS of a CU");
    static_assert(MI * BLOCK_BYTES <= 65536 && NI * BLOCK_BYTES <= 65536, "a fragment read reaches every block by its offset field");
    static_assert(WN >= 64 && (WN / 8 & (WN / 8 - 1)) == 0, "the parked piece is swizzled in rows of >= 8 pieces");
};

template <class S>
__global__ __launch_bounds__(S::NT) void hconv_mfma16_kernel(HalfImage img, HalfFilters fb, HalfTensorOut out, int Hout, int N,
                                                             int tiles_x, int tiles_m, int tiles_n) {
    constexpr int BN = S::BN, MI = S::MI, NI = S::NI, UM = S::UM, MH = S::MH, KS = S::KS, UNITS = S::UNITS, STAGES = S::STAGES;
    constexpr int A_BYTES = S::A_BYTES, B_BYTES = S::B_BYTES, BLOCK_BYTES = S::BLOCK_BYTES;
    constexpr int BLK = UM * NI;                                // matrix instructions per unit
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];   // [A stages][B stages]
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw;

    const TileCoord tc = xcd_grouped_tile((int)blockIdx.x, tiles_m, tiles_n, 8);
    const int tile_y = tc.tm / tiles_x, tile_x = tc.tm - tile_y * tiles_x;
    const int y0 = S::PATCH_Y * tile_y, x0 = S::PATCH_X * tile_x, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int lg = lane >> 4, li = lane & 15;                   // 16-lane group = k sub-block, lane in group = row of a block
    const int steps = img.kh * img.kw * (img.dpitch_w / 32);    // K steps of 64 halves = 32 words

    // ---- sources of this wave's loads.  A load moves 64 units = 8 rows; lane L moves, for row 8c + L/8, the unit whose slot
    // in the row is L%8 (slot = unit ^ ((row/2) % 8), a_unit_slot).  Rows 8c .. 8c+7 of A: column x0 + c/2, rows y0 + 8 (c%2) ...
    const i32x4 img_rsrc = raw_buffer_words(img.src, img.bytes), filt_rsrc = raw_buffer_words(fb.filt, fb.bytes);
    int a_x[S::A_LOADS];                                        // image column of tap column 0 of the load's pixels (wave-uniform)
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int chunk = wave * S::A_LOADS + j;
        const int r = 8 * chunk + lane / 8;
        const int unit = (lane % 8) ^ ((r / 2) % 8);
        const int y = y0 + 8 * (chunk % 2) + lane / 8, x = x0 + chunk / 2;
        // pixels below or right of the output are computed and never stored; what they load is range-checked like the rest
        a_x[j] = x - img.ox;
        a_off[j] = (uint32_t)(4 * ((y - img.oy) * img.row_stride_w + (x - img.ox) * img.dpitch_w) + 16 * unit);
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int r = (wave * S::B_LOADS + j) * 8 + lane / 8;
        const int unit = (lane % 8) ^ ((r / 2) % 8);
        int n = bn0 + r;
        if (n >= N) n = N - 1;                                  // such filters are computed and never stored
        b_off[j] = (uint32_t)(4 * n * fb.filt_stride_w + 16 * unit);
    }
    // ---- the walk over (tap column, channel block) of the steps to fetch: wave-uniform, on the scalar unit.  Taps of one
    // row are contiguous in both tensors; from the last tap of a row to the first of the next the offsets jump by the rest
    // of the tensors' rows.  (The tap row itself is never needed: image rows outside the tensor fall out of range.)
    int walk_c = 0, walk_kj = 0, fetch_step = 0;
    uint32_t walk_off_a = 0, walk_off_b = 0;                    // byte offsets of the step to fetch: in the image from tap (0,0), in a filter
    uint32_t walk_w = (uint32_t)img.W;                          // the image width while there are steps to fetch, then 0: every column "outside"
    const uint32_t wrap_a = 4u * (uint32_t)(img.row_stride_w - img.kw * img.dpitch_w), wrap_b = 4u * (uint32_t)(fb.row_stride_w - fb.kw * fb.dpitch_w);
    uint32_t a_next[S::A_LOADS], a_add[S::A_LOADS], b_soff_next = 0;
    constexpr int PREPARE_PIECES = 2 * S::A_LOADS, ADVANCE_PIECES = 3;
    auto prepare_piece = [&](auto p_tag) {                      // offsets of the next batch of loads, in pieces
        constexpr int P = decltype(p_tag)::value, J = P / 2;
        if constexpr (P % 2 == 0) {
            a_add[J] = (uint32_t)(a_x[J] + walk_kj) < walk_w ? walk_off_a : walk_off_a + kOutOfRange;
            if constexpr (P == 0) b_soff_next = walk_w != 0u ? walk_off_b : 0u;     // past the end of K: the first step again (never read)
        } else {
            a_next[J] = a_off[J] + a_add[J];
        }
    };
    auto advance_piece = [&](auto q_tag) {
        constexpr int Q = decltype(q_tag)::value;
        if constexpr (Q == 0) {
            walk_c += 32;
            ++fetch_step;
        } else if constexpr (Q == 1) {
            const bool carry_c = walk_c >= img.dpitch_w;
            walk_c = carry_c ? 0 : walk_c;
            walk_kj += carry_c ? 1 : 0;
            walk_w = fetch_step < steps ? walk_w : 0u;
        } else {
            const bool carry_kj = walk_kj >= img.kw;
            walk_kj = carry_kj ? 0 : walk_kj;
            walk_off_a += 128u + (carry_kj ? wrap_a : 0u);
            walk_off_b += 128u + (carry_kj ? wrap_b : 0u);
        }
    };
    auto issue_one = [&](auto stage_tag, auto j_tag, auto site_tag) {     // site_tag: a number of its own for every place of call
        constexpr int STG = decltype(stage_tag)::value, J = decltype(j_tag)::value, TAG = decltype(site_tag)::value * 64 + J;
        if constexpr (J < S::A_LOADS) {
            dma_buffer_load16_tagged<TAG>(img_rsrc, a_next[J], 0u, lds_base + (uint32_t)(STG * A_BYTES) + (uint32_t)(wave * S::A_LOADS + J) * 1024u);
        } else {
            constexpr int JB = J - S::A_LOADS;
            dma_buffer_load16_tagged<TAG>(filt_rsrc, b_off[JB], b_soff_next,
                                          lds_base + (uint32_t)(STAGES * A_BYTES + STG * B_BYTES) + (uint32_t)(wave * S::B_LOADS + JB) * 1024u);
        }
    };

    f32x4v acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4v{0.f, 0.f, 0.f, 0.f};

    // ---- fragment reads: lane (lg, li) reads the 8 halves k = 32 kb + 8 lg .. + 7 of row li of a block -- unit 4 kb + lg
    // of that row, wherever the swizzle put it.  One per-lane byte offset per operand, stage and k-block; the block is a
    // constant in the instruction (16 rows further do not change the swizzle).
    uint32_t a_rd[STAGES][KS], b_rd[STAGES][KS];
#pragma unroll
    for (int st = 0; st < STAGES; ++st)
#pragma unroll
        for (int kb = 0; kb < KS; ++kb) {
            a_rd[st][kb] = (uint32_t)(st * A_BYTES + a_unit_slot(wm0 + li, 4 * kb + lg, 8) * 16);
            b_rd[st][kb] = (uint32_t)(STAGES * A_BYTES + st * B_BYTES + a_unit_slot(wn0 + li, 4 * kb + lg, 8) * 16);
        }
    f16x8 af[2][UM];                                            // by unit parity
    f16x8 bf[2][NI];                                            // by the parity of the k-block (KS is even: the same in every step)
    static_assert(KS % 2 == 0 && UNITS % 2 == 0, "fragment sets alternate by unit and by k-block");
    auto read_a = [&](auto set_tag, auto slot_tag, auto stage_tag, auto kb_tag, auto rb_tag) {
        af[decltype(set_tag)::value][decltype(slot_tag)::value] = __builtin_bit_cast(
            f16x8, *reinterpret_cast<const u32x4*>(lds_raw + a_rd[decltype(stage_tag)::value][decltype(kb_tag)::value] + decltype(rb_tag)::value * BLOCK_BYTES));
    };
    auto read_b = [&](auto stage_tag, auto kb_tag, auto ni_tag) {
        bf[decltype(kb_tag)::value & 1][decltype(ni_tag)::value] = __builtin_bit_cast(
            f16x8, *reinterpret_cast<const u32x4*>(lds_raw + b_rd[decltype(stage_tag)::value][decltype(kb_tag)::value] + decltype(ni_tag)::value * BLOCK_BYTES));
    };
    // read number R of the fragments a K step in stage STG starts with (unit 0: row blocks 0 .. UM-1, k-block 0), in the
    // order its first matrix instructions need them: A block 0, all of B, the other A blocks
    constexpr int FIRST_READS = UM + NI;
    typedef std::integral_constant<int, 0> I0;
    auto read_first = [&](auto stage_tag, auto r_tag) {
        constexpr int R = decltype(r_tag)::value;
        if constexpr (R == 0) read_a(I0{}, I0{}, stage_tag, I0{}, I0{});
        else if constexpr (R <= NI) read_b(stage_tag, I0{}, std::integral_constant<int, R - 1>{});
        else read_a(I0{}, std::integral_constant<int, R - NI>{}, stage_tag, I0{}, std::integral_constant<int, R - NI>{});
    };
    // matrix instruction I of unit U: row blocks one after the other, the column order reversed on every other one
    auto mfma_one = [&](auto u_tag, auto i_tag) {
        constexpr int U = decltype(u_tag)::value, I = decltype(i_tag)::value;
        constexpr int ROWB = I / NI, NIX = (ROWB & 1) ? NI - 1 - I % NI : I % NI;
        constexpr int KB = U / MH, MIX = (U % MH) * UM + ROWB;
        acc[MIX][NIX] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[KB & 1][NIX], af[U & 1][ROWB], acc[MIX][NIX], 0, 0, 0);
    };
#define DECX_PIN() __builtin_amdgcn_sched_barrier(0)

    // One K step from stage STG.  On entry af[0] and bf[0] hold the fragments of unit 0; on exit those of the next step.
    // Units 0 .. UNITS-2: the first matrix instructions each carry one LDS read of the next unit's A fragments and of this
    // unit's share of the next k-block's B fragments; every PIECE_EVERY instructions a piece of the next loads' offsets.
    // Last unit: a few matrix instructions, then wait for the next step's data + barrier -- nobody reads this stage any
    // more -- and between the remaining ones the refill of this stage, the walk's move to the step after, and the first
    // fragments of the next step from the other stage.
    constexpr int PIECE_EVERY = (UNITS - 1) * BLK / PREPARE_PIECES;
    static_assert(PIECE_EVERY >= 1, "the pieces fit between the matrix instructions");
    auto k_step = [&](auto stage_tag, auto copy_tag) {
        constexpr int STG = decltype(stage_tag)::value, SITE = decltype(copy_tag)::value * STAGES + STG;
        typedef std::integral_constant<int, (STG + 1) % STAGES> Next;
        static_for<0, UNITS - 1>([&](auto u_tag) {
            constexpr int U = decltype(u_tag)::value, KB = U / MH, H = U % MH;
            constexpr int NU = U + 1, NKB = NU / MH, NH = NU % MH;
            constexpr int NB = (KB + 1 < KS) ? NI / MH : 0;      // B reads of the next k-block in this unit
            constexpr int NR = UM + NB;
            static_assert(NR <= BLK, "one read per matrix instruction");
            static_for<0, BLK>([&](auto i_tag) {
                constexpr int I = decltype(i_tag)::value, SLOT = U * BLK + I;
                if constexpr (I < UM) {
                    read_a(std::integral_constant<int, NU & 1>{}, i_tag, stage_tag, std::integral_constant<int, NKB>{},
                           std::integral_constant<int, NH * UM + I>{});
                } else if constexpr (I < NR) {
                    read_b(stage_tag, std::integral_constant<int, KB + 1>{}, std::integral_constant<int, H * NB + (I - UM)>{});
                }
                mfma_one(u_tag, i_tag);
                if constexpr (SLOT % PIECE_EVERY == PIECE_EVERY - 1 && SLOT / PIECE_EVERY < PREPARE_PIECES)
                    prepare_piece(std::integral_constant<int, SLOT / PIECE_EVERY>{});
                DECX_PIN();
            });
        });
        typedef std::integral_constant<int, UNITS - 1> Last;
        constexpr int PRE = BLK / 4, SLOTS = BLK - PRE;
        static_assert(SLOTS >= ADVANCE_PIECES, "the walk moves on inside the last unit");
        static_for<0, PRE>([&](auto i_tag) {
            mfma_one(Last{}, i_tag);
            DECX_PIN();
        });
        wait_dma_then_barrier<S::LOADS*(STAGES - 2)>();         // the next step has landed; this step's stage is free
        DECX_PIN();
        static_for<0, SLOTS>([&](auto i_tag) {
            constexpr int I = decltype(i_tag)::value;
            static_for<(I * S::LOADS) / SLOTS, ((I + 1) * S::LOADS) / SLOTS>([&](auto j_tag) {
                issue_one(stage_tag, j_tag, std::integral_constant<int, SITE>{});
            });
            if constexpr (I >= SLOTS - ADVANCE_PIECES) advance_piece(std::integral_constant<int, I - (SLOTS - ADVANCE_PIECES)>{});
            constexpr int R0 = 2 * I < FIRST_READS ? 2 * I : FIRST_READS, R1 = 2 * I + 2 < FIRST_READS ? 2 * I + 2 : FIRST_READS;
            static_for<R0, R1>([&](auto r_tag) { read_first(Next{}, r_tag); });
            mfma_one(Last{}, std::integral_constant<int, PRE + I>{});
            DECX_PIN();
        });
        static_assert(2 * SLOTS >= FIRST_READS, "the next step's first fragments go out in the last unit");
    };

    // prologue: both stages get a step (the second may lie past the end of K: zeros), K step j into stage j
    static_for<0, STAGES>([&](auto s_tag) {
        static_for<0, PREPARE_PIECES>([&](auto p) { prepare_piece(p); });
        static_for<0, S::LOADS>([&](auto j) { issue_one(s_tag, j, std::integral_constant<int, 2 * STAGES + decltype(s_tag)::value>{}); });
        static_for<0, ADVANCE_PIECES>([&](auto q) { advance_piece(q); });
    });
    wait_dma_then_barrier<S::LOADS*(STAGES - 1)>();             // step 0 has landed
    static_for<0, FIRST_READS>([&](auto r) { read_first(I0{}, r); });
    DECX_PIN();
    {
        typedef std::integral_constant<int, 1> I1;
        int t = 0;
        for (; t + STAGES <= steps; t += STAGES) static_for<0, STAGES>([&](auto st) { k_step(st, I0{}); });
        if (t < steps) k_step(I0{}, I1{});                       // an odd count: one more step from stage 0
    }
#undef DECX_PIN

    // ---- epilogue.  acc[mi][ni][e] is (row 16 mi + li, filter 16 ni + 4 lg + e) of the wave's piece; row r of the tile is
    // pixel (y0 + r % 16, x0 + r / 16).  The refills past the end of K still write when they land: wait for them before LDS
    // becomes the parking area.
    wait_dma_then_barrier<0>();
    constexpr int ROW_BYTES = S::WN * 2, PIECES = S::WN / 8, ROWS_PER_PASS = kWave / PIECES, PASSES = S::WM / ROWS_PER_PASS;
    unsigned char* park = lds_raw + (size_t)wave * (S::WM * ROW_BYTES);
    const int n_wave = bn0 + wn0;
    auto park_piece = [&](auto bias_tag, auto relu_tag) {      // one instance per combination, chosen by scalar branches
        constexpr bool BIAS = decltype(bias_tag)::value, RELU = decltype(relu_tag)::value;
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (BIAS) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int n = n_wave + 16 * ni + 4 * lg + e;
                    bv[e] = n < N ? (float)out.bias[n] : 0.f;
                }
            }
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                const int row = 16 * mi + li, col = 16 * ni + 4 * lg;
                f32x4v v = acc[mi][ni];
                if (BIAS) {                                     // (adding 0 would turn -0 into +0)
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] += bv[e];
                }
                if (RELU) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = relu_by_sign(v[e]);
                }
                const f16x4 h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
                const int piece = col >> 3;
                *reinterpret_cast<u32x2*>(park + row * ROW_BYTES + ((piece ^ (row & 7)) << 4) + ((lg & 1) << 3)) = __builtin_bit_cast(u32x2, h);
            }
        }
    };
    typedef std::integral_constant<bool, false> No;
    typedef std::integral_constant<bool, true> Yes;
    if (out.bias != nullptr) {
        if (out.relu) park_piece(Yes{}, Yes{});
        else park_piece(Yes{}, No{});
    } else {
        if (out.relu) park_piece(No{}, Yes{});
        else park_piece(No{}, No{});
    }
    // the wave reads back what it wrote itself: LDS operations of a wave complete in order, no barrier needed
    const bool vec = out.dpitch % 8 == 0 && out.row_stride % 8 == 0 && (reinterpret_cast<size_t>(out.dst) & 15) == 0;
    static_assert(ROWS_PER_PASS == 8 && S::PATCH_Y == 16 && S::WM % 16 == 0, "a pass is the upper or the lower half of one image column of the patch");
    if (vec && y0 + S::PATCH_Y <= Hout && x0 + S::PATCH_X <= out.Wout && bn0 + BN <= N) {
        // a patch that lies inside the output as a whole (one scalar test): no checks around the stores, and the address
        // moves from pass to pass by one of two wave-uniform steps -- 8 rows down, or up again and one column on
        const int row0 = lane / PIECES, piece = lane % PIECES;
        _Float16* dp = out.dst + (size_t)(y0 + row0) * out.row_stride + (size_t)(x0 + wm0 / S::PATCH_Y) * out.dpitch + n_wave + 8 * piece;
        const ptrdiff_t down = (ptrdiff_t)(8 * out.row_stride), over = (ptrdiff_t)out.dpitch - down;
        const unsigned char* src = park + row0 * ROW_BYTES + ((piece ^ row0) << 4);
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(src + pass * ROWS_PER_PASS * ROW_BYTES);
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dp));      // written once, not read by this launch
            dp += (pass & 1) ? over : down;
        }
        return;
    }
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
        const int row = pass * ROWS_PER_PASS + lane / PIECES, piece = lane % PIECES;
        const u32x4 v = *reinterpret_cast<const u32x4*>(park + row * ROW_BYTES + ((piece ^ (row & 7)) << 4));
        const int r = wm0 + row, y = y0 + r % S::PATCH_Y, x = x0 + r / S::PATCH_Y, n = n_wave + 8 * piece;
        if (y < Hout && x < out.Wout && n < N) {
            _Float16* dp = out.dst + (size_t)y * out.row_stride + (size_t)x * out.dpitch + n;
            if (vec && n + 8 <= N) {
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dp));
            } else {
                const f16x8 h = __builtin_bit_cast(f16x8, v);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (n + e < N) dp[e] = h[e];
            }
        }
    }
}

}  // namespace decx_hip
