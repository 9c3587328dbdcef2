// fp16-in / fp32-accumulate tile on v_mfma_f32_16x16x32_f16, fed by the LDS-DMA pipeline of hgemm_dma_tile.hpp.
//
// Why another MFMA shape: on real-valued operands the chip runs the fp16 matrix pipe against its power limit, not its
// issue rate (an MFMA-only loop reaches 2.45 PFLOP/s on all-zero registers and 1.67 on uniform[-1,1] ones with
// v_mfma_f32_32x32x16_f16 -- and 1.90-1.93 with v_mfma_f32_16x16x32_f16, which sums 32 products per accumulator access
// instead of 16).  Everything around the instruction is kept: 256 x 256 x 64 tile, 8 waves of 128 x 64 (two per SIMD),
// two LDS stages filled by global_load_lds_dwordx4, 16-byte units XOR-swizzled on the global side.
//
// What is new besides the instruction:
//   * LDS keeps the stages of one operand next to each other ([A0][A1][B0][B1]) and the K walk is unrolled over the two
//     stages, so that stage, k-block and row block of a fragment read are compile-time constants that fold into the
//     instruction's offset field: no address arithmetic between the MFMAs.
//   * The B swizzle also moves rows 8 apart (the four 16-lane groups of a transposing read fetch rows 8g .. 8g+3 of
//     the same columns) onto different banks.
//   * The matrix B fragment is the MFMA's first operand and the matrix A fragment its second: the accumulators then hold
//     the tile transposed, i.e. a lane owns 4 CONSECUTIVE COLUMNS of one row.  The epilogue rounds them to binary16,
//     parks the wave's 128 x 64 piece in LDS (the operand buffers are free by then) and writes it out as 16-byte
//     pieces, 128 contiguous bytes per row.
//   * A K step is cut into four units of 16 MFMAs (k-block x half of the wave's rows); a unit's fragments are fetched
//     during the unit before it, which keeps 2 x (4 A + 4 B) fragments in registers instead of 2 x (8 + 4).
// Needs 16-byte aligned A, B with lda, ldb multiples of 8, like the other LDS-DMA tiles.
#pragma once
#include "hgemm_dma_tile.hpp"

namespace decx_hip {

typedef float f32x4v __attribute__((ext_vector_type(4)));

// B unit (k, u) of a stage: as b_unit_slot, plus bit 1 of the unit index flipped for odd k / 8
__device__ __forceinline__ int b16_unit_slot(int k, int u, int UB) {
    return k * UB + (u ^ (((k & 3) << 2) | (((k >> 3) & 1) << 1)));
}

// A unit (m, q) of a stage with 4 units per row (BK = 32): the unit index rotated by 2 (m / 4), which keeps the fragment
// reads of 16-row blocks (lane group lg takes unit lg of rows m .. m + 15) on distinct banks in every service phase of a
// 16-byte LDS read.  With 8 units per row (BK = 64) the XOR swizzle of hgemm_tile.hpp already does.
__device__ __forceinline__ int a16_unit_slot(int m, int q, int UA) {
    return UA == 4 ? m * 4 + ((q + 2 * (m >> 2)) & 3) : a_unit_slot(m, q, UA);
}
// the unit that lands in slot s of row m (inverse of the above, for the global side of the DMA)
__device__ __forceinline__ int a16_unit_in_slot(int m, int s, int UA) {
    return UA == 4 ? ((s - 2 * (m >> 2)) & 3) : (s ^ ((m / (16 / UA)) % UA));
}

// dma_load16 with a tag in the instruction text.  Two branches of a dispatch that issue the same loads into different
// stages are otherwise merged by the compiler into one sequence whose operands are selected per branch -- in vector
// registers, which the scalar operands of this instruction do not accept.
template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_>
struct Hgemm16Shape {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, STAGES = STAGES_;
    static constexpr int NWAVES = WAVES_M * WAVES_N, NT = NWAVES * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 16, NI = WN / 16;            // 16 x 16 accumulator blocks of a wave
    static constexpr int MH = 2, UM = MI / MH;                  // a unit = one k-block x UM row blocks
    static constexpr int KS = BK / 32, UNITS = KS * MH;
    static constexpr int UA = BK / 8, UB = BN / 8;              // 16-byte units per LDS row
    static constexpr int A_UNITS = BM * UA, B_UNITS = BK * UB;
    static constexpr int A_BYTES = A_UNITS * 16, B_BYTES = B_UNITS * 16;
    static constexpr size_t LDS_BYTES = (size_t)STAGES * (A_BYTES + B_BYTES);
    // the many-tiles-per-workgroup build parks results in chunks of PARK_ROWS rows per wave behind the stages
    static constexpr int PARK_ROWS = 32;
    static constexpr size_t PERSIST_LDS_BYTES = LDS_BYTES + (size_t)WAVES_M_ * WAVES_N_ * PARK_ROWS * (BN_ / WAVES_N_) * 2;
    static constexpr int A_LOADS = A_UNITS / 64 / NWAVES, B_LOADS = B_UNITS / 64 / NWAVES, LOADS = A_LOADS + B_LOADS;
    static constexpr int A_PASSES = A_UNITS / NT, B_PASSES = B_UNITS / NT;
    static_assert(BK == 32 || BK == 64, "one or two k-blocks of 32 per K step");
    static_assert(MI % MH == 0 && UNITS % 2 == 0, "fragment sets of A alternate by unit");
    // fragment sets of B alternate by k-block, so the unrolled walk covers the stages once or (odd count of k-blocks) twice
    static constexpr int WALK = (STAGES * KS) % 2 == 0 ? STAGES : 2 * STAGES;
    static_assert(STAGES >= 2, "need at least double buffering");
    static_assert(UB >= 16 && (UB & (UB - 1)) == 0, "the B swizzle needs >= 16 units per row");
    static_assert(A_UNITS % (64 * NWAVES) == 0 && B_UNITS % (64 * NWAVES) == 0, "DMA chunks must divide over the waves");
    static_assert((size_t)NWAVES * WM * WN * 2 <= LDS_BYTES, "the epilogue parks every wave's piece in LDS");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS of a CU");
    // fragment reads address stage, k-block and row block through the 16-bit offset field, from one of two per-lane bases
    // (the second one HI_STAGE stages further on) when the stages of an operand span more than 64 KB
    static constexpr int HI_STAGE = (STAGES + 1) / 2;
    static_assert((HI_STAGE - 1) * A_BYTES + (MI - 1) * 16 * UA * 16 < 65536 && (HI_STAGE - 1) * B_BYTES + (32 * (KS - 1) + 4) * UB * 16 < 65536,
                  "offsets from a base must fit 16 bits");
    static_assert(LOADS * (STAGES - 2) <= 63, "vmcnt is a 6-bit counter");
};

// ABLATE != 0 builds measurement variants that leave work out of the K walk and produce no meaningful result (the cost of
// each part of the kernel is the difference between two of them): bit 0 = the K walk issues no DMA loads (LDS keeps
// the first two K steps), bit 1 = it issues no LDS reads (the registers keep the first fragments), bit 2 = the result
// is not stored, bit 3 = the loads of the K walk never move on (every step fetches the tile's first K step again, which
// the caches then hold: the loads without their misses).  Bits 4-5 pick the order of the 16 matrix instructions of a
// unit: 0 = row block by row block with the column order reversed on every other one, so that exactly one operand
// changes between any two instructions of a k-block (the product's order: on uniform[-1,1] operands the matrix pipe
// draws measurably less power than when both operands change at every row block, and the chip clocks 2 % higher);
// 1 = row block by row block, columns always ascending; 2 = column block by column block (the B fragment stays).
// The sums do not depend on the order: every accumulator sees its k-blocks ascending.  Only the probe library
// launches variants with any of these bits set.
//
// PERSIST: the grid holds one workgroup per compute unit and a workgroup walks the tiles blockIdx.x, blockIdx.x +
// gridDim.x, ... as one stream of K steps: the loads that refill the stages during a tile's last STAGES steps fetch the
// first steps of the next tile (where the one-tile kernel repeats the last step), so no tile after the first has a
// prologue, and the epilogue -- through a parking area of its own behind the stages, 4 KB per wave -- runs while
// those loads are in flight.  For whole tiles only: M % BM == 0, N % BN == 0, K % (BK * WALK) == 0, K >= BK * STAGES,
// one problem per launch (the host checks).
template <class S, bool HAS_C, int ABLATE = 0, bool PERSIST = false>
__global__ __launch_bounds__(S::NT) void hgemm_mfma16_kernel(const _Float16* __restrict__ A, int lda,
                                                             const _Float16* __restrict__ B, int ldb, const _Float16* Cin,
                                                             int ldc, _Float16* D, int ldd, int M, int N, int K, int tiles_m,
                                                             int tiles_n, int group_m, size_t a_batch_stride,
                                                             size_t b_batch_stride, size_t c_batch_stride, size_t d_batch_stride) {
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, NT = S::NT, UA = S::UA, UB = S::UB, MI = S::MI, NI = S::NI;
    constexpr int UM = S::UM, MH = S::MH, KS = S::KS, UNITS = S::UNITS, STAGES = S::STAGES, WALK = S::WALK;
    constexpr int A_BYTES = S::A_BYTES, B_BYTES = S::B_BYTES;
    constexpr int BLK = UM * NI;                                // MFMAs per unit
    constexpr int ORDER = (ABLATE >> 4) & 3;
    A += (size_t)blockIdx.y * a_batch_stride;
    B += (size_t)blockIdx.y * b_batch_stride;
    if (HAS_C) Cin += (size_t)blockIdx.y * c_batch_stride;
    D += (size_t)blockIdx.y * d_batch_stride;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];   // [A stages][B stages]
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw;

    const int total_tiles = tiles_m * tiles_n;
    int tile = blockIdx.x;
    const TileCoord tc = xcd_grouped_tile(tile, tiles_m, tiles_n, group_m);
    int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int lg = lane >> 4, li = lane & 15;                   // 16-lane group = k sub-block, lane in group = row / column

    // ---- DMA sources: wave-uniform bases that advance by one K step per fetched step + loop-invariant lane offsets
    const int m_first = bm0 < M ? bm0 : M - 1;
    const _Float16* a_base = A + (size_t)m_first * lda;
    const _Float16* b_base = PERSIST ? B + bn0 : B;              // PERSIST: lane offsets are the same for every (whole) tile
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int chunk = wave * S::A_LOADS + j;                // 64 units = 64 / UA rows
        const int r = chunk * (64 / UA) + lane / UA;
        const int q = a16_unit_in_slot(r, lane % UA, UA);       // the unit whose swizzled slot is this lane
        int m = bm0 + r;
        if (m >= M) m = M - 1;                                  // rows past the end are computed and never stored
        a_off[j] = (uint32_t)(((size_t)(m - m_first) * lda + 8 * q) * sizeof(_Float16));
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int chunk = wave * S::B_LOADS + j;                // 64 units = 64 / UB k-rows
        const int kr = chunk * (64 / UB) + lane / UB;
        const int u = (lane % UB) ^ (((kr & 3) << 2) | (((kr >> 3) & 1) << 1));
        const int col = PERSIST ? 8 * u : clamp_group_col(bn0 + 8 * u, N, 8);     // stay inside the operand; such columns are never stored
        b_off[j] = (uint32_t)(((size_t)kr * ldb + col) * sizeof(_Float16));
    }
    // Every K step fetches the step STAGES ahead of it into the stage it leaves, also the last STAGES, which have nothing
    // left to fetch: their loads repeat the last whole step (the bases stop there) into stages nobody reads again.  All
    // steps are then the same code with the same wait counts, at the price of STAGES redundant step loads per tile.
    const int full_steps = K / BK;
    int steps_fetched = 0;
    const size_t b_step = (size_t)BK * ldb;
    // PERSIST: where the fetches go on once the current tile's steps are all out (set before each tile's walk)
    const _Float16* a_next = a_base;
    const _Float16* b_next = b_base;
    bool has_next = false;
    auto plan_next_tile = [&]() {
        const int nt = tile + (int)gridDim.x;
        has_next = nt < total_tiles;
        const TileCoord nc = xcd_grouped_tile(has_next ? nt : tile, tiles_m, tiles_n, group_m);
        a_next = A + (size_t)(nc.tm * BM) * lda;
        b_next = B + nc.tn * BN;
    };
    if constexpr (PERSIST) plan_next_tile();
    auto issue_one = [&](auto stage_tag, auto j_tag, auto in_walk_tag) {
        constexpr int STG = decltype(stage_tag)::value, J = decltype(j_tag)::value;
        if constexpr ((ABLATE & 1) && decltype(in_walk_tag)::value) return;
        if constexpr (J < S::A_LOADS) {
            dma_load16_tagged<STG * 64 + J>(a_base, a_off[J], lds_base + (uint32_t)(STG * A_BYTES) + (uint32_t)(wave * S::A_LOADS + J) * 1024u);
        } else {
            constexpr int JB = J - S::A_LOADS;
            dma_load16_tagged<STG * 64 + J>(b_base, b_off[JB], lds_base + (uint32_t)(STAGES * A_BYTES + STG * B_BYTES) + (uint32_t)(wave * S::B_LOADS + JB) * 1024u);
        }
        if constexpr (J == S::LOADS - 1 && !(ABLATE & 8)) {
            ++steps_fetched;
            const bool more = steps_fetched < full_steps;        // scalar: the next fetch is a new step of this tile
            if constexpr (PERSIST) {
                const bool wrap = !more && has_next && steps_fetched == full_steps;      // ... or the first of the next
                a_base = more ? a_base + BK : (wrap ? a_next : a_base);
                b_base = more ? b_base + b_step : (wrap ? b_next : b_base);
                steps_fetched = wrap ? 0 : (more ? steps_fetched : full_steps);
            } else {
                a_base += more ? BK : 0;
                b_base += more ? b_step : (size_t)0;
            }
        }
    };

    f32x4v acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4v{0.f, 0.f, 0.f, 0.f};

    // ---- fragment reads: per-lane byte offsets inside stage 0; stage, k-block, row block and the low / high half of a
    // transposing read are constants added in the instruction
    //   A fragment of row block rb, k-block kb : lane (lg, li) reads the 8 halves k = 32 kb + 8 lg .. + 7 of row 16 rb + li
    //   B fragment of column block ni, k-block kb: two transposing reads of 4 rows each; lane (lg, li) supplies the address
    //     of row 32 kb + 8 lg + li / 4 (+ 4), columns 16 ni + 4 (li % 4) .. + 3, and receives column 16 ni + li of 4 rows
    constexpr int HI = S::HI_STAGE;
    constexpr bool TWO_BASES = (STAGES - 1) * A_BYTES + (MI - 1) * 16 * UA * 16 >= 65536 || (STAGES - 1) * B_BYTES + (32 * (KS - 1) + 4) * UB * 16 >= 65536;
    uint32_t a_rd[KS], b_rd[NI], a_rd_hi[KS], b_rd_hi[NI];
#pragma unroll
    for (int kb = 0; kb < KS; ++kb) {
        a_rd[kb] = (uint32_t)a16_unit_slot(wm0 + li, 4 * kb + lg, UA) * 16u;
        a_rd_hi[kb] = a_rd[kb] + (uint32_t)(HI * A_BYTES);
    }
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int col = wn0 + 16 * ni + 4 * (li & 3);
        b_rd[ni] = (uint32_t)(STAGES * A_BYTES) + (uint32_t)b16_unit_slot(8 * lg + (li >> 2), col >> 3, UB) * 16u + (uint32_t)(col & 7) * 2u;
        b_rd_hi[ni] = b_rd[ni] + (uint32_t)(HI * B_BYTES);
    }
    static_assert(UA == 4 || (16 % (16 / UA) == 0 && (16 / (16 / UA)) % UA == 0), "row blocks of 16 must not change the A swizzle");
    typedef short i16x8 __attribute__((ext_vector_type(8)));
    f16x8 af[2][UM];                                            // by unit parity
    i16x4 blo[2][NI], bhi[2][NI];                               // by the parity of the k-block counted over the whole walk
    if constexpr (ABLATE & 2) {
#pragma unroll
        for (int x = 0; x < NI; ++x) blo[0][x] = blo[1][x] = bhi[0][x] = bhi[1][x] = i16x4{0, 0, 0, 0};
    }
    auto read_a = [&](auto set_tag, auto slot_tag, auto stage_tag, auto kb_tag, auto rb_tag) {
        constexpr int STG = decltype(stage_tag)::value;
        constexpr bool HIGH = TWO_BASES && STG >= HI;
        constexpr int OFF = (HIGH ? STG - HI : STG) * A_BYTES + decltype(rb_tag)::value * (16 * UA * 16);
        const uint32_t base = HIGH ? a_rd_hi[decltype(kb_tag)::value] : a_rd[decltype(kb_tag)::value];
        af[decltype(set_tag)::value][decltype(slot_tag)::value] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(lds_raw + base + OFF));
    };
    auto read_b = [&](auto set_tag, auto stage_tag, auto kb_tag, auto ni_tag, auto hi_tag) {
        constexpr int SET = decltype(set_tag)::value, NIX = decltype(ni_tag)::value, HALF = decltype(hi_tag)::value;
        constexpr int STG = decltype(stage_tag)::value;
        constexpr bool HIGH = TWO_BASES && STG >= HI;
        constexpr int OFF = (HIGH ? STG - HI : STG) * B_BYTES + (32 * decltype(kb_tag)::value + 4 * HALF) * (UB * 16);
        const uint32_t base = HIGH ? b_rd_hi[NIX] : b_rd[NIX];
        const i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(lds_raw + base + OFF));
        if constexpr (HALF) bhi[SET][NIX] = v;
        else blo[SET][NIX] = v;
    };
    // The walk is unrolled over WALK steps; step V of it works in stage V % STAGES, and k-block KB of it uses B fragment set
#define DECX_BSET(V, KB) (((V) * KS + (KB)) & 1)
    // read number R of the fragments a K step in stage STG starts with (unit 0: row blocks 0 .. UM-1, k-block 0), in the
    // order its first MFMAs need them: A block 0, all of B, the other A blocks
    constexpr int FIRST_READS = UM + 2 * NI;
    auto read_first = [&](auto v_tag, auto r_tag) {
        constexpr int R = decltype(r_tag)::value, V = decltype(v_tag)::value;
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, V % STAGES> Stg;
        typedef std::integral_constant<int, DECX_BSET(V, 0)> BSet;
        if constexpr (R == 0) read_a(I0{}, I0{}, Stg{}, I0{}, I0{});
        else if constexpr (R <= 2 * NI)
            read_b(BSet{}, Stg{}, I0{}, std::integral_constant<int, (R - 1) / 2>{}, std::integral_constant<int, (R - 1) % 2>{});
        else read_a(I0{}, std::integral_constant<int, R - 2 * NI>{}, Stg{}, I0{}, std::integral_constant<int, R - 2 * NI>{});
    };
    // MFMA number I of unit U of walk step V: row block (U % MH) * UM + I / NI, column block I % NI
    auto mfma_one = [&](auto v_tag, auto u_tag, auto i_tag) {
        constexpr int U = decltype(u_tag)::value, I = decltype(i_tag)::value;
        constexpr int ROWB = ORDER == 2 ? I % UM : I / NI;                              // row block within the unit
        constexpr int NIX = ORDER == 2 ? I / UM : (ORDER == 0 && (ROWB & 1) ? NI - 1 - I % NI : I % NI);
        constexpr int KB = U / MH, MIX = (U % MH) * UM + ROWB, BS = DECX_BSET(decltype(v_tag)::value, KB);
        const i16x4 lo = blo[BS][NIX], hi = bhi[BS][NIX];
        const i16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        acc[MIX][NIX] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, both), af[U & 1][ROWB], acc[MIX][NIX], 0, 0, 0);
    };
#define DECX_PIN() __builtin_amdgcn_sched_barrier(0)

    // One K step from stage STG.  On entry af[0] and the B set of its first k-block hold the fragments of unit 0; on exit
    // those of the next step.  Units 0 .. UNITS-2: the first MFMAs each carry one LDS read of the next unit's A fragments
    // and of this unit's share of the next k-block's B fragments.  Last unit: a few MFMAs, then wait for the next step's
    // data + barrier -- nobody reads this stage any more -- and between the remaining MFMAs the DMA refill of this stage
    // (the loads of the STAGES - 2 steps in between may still be in flight at the wait) and the first fragments of the
    // next step from the next stage.
    auto k_step = [&](auto v_tag) {
        constexpr int V = decltype(v_tag)::value, STG = V % STAGES;
        typedef std::integral_constant<int, STG> Stg;
        typedef std::integral_constant<int, (V + 1) % WALK> Next;
        static_for<0, UNITS - 1>([&](auto u_tag) {
            constexpr int U = decltype(u_tag)::value, KB = U / MH, H = U % MH;
            constexpr int NU = U + 1, NKB = NU / MH, NH = NU % MH;
            constexpr int NB = (KB + 1 < KS) ? 2 * NI / MH : 0;          // B reads of the next k-block in this unit
            constexpr int NR = UM + NB;
            static_assert(NR <= BLK, "one read per MFMA slot");
            static_for<0, BLK>([&](auto i_tag) {
                constexpr int I = decltype(i_tag)::value;
                if constexpr (ABLATE & 2) {
                } else if constexpr (I < UM) {
                    read_a(std::integral_constant<int, NU & 1>{}, i_tag, Stg{}, std::integral_constant<int, NKB>{},
                           std::integral_constant<int, NH * UM + I>{});
                } else if constexpr (I < NR) {
                    constexpr int RB = H * NB + (I - UM);
                    read_b(std::integral_constant<int, DECX_BSET(V, KB + 1)>{}, Stg{}, std::integral_constant<int, KB + 1>{},
                           std::integral_constant<int, RB / 2>{}, std::integral_constant<int, RB % 2>{});
                }
                mfma_one(v_tag, u_tag, i_tag);
                DECX_PIN();
            });
        });
        typedef std::integral_constant<int, UNITS - 1> Last;
        constexpr int PRE = BLK / 4, SLOTS = BLK - PRE;
        static_for<0, PRE>([&](auto i_tag) {
            mfma_one(v_tag, Last{}, i_tag);
            DECX_PIN();
        });
        // loads of this wave that may still be in flight when it meets the others: those of the STAGES - 2 steps after the next
        constexpr int WAITN = (ABLATE & 1) ? 0 : S::LOADS * (STAGES - 2);
        wait_dma_then_barrier<WAITN>();
        DECX_PIN();
        static_for<0, SLOTS>([&](auto i_tag) {
            constexpr int I = decltype(i_tag)::value;
            static_for<(I * S::LOADS) / SLOTS, ((I + 1) * S::LOADS) / SLOTS>([&](auto j_tag) { issue_one(Stg{}, j_tag, std::true_type{}); });
            // two reads per slot until they are all out: the next step's first MFMAs follow closely
            constexpr int R0 = 2 * I < FIRST_READS ? 2 * I : FIRST_READS, R1 = 2 * I + 2 < FIRST_READS ? 2 * I + 2 : FIRST_READS;
            if constexpr (!(ABLATE & 2)) static_for<R0, R1>([&](auto r_tag) { read_first(Next{}, r_tag); });
            mfma_one(v_tag, Last{}, std::integral_constant<int, PRE + I>{});
            DECX_PIN();
        });
    };

    typedef std::integral_constant<int, 0> I0;
    bool first_tile = true;                                     // PERSIST: later tiles find their first steps fetched already
    for (;;) {
    if (full_steps > 0) {
        // The walk starts at walk step `first` such that it ends with step WALK - 1: a first pass that begins at `first`,
        // then whole passes.  The prologue fills all stages, K step j into stage (first + j) % STAGES.
        const int first = PERSIST ? 0 : (WALK - full_steps % WALK) % WALK;
        if (first_tile) {
            static_for<0, WALK>([&](auto v0) {
                if (first == decltype(v0)::value) {
                    static_for<0, STAGES>([&](auto j) {
                        typedef std::integral_constant<int, (decltype(v0)::value + decltype(j)::value) % STAGES> Stg;
                        static_for<0, S::LOADS>([&](auto l) { issue_one(Stg{}, l, std::false_type{}); });
                    });
                    wait_dma_then_barrier<S::LOADS*(STAGES - 1)>();          // step 0 has landed
                    static_for<0, FIRST_READS>([&](auto r) { read_first(v0, r); });
                }
            });
            DECX_PIN();
            if constexpr (ABLATE & 2) {                              // the sets the walk would have filled
#pragma unroll
                for (int x = 0; x < UM; ++x) af[1][x] = af[0][x];
#pragma unroll
                for (int x = 0; x < NI; ++x) {
                    const i16x4 lo = blo[0][x] | blo[1][x], hi = bhi[0][x] | bhi[1][x];      // whichever set was read
                    blo[0][x] = blo[1][x] = lo;
                    bhi[0][x] = bhi[1][x] = hi;
                }
            }
        }
        // the first pass skips the walk steps before `first` (a scalar branch around each step)
        int skip = first;
        for (int t = -first; t < full_steps; t += WALK) {
            static_for<0, WALK>([&](auto v) {
                if (decltype(v)::value >= skip) k_step(v);
            });
            skip = 0;
        }
    }

    // ---- partial last K step: through registers into stage 0 (zero-filled beyond K), then all of its units
    if (!PERSIST && full_steps * BK < K) {
        const int k0 = full_steps * BK;
        u32x4 a_stage[S::A_PASSES], b_stage[S::B_PASSES];
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) {
            const int id = tid + p * NT;
            const int r = id / UA, q = id % UA;
            int m = bm0 + r;
            if (m >= M) m = M - 1;
            const int k = k0 + 8 * q;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (k < K) {
                v = *reinterpret_cast<const u32x4*>(A + (size_t)m * lda + k);
                const int keep = K - k;
                if (keep < 8) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) v[w] &= (2 * w + 1 < keep) ? 0xffffffffu : (2 * w < keep ? 0x0000ffffu : 0u);
                }
            }
            a_stage[p] = v;
        }
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) {
            const int id = tid + p * NT;
            const int kr = id / UB, u = id % UB;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (k0 + kr < K) v = *reinterpret_cast<const u32x4*>(B + (size_t)(k0 + kr) * ldb + clamp_group_col(bn0 + 8 * u, N, 8));
            b_stage[p] = v;
        }
        wait_dma_then_barrier<0>();                             // everybody is done with every buffer
        u32x4* Ab = reinterpret_cast<u32x4*>(lds_raw);
        u32x4* Bb = reinterpret_cast<u32x4*>(lds_raw + STAGES * A_BYTES);
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) {
            const int id = tid + p * NT;
            Ab[a16_unit_slot(id / UA, id % UA, UA)] = a_stage[p];
        }
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) {
            const int id = tid + p * NT;
            Bb[b16_unit_slot(id / UB, id % UB, UB)] = b_stage[p];
        }
        __syncthreads();
        static_for<0, UNITS>([&](auto u_tag) {
            constexpr int U = decltype(u_tag)::value, KB = U / MH, H = U % MH;
            static_for<0, UM>([&](auto r) {
                read_a(std::integral_constant<int, U & 1>{}, r, I0{}, std::integral_constant<int, KB>{},
                       std::integral_constant<int, H * UM + decltype(r)::value>{});
            });
            if constexpr (H == 0)
                static_for<0, 2 * NI>([&](auto r) {
                    read_b(std::integral_constant<int, DECX_BSET(0, KB)>{}, I0{}, std::integral_constant<int, KB>{},
                           std::integral_constant<int, decltype(r)::value / 2>{}, std::integral_constant<int, decltype(r)::value % 2>{});
                });
            static_for<0, BLK>([&](auto i_tag) { mfma_one(I0{}, u_tag, i_tag); });
        });
    }

    // ---- epilogue.  acc[mi][ni][e] is element (row 16 mi + li, column 16 ni + 4 lg + e) of the wave's piece.  dst = A*B + C
    // adds C in fp32; one rounding to binary16; the piece goes to LDS in chunks of CH_ROWS rows (rows of WN halves, 16-byte
    // pieces XOR-swizzled by the row) and leaves as 16-byte stores.  One chunk in the operand buffers, which are free by
    // then; PERSIST: chunks of 32 rows in the wave's own 4 KB behind the stages, which are being refilled meanwhile.
    if constexpr (!PERSIST) wait_dma_then_barrier<0>();         // nobody reads operands any more, and the last (redundant) stage loads have landed
    constexpr int ROW_BYTES = S::WN * 2, PIECES = S::WN / 8, ROWS_PER_PASS = kWave / PIECES;
    constexpr int CH_ROWS = PERSIST ? S::PARK_ROWS : S::WM, CHUNKS = S::WM / CH_ROWS, PASSES = CH_ROWS / ROWS_PER_PASS;
    static_assert(PIECES >= 8 && (PIECES & (PIECES - 1)) == 0 && kWave % PIECES == 0, "piece swizzle");
    static_assert(CH_ROWS % 16 == 0 && S::WM % CH_ROWS == 0 && CH_ROWS % ROWS_PER_PASS == 0, "chunks of whole row blocks");
    unsigned char* park = PERSIST ? lds_raw + S::LDS_BYTES + (size_t)wave * (CH_ROWS * ROW_BYTES) : lds_raw + (size_t)wave * (S::WM * ROW_BYTES);
    const int m_wave = bm0 + wm0, n_wave = bn0 + wn0;
    // the wave reads back what it wrote itself: LDS operations of a wave complete in order, no barrier needed
    const bool vec_d = ((reinterpret_cast<uintptr_t>(D) | (uintptr_t)(ldd * 2)) & 15) == 0;
    const bool whole = bm0 + BM <= M && bn0 + BN <= N && vec_d;     // one scalar test instead of checks around every store
#pragma unroll
    for (int ch = 0; ch < CHUNKS; ++ch) {
#pragma unroll
        for (int mc = 0; mc < CH_ROWS / 16; ++mc)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int mi = ch * (CH_ROWS / 16) + mc;
                const int row = 16 * mc + li, col = 16 * ni + 4 * lg;           // row within the chunk
                f32x4v v = acc[mi][ni];
                if (HAS_C) {
                    const int m = m_wave + ch * CH_ROWS + row, n = n_wave + col;
                    if (m < M) {
                        const _Float16* crow = Cin + (size_t)m * ldc + n;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (n + e < N) v[e] += (float)crow[e];
                    }
                }
                const f16x4 h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
                const int piece = col >> 3;
                *reinterpret_cast<u32x2*>(park + row * ROW_BYTES + ((piece ^ (row & 7)) << 4) + ((lg & 1) << 3)) = __builtin_bit_cast(u32x2, h);
            }
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const int row = pass * ROWS_PER_PASS + lane / PIECES, piece = lane % PIECES;
            const u32x4 v = *reinterpret_cast<const u32x4*>(park + row * ROW_BYTES + ((piece ^ (row & 7)) << 4));
            const int m = m_wave + ch * CH_ROWS + row, n = n_wave + 8 * piece;
            _Float16* dp = D + (size_t)m * ldd + n;
            if ((ABLATE & 4) && K >= 0) continue;                    // (a condition the compiler cannot fold, so the sums stay live)
            if (whole) {
                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dp));      // written once, not read by this launch
            } else if (m < M) {
                if (vec_d && n + 8 <= N) {
                    *reinterpret_cast<u32x4*>(dp) = v;
                } else {
                    const f16x8 h = __builtin_bit_cast(f16x8, v);
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (n + e < N) dp[e] = h[e];
                }
            }
        }
    }
    if constexpr (!PERSIST) {
        break;
    } else {
        if (!has_next) break;
        tile += (int)gridDim.x;
        const TileCoord nc = xcd_grouped_tile(tile, tiles_m, tiles_n, group_m);
        bm0 = nc.tm * BM;
        bn0 = nc.tn * BN;
        plan_next_tile();
        first_tile = false;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = f32x4v{0.f, 0.f, 0.f, 0.f};
    }
    }   // tiles of this workgroup
    // PERSIST: the loads of the last steps (repeats, nobody reads them) must have landed before the workgroup gives up its LDS
    if constexpr (PERSIST) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#undef DECX_BSET
#undef DECX_PIN
}

}  // namespace decx_hip
