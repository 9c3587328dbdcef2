// fp32 GEMM for results of a few tiles per CU (1024^3: 256 tiles of 64x64 on 256 CUs): operands go from global memory
// straight into LDS, and nothing but matrix instructions and their operand reads runs on the computing waves.
//
// A workgroup is four waves, one per SIMD, each owning MI x NI blocks of 32x32.  With one 64x64 tile per CU that is ONE
// block per wave = one dependent chain of v_mfma_f32_32x32x2_f32 (64 cycles each), and every other instruction the SIMD
// has to issue delays that chain.  The
// register-staged kernels spend a global load, two LDS stores and their address arithmetic per 16 bytes of operand;
// measured on the block-chain kernel at this size, the staging costs a quarter of the matrix pipe's time.  Here a
// global_load_lds_dwordx4 moves 16 bytes per lane into LDS with no register, no LDS store and no wait on the wave's
// side: 4 such loads per wave and K step of 32 on the 64x64 tile, against 16 MFMAs.
//
// The price is that LDS holds the operands as they lie in memory, and a lane of the 32x32x2 instruction wants ONE
// float per operand and instruction: lane (i, s), i = 0..31, s = 0..1, feeds A[i][2j + s] and B[2j + s][i] to MFMA j.
//   B [k][64 columns]: 32 lanes read 32 consecutive floats of row 2j + s -- conflict-free; rows 2j+s and 2j+2+s of
//     two successive MFMAs come with one ds_read2st64_b32.
//   A [row][k]: a 16-byte unit holds k = 4q .. 4q+3 of a row, i.e. the operands of MFMAs 2q and 2q+1 for both s: lane
//     (i, s) reads floats s and s + 2 of it with one ds_read2_b32.  Unit q of row r sits in slot q ^ (r % 8) of the
//     row, so that the 32 rows of a read spread over all banks (each bank four times -- one float per lane and unit
//     allows no less).  The swizzle is applied on the global side: the lane whose LDS place is slot t of row r fetches
//     unit t ^ (r % 8).
// One LDS read per MFMA in all on the 64x64 tile (wave blocks of 2x2 re-use each operand twice: one read per two MFMAs,
// and four interleaved chains), issued right behind it.
//
// The same kernel on 16x16 blocks (v_mfma_f32_16x16x4_f32: four k per instruction, 32 cycles, so a chain walks K twice
// as fast) serves results with fewer than four 32x32 blocks per CU, and results whose 64x64 tiles fill the last round of
// CUs badly.  Lane (i, s), i = 0..15, s = 0..3, feeds A[i][4j + s] and B[4j + s][i] to MFMA j: float s of unit j of its row
// of A -- ONE ds_read_b32 per MFMA, the 16 rows of a read in 8 different slots, so every bank serves two lanes, which is
// all 64 lanes on 32 banks can have; reading two units with one ds_read2_b32 ties the slots of a row to pairs, leaves
// four lanes on a bank, and with four waves reading made the LDS the bound (384x8192x384: 41.4 us against 32.9) -- and
// 16 consecutive floats of row 4j + s of B, where the units of odd rows swap halves of 32 columns so that the four rows
// of a read cover all banks twice; rows 4j + s and 4j + 4 + s again come with one read.
//
// Pipeline: STAGES LDS buffers, one barrier per K step.  The step is computed in two halves from two fragment sets:
// during the first half the second half's fragments are read; the second half starts with the barrier (before it the
// wave waits for its own loads of step t+1, after it nobody reads step t's buffer any more), then issues the loads of
// step t+STAGES into that buffer and reads the first half of step t+1, all between its MFMAs.  Loads never run past
// the last whole step: the source pointers stop there (later refills fetch that step again and are never read), which
// keeps every step the same code with the same wait counts.  The walk is whole passes over the buffers, unrolled and free
// of branches, then the steps that are left behind a test each; the loads of the two copies carry different tags in
// their text (dma_load16_tagged), without which the compiler merges them and does not assemble.  A ragged last step (K % BK) is staged through registers
// with zeros past K and only the MFMAs that hold a k < K are issued.
//
// Arithmetic: per output one fused multiply-add chain over ascending k -- slot 0 then slot 1 inside an instruction,
// instructions in order -- exactly the chain of sgemm_tile_kernel and of the reference.
// Requires 16-byte aligned A and B with lda, ldb multiples of 4 (and below 2^21 so that a tile's byte offsets fit 32 bits).
#pragma once
#include "sgemm_tile.hpp"

namespace decx_hip {

// BLK_ = 32: blocks of 32x32 on v_mfma_f32_32x32x2_f32 (two k per instruction, 64 cycles); BLK_ = 16: blocks of 16x16 on
// v_mfma_f32_16x16x4_f32 (four k per instruction, 32 cycles: a chain walks K twice as fast), for results with fewer
// than four 32x32 blocks per CU.
template <int BM_, int BN_, int BK_, int STAGES_, int BLK_ = 32, int WAVES_M_ = 2, int WAVES_N_ = 2>
struct DmaTile {
    static constexpr bool APAIR = BLK_ == 32;                         // one read of A serves two MFMAs of a block
    static constexpr int BM = BM_, BN = BN_, BK = BK_, STAGES = STAGES_, BLK = BLK_;
    static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NWAVES = WAVES_M * WAVES_N, NT = 64 * NWAVES;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, MI = WM / BLK, NI = WN / BLK;    // waves of MI x NI blocks
    static constexpr int KI = BLK == 32 ? 2 : 4;                        // k per instruction
    static constexpr int UA = BK / 4;                                   // 16-byte units per row of A and step
    static constexpr int BN_LDS = BN <= 32 ? 32 : BN <= 64 ? 64 : BN <= 128 ? 128 : 256;    // columns of B staged per row: a load of 64 units covers whole rows
    static constexpr int UB = BN_LDS / 4;                               // 16-byte units per row of B in LDS
    static constexpr int A_UNITS = BM * UA, B_UNITS = BK * UB;
    static constexpr int A_LOADS = A_UNITS / 64 / NWAVES, B_LOADS = B_UNITS / 64 / NWAVES;   // per wave and step, 1 KiB each
    static constexpr int LOADS = A_LOADS + B_LOADS;
    static constexpr int STAGE_FLOATS = (A_UNITS + B_UNITS) * 4;
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_FLOATS * sizeof(float);
    // slot of unit q of row `row` of A inside its row, and of unit u of row k of B (see the header)
    __device__ static constexpr int a_slot(int row, int q) { return UA >= 8 ? q ^ (row & 7) : q ^ ((row >> 1) & 3); }
    __device__ static constexpr int b_slot(int k, int u) { return BLK == 32 ? u : u ^ (4 * (k & 1)); }
    static constexpr int HALF = BK / KI / 2;                            // MFMAs per block and half step
    static constexpr int READS = ((APAIR ? MI : 2 * MI) + NI) * HALF / 2, MFMAS = HALF * MI * NI;       // per half step and wave
    static_assert((BLK == 32 || BLK == 16) && BM % (WAVES_M * BLK) == 0 && BN % (WAVES_N * BLK) == 0 && BN_LDS <= 256 && UB >= 8 && 64 % UB == 0,
                  "whole blocks per wave; a load covers whole rows of B");
    static_assert(BK % 16 == 0 && (UA >= 8 || (UA == 4 && BLK == 32)) && 64 % UA == 0 && HALF % 2 == 0,
                  "whole units per half step; the swizzle spreads a read over 8 slots (of one row, or of two rows of 4)");
    static_assert(A_UNITS % (64 * NWAVES) == 0 && B_UNITS % (64 * NWAVES) == 0, "loads divide over the waves");
    static_assert(STAGES >= 2 && LOADS * (STAGES - 1) <= 63, "vmcnt is a 6-bit counter");
    static_assert(LOADS <= MFMAS - 1, "the loads go out behind the MFMAs of a half step");
};

template <class S, bool HAS_C>
__global__ __launch_bounds__(S::NT) void sgemm_dma_kernel(const float* __restrict__ A, int lda, const float* __restrict__ B,
                                                          int ldb, const float* Cin, int ldc, float* D, int ldd, int M, int N,
                                                          int K, int tiles_m, int tiles_n, int group_m, bool relu,
                                                          size_t a_batch_stride, size_t b_batch_stride, size_t c_batch_stride,
                                                          size_t d_batch_stride) {
    constexpr int BK = S::BK, UA = S::UA, UB = S::UB, STAGES = S::STAGES, HALF = S::HALF, MI = S::MI, NI = S::NI;
    constexpr int READS = S::READS, MFMAS = S::MFMAS;
    A += (size_t)blockIdx.y * a_batch_stride;
    B += (size_t)blockIdx.y * b_batch_stride;
    if (HAS_C) Cin += (size_t)blockIdx.y * c_batch_stride;
    D += (size_t)blockIdx.y * d_batch_stride;
    extern __shared__ __attribute__((aligned(16))) float lds[];      // [STAGES][A: BM rows x UA units | B: BK rows x UB units]
    const uint32_t lds_base = lds_byte_address(lds);

    const TileCoord tc = xcd_grouped_tile(blockIdx.x, tiles_m, tiles_n, group_m);
    const int bm0 = tc.tm * S::BM, bn0 = tc.tn * S::BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane % S::BLK, ls = lane / S::BLK;  // row (of A) or column (of B) inside a block, and k-slot
    const int full_steps = K / BK, rem = K - full_steps * BK;

    // ---- sources of this wave's loads: a wave-uniform base per operand that moves one K step per fetched step, plus
    // loop-invariant byte offsets per lane (rows of this tile only)
    const float* a_base = A + (size_t)bm0 * lda;
    const float* b_base = B;
    const size_t b_step = (size_t)BK * ldb;
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int row = (wave * S::A_LOADS + j) * (64 / UA) + lane / UA;     // 64 units = 64 / UA rows
        const int q = S::a_slot(row, lane % UA);                              // the unit whose swizzled slot is this lane (the swizzles are involutions)
        int m = bm0 + row;
        if (m >= M) m = M - 1;                                                // rows past the end are computed and never stored
        a_off[j] = (uint32_t)(((size_t)(m - bm0) * lda + 4 * q) * sizeof(float));
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int kr = (wave * S::B_LOADS + j) * (64 / UB) + lane / UB;      // 64 units = 64 / UB rows of k
        const int col = clamp_group_col(bn0 + 4 * S::b_slot(kr, lane % UB), N, 4);    // stay inside the operand; such columns are never stored
        b_off[j] = (uint32_t)(((size_t)kr * ldb + col) * sizeof(float));
    }
    int fetch_step = 0;                                // steps whose loads have gone out
    auto issue_one = [&](int stage, auto j_tag, auto site_tag) {       // site_tag: a number of its own for every place of call
        constexpr int J = decltype(j_tag)::value, TAG = decltype(site_tag)::value * 64 + J;
        const uint32_t base = lds_base + (uint32_t)stage * (S::STAGE_FLOATS * 4u);
        if constexpr (J < S::A_LOADS) {
            dma_load16_tagged<TAG>(a_base, a_off[J], base + (uint32_t)(wave * S::A_LOADS + J) * 1024u);
        } else {
            dma_load16_tagged<TAG>(b_base, b_off[J - S::A_LOADS], base + (uint32_t)(S::A_UNITS * 16) + (uint32_t)(wave * S::B_LOADS + J - S::A_LOADS) * 1024u);
        }
        if constexpr (J == S::LOADS - 1) {
            ++fetch_step;
            const bool more = fetch_step < full_steps;                        // scalar: the pointers stop on the last whole step
            a_base += more ? BK : 0;
            b_base += more ? b_step : (size_t)0;
        }
    };

    // ---- where this lane's operands lie: unit q of its row of every row block of A in every buffer, its column of every
    // column block of B in rows s, s+2, ...
    // 32x32 blocks: a register per (buffer, row block, unit) -- ds_read2_b32 carries offsets of up to 255 floats only.
    // 16x16 blocks: a register per unit -- the swizzle of A looks at the low bits of the row only, which blocks and
    // waves do not change, so unit q of a lane's row lies at the same place in every row block and buffer, a whole
    // number of rows further: an offset ds_read_b32 can carry.
    constexpr int BLK = S::BLK;
    const float* pa_all[BLK == 32 ? STAGES : 1][BLK == 32 ? MI : 1][UA];
    const float* pb_all[BLK == 32 ? STAGES : 1][NI];
#pragma unroll
    for (int st = 0; st < (BLK == 32 ? STAGES : 1); ++st) {
#pragma unroll
        for (int mi = 0; mi < (BLK == 32 ? MI : 1); ++mi) {
            const int row = wm0 + BLK * mi + li;
#pragma unroll
            for (int q = 0; q < UA; ++q) pa_all[st][mi][q] = lds + st * S::STAGE_FLOATS + (row * UA + S::a_slot(li, q)) * 4 + ls;
        }
#pragma unroll
        for (int ni = 0; ni < NI; ++ni) {
            const int col = wn0 + BLK * ni + li;                  // rows ls, ls + KI, ... of B: their parity is that of ls
            pb_all[st][ni] = lds + st * S::STAGE_FLOATS + S::A_UNITS * 4 + ls * S::BN_LDS + S::b_slot(ls, col / 4) * 4 + col % 4;
        }
    }
    auto pa = [&](auto st_tag, auto mi_tag, auto q_tag) {
        constexpr int ST = decltype(st_tag)::value, MIV = decltype(mi_tag)::value, Q = decltype(q_tag)::value;
        if constexpr (BLK == 32) return pa_all[ST][MIV][Q];
        else return pa_all[0][0][Q] + ST * S::STAGE_FLOATS + BLK * MIV * UA * 4;
    };
    auto pb = [&](auto st_tag, auto ni_tag) {
        constexpr int ST = decltype(st_tag)::value, NIV = decltype(ni_tag)::value;
        if constexpr (BLK == 32) return pb_all[ST][NIV];
        else return pb_all[0][NIV] + ST * S::STAGE_FLOATS;
    };

    // accumulators: lane holds, of each of its blocks, D[8 (r / 4) + 4 ls + r % 4][li], r = 0 .. 15 (32x32), or
    // D[4 ls + r][li], r = 0 .. 3 (16x16); the chains start at C when there is one
    constexpr int ACC = BLK == 32 ? 16 : 4;
    typedef float acc_t __attribute__((ext_vector_type(ACC)));
    auto acc_row = [&](int mi, int r) { return wm0 + BLK * mi + (BLK == 32 ? (r >> 2) * 8 + ls * 4 + (r & 3) : 4 * ls + r); };
    acc_t acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < ACC; ++r) {
                acc[mi][ni][r] = 0.f;
                if (HAS_C) {
                    const int m = bm0 + acc_row(mi, r), n = bn0 + wn0 + BLK * ni + li;
                    if (m < M && n < N) acc[mi][ni][r] = Cin[(size_t)m * ldc + n];
                }
            }

    // fragment sets: set 0 feeds the first half of a step, set 1 the second
    // (the two operands one read brings lie side by side, as the read delivers them: no register moves)
    float af[2][HALF / 2][MI][2], bf[2][HALF / 2][NI][2];
    // Read number n (0 .. READS-1) of half `h` of the step that lies `stage_floats` past the pointers of buffer ST.  The
    // reads come in groups that fetch the operands of MFMAs 2u and 2u + 1 (of every block) of the half: per row block one
    // read of A (32x32: both floats of a unit) or two (16x16: a float of each of two units), then two rows of B per
    // column block.
    auto read_one = [&](auto st_tag, auto h_tag, auto n_tag, int stage_floats) {
        constexpr int ST = decltype(st_tag)::value, H = decltype(h_tag)::value, NR = decltype(n_tag)::value;
        constexpr int AR = S::APAIR ? MI : 2 * MI;      // reads of A per two k steps
        constexpr int U = NR / (AR + NI), W = NR % (AR + NI);
        if constexpr (W < AR && S::APAIR) {
            const float* p = pa(st_tag, std::integral_constant<int, W < MI ? W : 0>{}, std::integral_constant<int, (H * (HALF / 2) + U) % UA>{}) + stage_floats;   // floats s and s + 2 of a unit
            af[H][U][W][0] = p[0];
            af[H][U][W][1] = p[2];
        } else if constexpr (W < AR) {                                           // float s of one unit
            af[H][U][W % MI][W / MI] = pa(st_tag, std::integral_constant<int, W % MI>{}, std::integral_constant<int, (H * HALF + 2 * U + W / MI) % UA>{})[stage_floats];
        } else {
            const float* p = pb(st_tag, std::integral_constant<int, W >= AR ? W - AR : 0>{}) + S::KI * (H * HALF + 2 * U) * S::BN_LDS + stage_floats;
            bf[H][U][W - AR][0] = p[0];
            bf[H][U][W - AR][1] = p[S::KI * S::BN_LDS];
        }
    };
    // MFMA number m (0 .. MFMAS-1) of half `h`: k pair m / (MI NI) of the half, blocks in turn
    auto mfma_one = [&](auto h_tag, auto m_tag) {
        constexpr int H = decltype(h_tag)::value, MM = decltype(m_tag)::value;
        constexpr int I = MM / (MI * NI), BMI = (MM / NI) % MI, BNI = MM % NI;
        if constexpr (BLK == 32) acc[BMI][BNI] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[H][I / 2][BMI][I % 2], bf[H][I / 2][BNI][I % 2], acc[BMI][BNI], 0, 0, 0);
        else acc[BMI][BNI] = __builtin_amdgcn_mfma_f32_16x16x4f32(af[H][I / 2][BMI][I % 2], bf[H][I / 2][BNI][I % 2], acc[BMI][BNI], 0, 0, 0);
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    if (full_steps > 0) {
        static_for<0, STAGES>([&](auto s_tag) { static_for<0, S::LOADS>([&](auto j) { issue_one(decltype(s_tag)::value, j, std::integral_constant<int, 2 * STAGES + decltype(s_tag)::value>{}); }); });
        wait_dma_then_barrier<S::LOADS*(STAGES - 1)>();                      // step 0 has landed
        static_for<0, READS>([&](auto n) { read_one(I0{}, I0{}, n, 0); });  // its first half

        auto k_step = [&](auto st_tag, auto copy_tag) {
            constexpr int ST = decltype(st_tag)::value, SITE = decltype(copy_tag)::value * STAGES + ST;
            typedef std::integral_constant<int, (ST + 1) % STAGES> NextStage;
            // first half: read n goes out behind MFMA n MFMAS / READS
            static_for<0, MFMAS>([&](auto m_tag) {
                constexpr int MM = decltype(m_tag)::value;
                mfma_one(I0{}, m_tag);
                static_for<0, READS>([&](auto n_tag) {
                    if constexpr (decltype(n_tag)::value * MFMAS / READS == MM) read_one(st_tag, I1{}, n_tag, 0);
                });
                __builtin_amdgcn_sched_barrier(0);
            });
            // second half: the barrier behind its first MFMA, then the loads of step t+STAGES behind MFMAs 1, 2, ... and
            // read n of the next step's first half behind MFMA 1 + n (MFMAS - 1) / READS
            static_for<0, MFMAS>([&](auto m_tag) {
                constexpr int MM = decltype(m_tag)::value;
                mfma_one(I1{}, m_tag);
                if constexpr (MM == 0) {
                    __builtin_amdgcn_sched_barrier(0);
                    wait_dma_then_barrier<S::LOADS*(STAGES - 2)>();          // step t+1 has landed; step t's buffer is free
                } else {
                    if constexpr (MM - 1 < S::LOADS) issue_one(ST, std::integral_constant<int, MM - 1>{}, std::integral_constant<int, SITE>{});
                    static_for<0, READS>([&](auto n_tag) {
                        if constexpr (1 + decltype(n_tag)::value * (MFMAS - 1) / READS == MM) read_one(NextStage{}, I0{}, n_tag, 0);
                    });
                }
                __builtin_amdgcn_sched_barrier(0);
            });
        };
        // whole passes over the buffers, free of branches, then the steps that are left
        int t0 = 0;
        for (; t0 + STAGES <= full_steps; t0 += STAGES) static_for<0, STAGES>([&](auto st) { k_step(st, I0{}); });
        static_for<0, STAGES>([&](auto st) {
            if (t0 + decltype(st)::value < full_steps) k_step(st, I1{});
        });
        wait_dma_then_barrier<0>();                                          // nothing is in flight into LDS any more
    }

    if (rem > 0) {
        // the ragged last step, through registers into buffer 0: zeros from K on
        const int k0 = full_steps * BK;
#pragma unroll
        for (int p = 0; p < S::A_UNITS / S::NT; ++p) {
            const int id = tid + p * S::NT, row = id / UA, q = id % UA, k = k0 + 4 * q;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (k < K) {
                int m = bm0 + row;
                if (m >= M) m = M - 1;
                v = *reinterpret_cast<const f32x4*>(A + (size_t)m * lda + k);      // lda % 4 == 0 keeps the quad inside the pitch
                if (k + 1 >= K) v[1] = 0.f;
                if (k + 2 >= K) v[2] = 0.f;
                if (k + 3 >= K) v[3] = 0.f;
            }
            *reinterpret_cast<f32x4*>(lds + (row * UA + S::a_slot(row, q)) * 4) = v;
        }
#pragma unroll
        for (int p = 0; p < S::B_UNITS / S::NT; ++p) {
            const int id = tid + p * S::NT, kr = id / UB, u = id % UB, k = k0 + kr;
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (k < K) v = *reinterpret_cast<const f32x4*>(B + (size_t)k * ldb + clamp_group_col(bn0 + 4 * u, N, 4));
            *reinterpret_cast<f32x4*>(lds + S::A_UNITS * 4 + (kr * UB + S::b_slot(kr, u)) * 4) = v;
        }
        lds_sync();
        static_for<0, 2>([&](auto h_tag) {
            constexpr int H = decltype(h_tag)::value;
            static_for<0, READS>([&](auto n) { read_one(I0{}, h_tag, n, 0); });
            static_for<0, MFMAS>([&](auto m_tag) {
                if (S::KI * (H * HALF + decltype(m_tag)::value / (MI * NI)) < rem) mfma_one(h_tag, m_tag);
            });
        });
    }

#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int r = 0; r < ACC; ++r) {
            const int m = bm0 + acc_row(mi, r);
            if (m < M) {
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const int n = bn0 + wn0 + BLK * ni + li;
                    if (n < N) D[(size_t)m * ldd + n] = relu ? relu_by_sign(acc[mi][ni][r]) : acc[mi][ni][r];
                }
            }
        }
}

}  // namespace decx_hip
