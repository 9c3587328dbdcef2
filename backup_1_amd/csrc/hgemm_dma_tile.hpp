// fp16-in / fp32-accumulate MFMA tile with a multi-stage global->LDS pipeline (gfx950 LDS-DMA loads).
//
// Same tile geometry, LDS layout and fragment reads as hgemm_tile.hpp (XOR-swizzled 16-byte units, ds_read_b128 for
// A, ds_read_b64_tr_b16 for B, 32x32x16 f16 MFMA).  What changes is the staging: global_load_lds_dwordx4 moves 16
// bytes per lane straight from global memory into LDS (lane L of an instruction lands at base + 16*L), so the data
// never passes through VGPRs and several K steps can be in flight at once.  The swizzle is applied on the GLOBAL
// side: lane L of a 64-unit chunk fetches the unit whose swizzled slot is L.
//
// Pipeline with STAGES LDS buffers, one barrier per K step, placed inside the step's last MFMA block: before it the
// wave waits until its own loads of step t+1 have landed (vmcnt <= loads issued after them); once all waves are past
// it nobody reads step t's buffer any more, so the loads of step t+STAGES go out at once and the first fragments of
// step t+1 are fetched, all of it between the remaining MFMAs of step t.
// The loads are issued through inline asm so that the compiler's wait-count insertion does not serialise them; the
// waits are written out explicitly.  M0 (the LDS base of such a load) is written only by those asm statements.
//
// The last, partial K step (K % BK != 0) cannot zero-fill through the DMA path and is staged through registers.
// Requires 16-byte aligned operands with lda, ldb multiples of 8.
#pragma once
#include <type_traits>
#include "hgemm_tile.hpp"

namespace decx_hip {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int STAGES_>
struct HgemmDmaShape : HgemmShape<BM_, BN_, BK_, WAVES_M_, WAVES_N_> {
    typedef HgemmShape<BM_, BN_, BK_, WAVES_M_, WAVES_N_> Base;
    static constexpr int STAGES = STAGES_;
    static constexpr int NWAVES = WAVES_M_ * WAVES_N_;
    static constexpr int A_CHUNKS = Base::A_UNITS / 64, B_CHUNKS = Base::B_UNITS / 64;    // 1 KiB per load instruction
    static constexpr int A_LOADS = A_CHUNKS / NWAVES, B_LOADS = B_CHUNKS / NWAVES;      // per wave and stage
    static constexpr int LOADS = A_LOADS + B_LOADS;
    static constexpr int STAGE_UNITS = Base::A_UNITS + Base::B_UNITS;
    static constexpr size_t LDS_BYTES = (size_t)STAGES * STAGE_UNITS * 16;
    static_assert(A_CHUNKS % NWAVES == 0 && B_CHUNKS % NWAVES == 0, "chunks must divide over the waves");
    static_assert(64 % Base::UA == 0 && Base::UB <= 64 && 64 % Base::UB == 0, "a chunk covers whole rows");
    static_assert(LOADS * (STAGES - 2) <= 63, "vmcnt is a 6-bit counter");
    static_assert(STAGES >= 2, "need at least double buffering");
};

// SPLIT_K: blockIdx.z selects a range of K (k_split_len long, a multiple of BK); the tile's fp32 partial sums go to a
// workspace of dense M x N fp32 planes instead of being rounded and stored.  partial_plane != 0: range z stores its
// sums into plane z (partial + z * partial_plane) with plain stores -- every element of a plane inside the result is
// written by exactly one workgroup, so nothing has to be zeroed, and the finishing kernel adds the planes in range
// order: a result that is the same on every run.  partial_plane == 0: all ranges add into one plane (zeroed
// beforehand) with atomics, in whatever order they arrive.
template <class S, bool HAS_C, bool SPLIT_K = false>
__global__ __launch_bounds__(S::NT) void hgemm_dma_kernel(const _Float16* __restrict__ A, int lda,
                                                          const _Float16* __restrict__ B, int ldb, const _Float16* Cin,
                                                          int ldc, _Float16* D, int ldd, int M, int N, int K, int tiles_m,
                                                          int tiles_n, int group_m, size_t a_batch_stride,
                                                          size_t b_batch_stride, size_t c_batch_stride, size_t d_batch_stride,
                                                          float* partial, int k_split_len, size_t partial_plane) {
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, NT = S::NT, UA = S::UA, UB = S::UB, MI = S::MI, NI = S::NI;
    constexpr int STAGES = S::STAGES;
    static_assert(!(SPLIT_K && HAS_C), "C joins a split product in the finishing kernel");
    // blockIdx.y walks a batch of independent problems of the same shape
    A += (size_t)blockIdx.y * a_batch_stride;
    B += (size_t)blockIdx.y * b_batch_stride;
    if (HAS_C) Cin += (size_t)blockIdx.y * c_batch_stride;
    D += (size_t)blockIdx.y * d_batch_stride;
    if (SPLIT_K) {
        const int k_begin = (int)blockIdx.z * k_split_len;
        A += k_begin;                             // a multiple of BK halves: rows keep their 16-byte alignment
        B += (size_t)k_begin * ldb;
        K = K - k_begin < k_split_len ? K - k_begin : k_split_len;
    }
    constexpr int KS = BK / 16;                                // MFMA k-blocks per K step
    constexpr int BLK = MI * NI;                               // MFMAs per k-block
    static_assert(KS >= 2, "the schedule below needs at least two k-blocks per K step");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    u32x4* lds = reinterpret_cast<u32x4*>(lds_raw);            // [STAGES][A_UNITS | B_UNITS]
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw;

    const TileCoord tc = xcd_grouped_tile(blockIdx.x, tiles_m, tiles_n, group_m);
    const int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;

    // ---- global sources of this wave's DMA loads: a wave-uniform base per operand that advances by one K step per
    // fetched step, plus loop-invariant per-lane byte offsets (rows of this tile only, so 32 bits are plenty)
    int m_first = bm0 < M ? bm0 : M - 1;
    const _Float16* a_base = A + (size_t)m_first * lda;        // + BK halves per step
    const _Float16* b_base = B;                                // + BK rows per step
    uint32_t a_off[S::A_LOADS], b_off[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int chunk = wave * S::A_LOADS + j;               // 64 units = 64/UA rows
        const int r = chunk * (64 / UA) + lane / UA;
        const int q = (lane % UA) ^ ((r / (16 / UA)) % UA);    // the unit whose swizzled slot is this lane
        int m = bm0 + r;
        if (m >= M) m = M - 1;
        a_off[j] = (uint32_t)(((size_t)(m - m_first) * lda + 8 * q) * sizeof(_Float16));
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int chunk = wave * S::B_LOADS + j;               // 64 units = 64/UB k-rows
        const int kr = chunk * (64 / UB) + lane / UB;
        const int u = (lane % UB) ^ ((kr & 3) << 2);
        int col = bn0 + 8 * u;
        col = clamp_group_col(col, N, 8);                      // stay inside the operand; such columns are never stored
        b_off[j] = (uint32_t)(((size_t)kr * ldb + col) * sizeof(_Float16));
    }
    const size_t b_step = (size_t)BK * ldb;

    // load number j (A loads first, then B) of the next K step to be fetched, into LDS buffer `stage`; the bases move
    // on after the last load of a step
    auto issue_one = [&](int stage, int j) {
        const uint32_t base = lds_base + (uint32_t)stage * (S::STAGE_UNITS * 16);
        if (j < S::A_LOADS) {
            dma_load16(a_base, a_off[j], base + (uint32_t)(wave * S::A_LOADS + j) * 1024u);
        } else {
            const int jb = j - S::A_LOADS;
            dma_load16(b_base, b_off[jb], base + (uint32_t)(S::A_UNITS * 16) + (uint32_t)(wave * S::B_LOADS + jb) * 1024u);
        }
        if (j == S::LOADS - 1) {
            a_base += BK;
            b_base += b_step;
        }
    };
    auto issue_stage = [&](int stage) {
#pragma unroll
        for (int j = 0; j < S::LOADS; ++j) issue_one(stage, j);
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    const int full_steps = K / BK;

    // prologue: every LDS buffer gets a K step (issue nothing for steps that do not exist)
#pragma unroll
    for (int s = 0; s < STAGES; ++s)
        if (s < full_steps) issue_stage(s);

    // ---- fragment reads -------------------------------------------------------------------------------------------
    // Loop-invariant per-lane byte offsets inside one LDS buffer; everything else about a read (row block, k-block,
    // low/high half) is a compile-time constant that folds into the instruction's offset field, because the swizzle
    // terms only depend on address bits those constants do not touch.
    const int tg = lane >> 4, ts = lane & 15;
    const int t_row = 8 * (tg >> 1) + (ts >> 2);               // transposed read: row inside a 16-row k-block (+4: high half)
    const int t_col = 16 * (tg & 1) + 4 * (ts & 3);            // and column inside a 32-column block
    typedef short i16x8 __attribute__((ext_vector_type(8)));
    struct Frags {
        f16x8 a[MI];
        i16x4 b_lo[NI], b_hi[NI];
    };
    uint32_t a_frag_off[KS], b_frag_off[NI];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a_frag_off[ks] = (uint32_t)a_unit_slot(wm0 + li, 2 * ks + lh, UA) * 16u;   // + mi*32 rows
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int col = wn0 + ni * 32 + t_col;
        b_frag_off[ni] = (uint32_t)(S::A_UNITS * 16) + (uint32_t)b_unit_slot(t_row, col >> 3, UB) * 16u + (uint32_t)(col & 7) * 2u;
    }
    static_assert(32 % (16 / UA) == 0 && (32 / (16 / UA)) % UA == 0, "row blocks of 32 must not change the A swizzle");
    // The reads of one k-block, numbered in the order the MFMAs (mi-major) first need them:
    //   0: a[0], then b_lo/b_hi of ni = 0..NI-1, then a[1..MI-1]
    constexpr int FRAG_READS = MI + 2 * NI;
    auto read_one = [&](Frags& f, int stage, int ks, int r) {
        const unsigned char* buf = lds_raw + (size_t)stage * (S::STAGE_UNITS * 16);
        if (r == 0 || r > 2 * NI) {
            const int mi = r == 0 ? 0 : r - 2 * NI;
            u32x4 raw = *reinterpret_cast<const u32x4*>(buf + a_frag_off[ks] + mi * (32 * UA * 16));
            f.a[mi] = __builtin_bit_cast(f16x8, raw);
        } else {
            const int ni = (r - 1) / 2, hi = (r - 1) % 2;
            const unsigned char* p = buf + b_frag_off[ni] + (16 * ks + 4 * hi) * (UB * 16);   // rows k and k+4 share k & 3
            i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)p);
            if (hi) f.b_hi[ni] = v;
            else f.b_lo[ni] = v;
        }
    };
    auto mfma_one = [&](const Frags& f, int i) {
        const int mi = i / NI, ni = i % NI;
        i16x8 both = {f.b_lo[ni][0], f.b_lo[ni][1], f.b_lo[ni][2], f.b_lo[ni][3],
                      f.b_hi[ni][0], f.b_hi[ni][1], f.b_hi[ni][2], f.b_hi[ni][3]};
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(f.a[mi], __builtin_bit_cast(f16x8, both), acc[mi][ni], 0, 0, 0);
    };
#define DECX_PIN() __builtin_amdgcn_sched_barrier(0)

    Frags f0, f1;

    // One K step.  f0 holds the fragments of its first k-block on entry and those of the NEXT step's first k-block on
    // exit.  Source order is the issue order (every slot is pinned): memory instructions ride between MFMAs.
    //   block 0 (f0): MFMA i + LDS read i of block 1                          (reads finish ahead of block 1)
    //   block 1 (f1): first half plain, then wait for the next step's data + barrier -- at this point every wave has
    //                 finished reading this step's buffer, so it is refilled right away (DMA loads of step t+STAGES),
    //                 and the next step's first fragments are read, all between the MFMAs of the second half.
    auto k_step = [&](int stg, int next, auto wait_tag, bool refill, bool has_next) {
        constexpr int WAITN = decltype(wait_tag)::value;
        // k-blocks 0 .. KS-2: MFMA i of block b rides with LDS read i of block b+1 (fragment sets alternate f0, f1)
#pragma unroll
        for (int b = 0; b + 1 < KS; ++b) {
#pragma unroll
            for (int i = 0; i < BLK; ++i) {
                constexpr int RPS = (FRAG_READS + BLK - 1) / BLK;      // reads per MFMA slot, front-loaded
#pragma unroll
                for (int r = i * RPS; r < (i + 1) * RPS && r < FRAG_READS; ++r) read_one((b & 1) ? f0 : f1, stg, b + 1, r);
                mfma_one((b & 1) ? f1 : f0, i);
                DECX_PIN();
            }
        }
        // last k-block: a few MFMAs, the barrier, then refill + next step's first fragments between the rest
        Frags& fl = ((KS - 1) & 1) ? f1 : f0;
        Frags& fn = ((KS - 1) & 1) ? f0 : f1;      // receives the next step's block 0 (KS even: this is f0 again)
        constexpr int PRE = BLK / 4;
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            mfma_one(fl, i);
            DECX_PIN();
        }
        if (has_next) {
            wait_dma_then_barrier<WAITN>();
            DECX_PIN();
        }
        constexpr int SLOTS = BLK - PRE;
#pragma unroll
        for (int i = 0; i < SLOTS; ++i) {
            if (refill) {
#pragma unroll
                for (int j = (i * S::LOADS) / SLOTS; j < ((i + 1) * S::LOADS) / SLOTS; ++j) issue_one(stg, j);
            }
            if (has_next) {
#pragma unroll
                for (int r = (i * FRAG_READS) / SLOTS; r < ((i + 1) * FRAG_READS) / SLOTS; ++r) read_one(fn, next, 0, r);
            }
            mfma_one(fl, PRE + i);
            DECX_PIN();
        }
    };
    static_assert(KS % 2 == 0, "fragment sets must line up across K steps (block 0 always in f0)");

    if (full_steps > 0) {
        wait_dma_then_barrier<0>();                            // step 0 (and whatever else the prologue fetched) has landed
#pragma unroll
        for (int r = 0; r < FRAG_READS; ++r) read_one(f0, 0, 0, r);
        DECX_PIN();

        // steady state: every step refills its buffer (t + STAGES < full_steps).  Before the barrier of step t the data of
        // step t+1 must have landed; the loads of steps t+2 .. t+STAGES-1, issued later, may still be in flight.
        const int steady = full_steps > STAGES ? full_steps - STAGES : 0;
        int stg = 0;
        for (int t = 0; t < steady; ++t) {
            const int next = stg + 1 == STAGES ? 0 : stg + 1;
            k_step(stg, next, std::integral_constant<int, S::LOADS*(STAGES - 2)>{}, true, true);
            stg = next;
        }
        // the last (<= STAGES) steps: nothing left to fetch, conservative waits
        for (int t = steady; t < full_steps; ++t) {
            const int next = stg + 1 == STAGES ? 0 : stg + 1;
            k_step(stg, next, std::integral_constant<int, 0>{}, false, t + 1 < full_steps);
            stg = next;
        }
    }

    // ---- partial last K step through registers --------------------------------------------------------------------
    if (full_steps * BK < K) {
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
            if (k0 + kr < K) {
                int col = bn0 + 8 * u;
                col = clamp_group_col(col, N, 8);
                v = *reinterpret_cast<const u32x4*>(B + (size_t)(k0 + kr) * ldb + col);
            }
            b_stage[p] = v;
        }
        wait_dma_then_barrier<0>();                            // everybody is done with every buffer
        u32x4* Ab = lds;
        u32x4* Bb = lds + S::A_UNITS;
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) {
            const int id = tid + p * NT;
            Ab[a_unit_slot(id / UA, id % UA, UA)] = a_stage[p];
        }
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) {
            const int id = tid + p * NT;
            Bb[b_unit_slot(id / UB, id % UB, UB)] = b_stage[p];
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int r = 0; r < FRAG_READS; ++r) read_one(f0, 0, ks, r);
#pragma unroll
            for (int i = 0; i < BLK; ++i) mfma_one(f0, i);
        }
    }
#undef DECX_PIN

    if (SPLIT_K) {
        const bool ordered = partial_plane != 0;                 // uniform over the launch
        float* plane = partial + (size_t)blockIdx.z * partial_plane;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (m < M) {
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int n = bn0 + wn0 + ni * 32 + li;
                        if (n < N) {
                            if (ordered) plane[(size_t)m * N + n] = acc[mi][ni][r];
                            else unsafeAtomicAdd(plane + (size_t)m * N + n, acc[mi][ni][r]);
                        }
                    }
                }
            }
        return;
    }
    // ---- epilogue: round once to binary16; dst = A*B + C adds C (as fp32) first.  A tile that lies wholly inside the
    // result stores without bounds checks (each one is a branch around its store; one scalar test per workgroup).
    auto store_tile = [&](auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (FULL || m < M) {
                    _Float16* drow = D + (size_t)m * ldd;
                    const _Float16* crow = HAS_C ? Cin + (size_t)m * ldc : nullptr;
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int n = bn0 + wn0 + ni * 32 + li;
                        if (FULL || n < N) drow[n] = (_Float16)(HAS_C ? acc[mi][ni][r] + (float)crow[n] : acc[mi][ni][r]);
                    }
                }
            }
    };
    if (bm0 + BM <= M && bn0 + BN <= N) store_tile(std::true_type{});
    else store_tile(std::false_type{});
}

}  // namespace decx_hip
