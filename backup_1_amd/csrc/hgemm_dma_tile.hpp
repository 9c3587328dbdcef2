// fp16-in / fp32-accumulate MFMA tile with a multi-stage global->LDS pipeline (gfx950 LDS-DMA loads).
//
// Same tile geometry, LDS layout and fragment reads as hgemm_tile.hpp (XOR-swizzled 16-byte units, ds_read_b128 for
// A, ds_read_b64_tr_b16 for B, 32x32x16 f16 MFMA).  What changes is the staging: global_load_lds_dwordx4 moves 16
// bytes per lane straight from global memory into LDS (lane L of an instruction lands at base + 16*L), so the data
// never passes through VGPRs and several K steps can be in flight at once.  The swizzle is applied on the GLOBAL
// side: lane L of a 64-unit chunk fetches the unit whose swizzled slot is L.
//
// Pipeline with STAGES LDS buffers: at the top of step t the wave waits until its own loads of step t have landed
// (vmcnt <= loads issued after them), all waves meet at one barrier (which also guarantees everybody finished reading
// the buffer of step t-1), then the loads of step t+STAGES-1 are issued into that freed buffer and step t is computed.
// The loads are issued through inline asm so that the compiler's wait-count insertion does not serialise them; the
// waits are written out explicitly.  M0 (the LDS base of such a load) is written only by those asm statements.
//
// The last, partial K step (K % BK != 0) cannot zero-fill through the DMA path and is staged through registers.
// Requires 16-byte aligned operands with lda, ldb multiples of 8.
#pragma once
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

// One 16-byte-per-lane load from global memory straight into LDS at lds_base + 16*lane (lds_base wave-uniform).
__device__ __forceinline__ void dma_load16(const void* gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(lds_base) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_dma_then_barrier() {
    // my loads older than the N most recent have landed; my LDS reads are done; then everybody meets
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}

template <class S>
__global__ __launch_bounds__(S::NT) void hgemm_dma_kernel(const _Float16* __restrict__ A, int lda,
                                                          const _Float16* __restrict__ B, int ldb, const _Float16* Cin,
                                                          int ldc, _Float16* D, int ldd, int M, int N, int K, int tiles_m,
                                                          int tiles_n, int group_m) {
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, NT = S::NT, UA = S::UA, UB = S::UB, MI = S::MI, NI = S::NI;
    constexpr int STAGES = S::STAGES;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    u32x4* lds = reinterpret_cast<u32x4*>(lds_raw);            // [STAGES][A_UNITS | B_UNITS]
    const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)lds_raw;

    const TileCoord tc = xcd_grouped_tile(blockIdx.x, tiles_m, tiles_n, group_m);
    const int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;

    // ---- per-lane global sources of this wave's DMA loads (advance by one K step per stage) -----------------------
    const _Float16* a_src[S::A_LOADS];
    const _Float16* b_src[S::B_LOADS];
#pragma unroll
    for (int j = 0; j < S::A_LOADS; ++j) {
        const int chunk = wave * S::A_LOADS + j;               // 64 units = 64/UA rows
        const int r = chunk * (64 / UA) + lane / UA;
        const int q = (lane % UA) ^ ((r / (16 / UA)) % UA);    // the unit whose swizzled slot is this lane
        int m = bm0 + r;
        if (m >= M) m = M - 1;
        a_src[j] = A + (size_t)m * lda + 8 * q;
    }
#pragma unroll
    for (int j = 0; j < S::B_LOADS; ++j) {
        const int chunk = wave * S::B_LOADS + j;               // 64 units = 64/UB k-rows
        const int kr = chunk * (64 / UB) + lane / UB;
        const int u = (lane % UB) ^ ((kr & 3) << 2);
        int col = bn0 + 8 * u;
        if (col > ldb - 8) col = ldb - 8;                      // stay inside the pitch; such columns are never stored
        b_src[j] = B + (size_t)kr * ldb + col;
    }
    const size_t b_step = (size_t)BK * ldb;

    auto issue_stage = [&](int stage, int t) {
        const uint32_t base = lds_base + (uint32_t)stage * (S::STAGE_UNITS * 16);
#pragma unroll
        for (int j = 0; j < S::A_LOADS; ++j)
            dma_load16(a_src[j] + (size_t)t * BK, base + (uint32_t)(wave * S::A_LOADS + j) * 1024u);
#pragma unroll
        for (int j = 0; j < S::B_LOADS; ++j)
            dma_load16(b_src[j] + (size_t)t * b_step, base + (uint32_t)(S::A_UNITS * 16) + (uint32_t)(wave * S::B_LOADS + j) * 1024u);
    };

    // ---- accumulators ------------------------------------------------------------------------------------------------
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    const int full_steps = K / BK;

    // prologue: fill STAGES-1 buffers (issue nothing for steps that do not exist)
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < full_steps) issue_stage(s, s);

    if (Cin != nullptr) {
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                if (m < M) {
                    const _Float16* crow = Cin + (size_t)m * ldc;
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int n = bn0 + wn0 + ni * 32 + li;
                        if (n < N) acc[mi][ni][r] = (float)crow[n];
                    }
                }
            }
    }

    // transposed-read geometry of this lane (see hgemm_tile.hpp)
    const int tg = lane >> 4, ts = lane & 15;
    const int t_row = 8 * (tg >> 1) + (ts >> 2);
    const int t_col = 16 * (tg & 1) + 4 * (ts & 3);

    auto compute_stage = [&](int stage) {
        const u32x4* Ab = lds + stage * S::STAGE_UNITS;
        const unsigned char* Bb = reinterpret_cast<const unsigned char*>(Ab + S::A_UNITS);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            f16x8 af[MI], bf[NI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) {
                u32x4 raw = Ab[a_unit_slot(wm0 + mi * 32 + li, 2 * ks + lh, UA)];
                af[mi] = __builtin_bit_cast(f16x8, raw);
            }
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) {
                const int col = wn0 + ni * 32 + t_col;
                const int k_lo = 16 * ks + t_row, k_hi = k_lo + 4;
                const int off_lo = b_unit_slot(k_lo, col >> 3, UB) * 16 + (col & 7) * 2;
                const int off_hi = b_unit_slot(k_hi, col >> 3, UB) * 16 + (col & 7) * 2;
                i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(Bb + off_lo));
                i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(Bb + off_hi));
                typedef short i16x8 __attribute__((ext_vector_type(8)));
                i16x8 both = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                bf[ni] = __builtin_bit_cast(f16x8, both);
            }
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[mi], bf[ni], acc[mi][ni], 0, 0, 0);
        }
    };

    // ---- main loop over full K steps -------------------------------------------------------------------------------
    // unrolled by STAGES so that every LDS buffer index is a compile-time constant
    for (int t0 = 0; t0 < full_steps; t0 += STAGES) {
#pragma unroll
        for (int s = 0; s < STAGES; ++s) {
            const int t = t0 + s;
            if (t < full_steps) {
                // groups issued after step t's: min(STAGES-2, full_steps-1-t); the steady-state count is a constant
                if (t + STAGES - 2 < full_steps) wait_dma_then_barrier<S::LOADS*(STAGES - 2)>();
                else wait_dma_then_barrier<0>();
                if (t + STAGES - 1 < full_steps) issue_stage((s + STAGES - 1) % STAGES, t + STAGES - 1);
                compute_stage(s);
            }
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
                if (col > ldb - 8) col = ldb - 8;
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
        compute_stage(0);
    }

#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
            if (m < M) {
                _Float16* drow = D + (size_t)m * ldd;
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const int n = bn0 + wn0 + ni * 32 + li;
                    if (n < N) drow[n] = (_Float16)acc[mi][ni][r];
                }
            }
        }
}

}  // namespace decx_hip
