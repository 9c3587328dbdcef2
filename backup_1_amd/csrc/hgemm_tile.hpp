// fp16-in / fp32-accumulate MFMA contraction tile for gfx950.
//
// One workgroup owns a BM x BN tile and walks K in steps of BK halves; its waves are laid out WAVES_M x WAVES_N and
// each keeps a grid of 32x32 v_mfma_f32_32x32x16_f16 accumulators (fp32) in registers for the whole K walk.
//
// LDS holds both operands exactly as they lie in memory (A row-major [m][k], B row-major [k][n]) in 16-byte units of
// 8 halves, with the unit index XOR-swizzled so that every read below is bank-conflict free without padding:
//   A unit (m, q)  at  m*UA + (q ^ ((m / (16/UA)) % UA)),      UA = BK/8 units per row
//   B unit (k, u)  at  k*UB + (u ^ (4 * (k & 3))),              UB = BN/8 units per row
// A fragments (8 consecutive k of one row per lane) are plain ds_read_b128.  B fragments need 8 consecutive k of one
// COLUMN per lane, i.e. a transpose of the row-major tile: ds_read_b64_tr_b16 does it inside the LDS read (each group
// of 16 lanes reads a 4(k) x 16(n) block, lane i of the group receives column i), two reads per fragment.
//
// Ragged edges as in the fp32 tile: rows / columns beyond the matrix are read from clamped addresses and never
// stored, only the last partial K step zero-fills.  The fp32 accumulator is rounded to binary16 (nearest even) once,
// when it is stored.
#pragma once
#include "tile_common.hpp"

namespace decx_hip {

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_>
struct HgemmShape {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NT = WAVES_M * WAVES_N * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int UA = BK / 8, UB = BN / 8;           // 16-byte units per LDS row
    static constexpr int A_UNITS = BM * UA, B_UNITS = BK * UB;
    static constexpr int A_PASSES = A_UNITS / NT, B_PASSES = B_UNITS / NT;
    static constexpr size_t LDS_BYTES = 2 * (size_t)(A_UNITS + B_UNITS) * 16;
    static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(BK % 16 == 0 && (UA == 2 || UA == 4 || UA == 8), "K step is whole MFMA k-blocks");
    static_assert(UB >= 16 && (UB & (UB - 1)) == 0, "B swizzle needs >= 16 units per row");
    static_assert(A_UNITS % NT == 0 && B_UNITS % NT == 0, "staging must divide evenly");
};

__device__ __forceinline__ int a_unit_slot(int m, int q, int UA) { return m * UA + (q ^ ((m / (16 / UA)) % UA)); }
__device__ __forceinline__ int b_unit_slot(int k, int u, int UB) { return k * UB + (u ^ ((k & 3) << 2)); }

template <class S, bool VEC>
__global__ __launch_bounds__(S::NT) void hgemm_tile_kernel(const _Float16* __restrict__ A, int lda,
                                                           const _Float16* __restrict__ B, int ldb, const _Float16* Cin,
                                                           int ldc, _Float16* D, int ldd, int M, int N, int K,
                                                           int tiles_m, int tiles_n, int group_m, size_t a_batch_stride,
                                                           size_t b_batch_stride, size_t c_batch_stride, size_t d_batch_stride) {
    // blockIdx.y walks a batch of independent problems of the same shape
    A += (size_t)blockIdx.y * a_batch_stride;
    B += (size_t)blockIdx.y * b_batch_stride;
    if (Cin != nullptr) Cin += (size_t)blockIdx.y * c_batch_stride;
    D += (size_t)blockIdx.y * d_batch_stride;
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, NT = S::NT, UA = S::UA, UB = S::UB, MI = S::MI, NI = S::NI;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    u32x4* As = reinterpret_cast<u32x4*>(lds_raw);            // [2][A_UNITS]
    u32x4* Bs = As + 2 * S::A_UNITS;                          // [2][B_UNITS]

    const TileCoord tc = xcd_grouped_tile(blockIdx.x, tiles_m, tiles_n, group_m);
    const int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;

    u32x4 a_stage[S::A_PASSES], b_stage[S::B_PASSES];

    auto load_unit = [&](const _Float16* row, int k, int kvalid, bool tail) -> u32x4 {
        // 8 halves row[k..k+7]; elements at or beyond kvalid read as zero when tail
        u32x4 v = {0u, 0u, 0u, 0u};
        if (VEC) {
            if (!tail) return *reinterpret_cast<const u32x4*>(row + k);
            if (k < kvalid) {
                v = *reinterpret_cast<const u32x4*>(row + k);
                const int keep = kvalid - k;                  // 1..8 halves are real
                if (keep < 8) {
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const int e = 2 * w;
                        uint32_t mask = (e + 1 < keep) ? 0xffffffffu : (e < keep ? 0x0000ffffu : 0u);
                        v[w] &= mask;
                    }
                }
            }
        } else {
            const uint16_t* r16 = reinterpret_cast<const uint16_t*>(row);
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (k + e < kvalid) v[e >> 1] |= (uint32_t)r16[k + e] << ((e & 1) * 16);
        }
        return v;
    };

    auto load_stage = [&](int k0, bool tail) {
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) {
            const int id = tid + p * NT;
            const int r = id / UA, q = id % UA;
            int m = bm0 + r;
            if (m >= M) m = M - 1;
            a_stage[p] = load_unit(A + (size_t)m * lda, k0 + 8 * q, K, tail);
        }
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) {
            const int id = tid + p * NT;
            const int kr = id / UB, u = id % UB;
            const int k = k0 + kr;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (!tail || k < K) {
                const int col = bn0 + 8 * u;
                if (VEC) {
                    const int cc = clamp_group_col(col, N, 8);    // stay inside the operand; such columns are never stored
                    v = *reinterpret_cast<const u32x4*>(B + (size_t)k * ldb + cc);
                } else {
                    v = load_unit(B + (size_t)k * ldb, col, N, true);
                }
            }
            b_stage[p] = v;
        }
    };

    auto store_stage = [&](int buf) {
        u32x4* Ab = As + buf * S::A_UNITS;
        u32x4* Bb = Bs + buf * S::B_UNITS;
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
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;
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

    const int full_steps = K / BK;
    const int steps = (K + BK - 1) / BK;

    // transposed-read geometry of this lane: group g of 16 lanes reads rows kb+j (j = 0..3), 4 columns each
    const int tg = lane >> 4, ts = lane & 15;
    const int t_row = 8 * (tg >> 1) + (ts >> 2);              // + 16*kstep (+4 for the second read)
    const int t_col = 16 * (tg & 1) + 4 * (ts & 3);           // + wn0 + 32*ni

    load_stage(0, full_steps == 0);
    store_stage(0);
    __syncthreads();

    for (int t = 0; t < steps; ++t) {
        const int buf = t & 1;
        if (t + 1 < steps) load_stage((t + 1) * BK, t + 1 >= full_steps);
        const u32x4* Ab = As + buf * S::A_UNITS;
        const unsigned char* Bb = reinterpret_cast<const unsigned char*>(Bs + buf * S::B_UNITS);
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
                i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) i16x4*)(Bb + off_lo));
                i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) i16x4*)(Bb + off_hi));
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
        if (t + 1 < steps) {
            store_stage(buf ^ 1);
            __syncthreads();
        }
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

// D = half(plane 0 + plane 1 + ... + C), added in that order: the end of a split-K product (hgemm_dma_kernel with
// SPLIT_K).  partial holds `planes` dense M x N fp32 planes, `plane` floats apart (one plane in the atomic mode).
static __global__ __launch_bounds__(256) void hgemm_split_finish_kernel(const float* __restrict__ partial, int planes, size_t plane,
                                                                 const _Float16* Cin, int ldc, _Float16* D, int ldd, int M, int N) {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / N, n = i - m * N;
        float v = ordered_plane_sum(partial, planes, plane, i);
        if (Cin != nullptr) v += (float)Cin[m * ldc + n];
        D[m * ldd + n] = (_Float16)v;
    }
}

}  // namespace decx_hip
