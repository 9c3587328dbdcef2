// fp32 GEMM for problems with few output tiles and a long K: one wave per 16x16 block of the result.
//
// Every output of the reference is one fused multiply-add chain over ascending k, and a chain cannot be cut into
// parallel pieces without changing its rounding.  What bounds a long, thin problem (say 64 x 65536 x 1024) is then how
// fast ONE accumulator can walk K.  v_mfma_f32_16x16x4_f32 consumes four k per instruction -- per output element
// fma(a3,b3, fma(a2,b2, fma(a1,b1, fma(a0,b0, c)))) with k-slot s taken from lanes 16s .. 16s+15 (checked bit for bit on
// the hardware) -- and dependent instructions issue back to back every 32 cycles, i.e. 8 cycles per k, four times the
// pace of the 32x32x2 form the big tiles use.  The big tiles win on everything else (16 times the reuse per operand
// byte), so this kernel is only chosen when the result has too few tiles to fill the chip anyway.
//
// Nothing but the MFMAs may sit on that chain, and on this hardware every other instruction does: measured per chunk of
// 16 MFMAs (518 cycles alone), the wave's own eight 16-byte LDS reads add 55 cycles, and with loads, LDS stores and
// address arithmetic in the same wave the chunk took 970 -- the sum of everybody's issue time, bank conflicts or not.
// Instructions of ANOTHER wave on the same SIMD cost the chain about as much (+210 cycles for the 25 instructions that
// stage a chunk); only a wave on another SIMD is free.  So the work is split by role.  Computing waves do per chunk of
// 64 k the 16 MFMAs and the 8 LDS reads of the next chunk's operands, nothing else; moving waves bring the data: global
// memory -> DEPTH register sets -> LDS, DEPTH chunks ahead.  Three LDS buffers: while chunk c is computed from
// registers, chunk c+1 is read from one buffer and chunk c+2 written into another; one barrier per chunk (free: the
// moving waves are always early).  Two shapes:
//   T = 1: a 16x16 tile, one computing wave and two moving waves -- three waves on three different SIMDs of a CU, so
//          the chain runs undisturbed: for results of at most one block per CU (241 ns per chunk, against 218 for bare
//          MFMAs);
//   1 x 2: a 16x32 tile, two computing and two moving waves -- four waves on the four SIMDs of a CU, the chains as
//          undisturbed as in the 16x16 shape, A staged once for both blocks and B in whole 128-byte lines: for results
//          of more than one 16x16 block per CU but at most one such tile (14x14x512 under 512 filters: 208 tiles);
//   T = 2: a 32x32 tile, 2x2 computing waves and four moving waves, one of each per SIMD: half the staging work per
//          block (A and B tiles are shared) but it runs on the computing waves' SIMDs: for more blocks than CUs.  Built
//          with 4 register sets for 128 registers, so that two workgroups share a CU and one's MFMAs fill the gaps
//          the other's staging leaves;
//   T = 4: a 64x64 tile, eight computing waves of two blocks each (two chains per wave, interleaved, one set of A
//          operands for both) and four moving waves: a quarter of the staging work per block, and four chains per SIMD
//          keep its matrix pipe busy while one of them waits: for results of about one such tile per CU and more.
//
// Lane (r, s) of a computing wave feeds row r (of A) or column r (of B) of its block and k-slot s; so that its operands
// for the 16 MFMAs of a chunk (k = 4j + s, j = 0..15) are 16 consecutive floats -- four 16-byte reads -- the chunk lies in
// LDS as  As[s][row][j]  and  Bs[s][col][j]  with lines of 20 floats (16 lanes of a 16-byte read then cover all banks).
// The moving waves scatter each loaded quad into that layout with ds_write2 pairs; quads are dealt to lanes, and B's
// planes padded by 4 floats, so that the 32 lanes of one store pass fall on 32 different banks.  The k order inside an
// instruction (slot 0..3) and across instructions (j) is ascending, so results are bit-identical to
// sgemm_tile_kernel's and to the reference's chain.
//
// Loads never run past the last whole chunk: the fetch pointers stop advancing there (later refills fetch that chunk
// again and are never used), which keeps the loop free of bounds checks.  A ragged last chunk is fetched with masks once,
// at the start, into registers of its own, and computed after the loop.
#pragma once
#include "sgemm_tile.hpp"

namespace decx_hip {

// TM x TN blocks of 16x16 per workgroup tile; a computing wave owns NB blocks that lie side by side (NB independent chains,
// interleaved, sharing the A operands); DEPTH_ register sets; WAVES_PER_SIMD_ is what the register budget is cut for.
template <int TM, int TN, int NB_, int DEPTH_, int WAVES_PER_SIMD_>
struct Chain16Rect {
    static_assert((TM == 1 || TM == 2 || TM == 4) && (TN == 1 || TN == 2 || TN == 4) && TN % NB_ == 0, "tiles of 1, 2 or 4 blocks a side");
    static constexpr int WAVES_PER_SIMD = WAVES_PER_SIMD_;
    static constexpr int BM = 16 * TM, BN = 16 * TN, BK = 64, NB = NB_;
    static constexpr int COMPUTE_WAVES = TM * TN / NB, MOVE_THREADS = TM * TN <= 2 ? 128 : 256;
    static constexpr int NT = 64 * COMPUTE_WAVES + MOVE_THREADS;     // computing waves first, then the moving waves
    static constexpr int PA = 16 * BM / MOVE_THREADS, PB = 16 * BN / MOVE_THREADS;   // quads of A and of B per moving thread and chunk
    static constexpr int DEPTH = DEPTH_;                             // register sets: chunks of K in flight from global memory (even)
    static constexpr int LINE = 20;                                  // floats per (k-slot, row or column) line in LDS: 16 + 4
    static constexpr int A_PLANE = BM * LINE, B_PLANE = BN * LINE + 4;   // floats per k-slot plane
    static constexpr int A_FLOATS = 4 * A_PLANE, B_FLOATS = 4 * B_PLANE;
    static constexpr int LDS_BUFFERS = 3;
    static constexpr size_t LDS_BYTES = LDS_BUFFERS * (size_t)(A_FLOATS + B_FLOATS) * sizeof(float);
    static_assert(16 * BM % MOVE_THREADS == 0 && 16 * BN % MOVE_THREADS == 0 && NT <= 1024, "staging divides evenly");
};
template <int T, int NB_, int DEPTH_, int WAVES_PER_SIMD_>
using Chain16 = Chain16Rect<T, T, NB_, DEPTH_, WAVES_PER_SIMD_>;

// two floats to LDS, OFF0 and OFF1 dwords past byte_addr (each below 256)
template <int OFF0, int OFF1>
__device__ __forceinline__ void lds_write2(unsigned byte_addr, float x, float y) {
    asm volatile("ds_write2_b32 %0, %1, %2 offset0:%3 offset1:%4" : : "v"(byte_addr), "v"(x), "v"(y), "n"(OFF0), "n"(OFF1) : "memory");
}
// the same with offsets in units of 64 dwords
template <int OFF0, int OFF1>
__device__ __forceinline__ void lds_write2_st64(unsigned byte_addr, float x, float y) {
    asm volatile("ds_write2st64_b32 %0, %1, %2 offset0:%3 offset1:%4" : : "v"(byte_addr), "v"(x), "v"(y), "n"(OFF0), "n"(OFF1) : "memory");
}

// The computing side of a workgroup: walks the chunks the moving waves put into LDS and returns with the finished
// accumulators.  full_chunks chunks arrive through the three-buffer pipeline (one barrier after the prologue, one per
// chunk); if chunks > full_chunks one more, ragged, chunk arrives in buffer 0 behind a barrier of its own.
template <class S>
__device__ __forceinline__ void chain16_consume(const float* As, const float* Bs, int wm0, int wn0, int lr, int ls, int full_chunks,
                                                int chunks, f32x4 (&acc)[S::NB]) {
    constexpr int NB = S::NB;
    typedef std::integral_constant<int, 0> I0;
    const float* a_frag = As + ls * S::A_PLANE + (wm0 + lr) * S::LINE;       // this lane's 16 operands of a chunk, buffer 0
    const float* b_frag = Bs + ls * S::B_PLANE + (wn0 + lr) * S::LINE;       // block b: 16 lines further per block
    f32x4 av[2][4], bv[2][NB][4];
    constexpr int READS = 4 + 4 * NB;             // 16-byte operand reads per chunk: 4 of A, then 4 per block of B
    auto read_one = [&](auto f_tag, auto r_tag, int buf) {
        constexpr int F = decltype(f_tag)::value, R = decltype(r_tag)::value;
        if constexpr (R < 4) av[F][R] = reinterpret_cast<const f32x4*>(a_frag + buf * S::A_FLOATS)[R];
        else bv[F][(R - 4) / 4][(R - 4) % 4] = reinterpret_cast<const f32x4*>(b_frag + buf * S::B_FLOATS + ((R - 4) / 4) * 16 * S::LINE)[(R - 4) % 4];
    };
    if (full_chunks > 0) {
        lds_sync();
        static_for<0, READS>([&](auto r) { read_one(I0{}, r, 0); });
        // chunk c: its operands are in fragment set c % 2; buffer (c+1) % 3 holds chunk c+1 since the previous barrier.
        // The NB chains advance in turn; behind each of the first READS MFMAs goes one read of the next chunk's operands.
        // The walk is unrolled by 6, the period of set and buffer together, so that every read has its address in the
        // instruction: with the buffer in a register (an unroll by 2, 4 or 8) each read needs an addition first, and
        // on a wave that is one dependent chain that costs 8 % of the pace (64x65536x1024: 0.268 -> 0.260 ms, 256x8192x256:
        // 34.2 -> 30.9 us).
        constexpr int UNROLL = 6;
        auto chunk = [&](auto d) {
            constexpr int NOW = decltype(d)::value & 1, BUF_NEXT = (decltype(d)::value + 1) % 3;
            typedef std::integral_constant<int, NOW ^ 1> Next;
            static_for<0, 16 * NB>([&](auto i_tag) {
                constexpr int I = decltype(i_tag)::value, J = I / NB, BLK = I % NB;
                acc[BLK] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[NOW][J / 4][J % 4], bv[NOW][BLK][J / 4][J % 4], acc[BLK], 0, 0, 0);
                if constexpr (I < READS) read_one(Next{}, i_tag, BUF_NEXT);
                __builtin_amdgcn_sched_barrier(0);
            });
            lds_sync();
            __builtin_amdgcn_sched_barrier(0);
        };
        int c0 = 0;
        for (; c0 + UNROLL <= full_chunks; c0 += UNROLL) static_for<0, UNROLL>([&](auto d) { chunk(d); });
        static_for<0, UNROLL>([&](auto d) {
            if (c0 + decltype(d)::value < full_chunks) chunk(d);
        });
    }
    if (chunks > full_chunks) {
        lds_sync();
        static_for<0, READS>([&](auto r) { read_one(I0{}, r, 0); });
#pragma unroll
        for (int j = 0; j < 16; ++j)
#pragma unroll
            for (int b = 0; b < NB; ++b)
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[0][j / 4][j % 4], bv[0][b][j / 4][j % 4], acc[b], 0, 0, 0);
    }
}

template <class S, bool HAS_C>
__global__ __launch_bounds__(S::NT, S::WAVES_PER_SIMD) void sgemm_chain16_kernel(const float* __restrict__ A, int lda,
                                                                    const float* __restrict__ B, int ldb, const float* Cin,
                                                                    int ldc, float* D, int ldd, int M, int N, int K,
                                                                    int tiles_n, bool relu, size_t a_batch_stride,
                                                                    size_t b_batch_stride, size_t c_batch_stride,
                                                                    size_t d_batch_stride) {
    constexpr int DEPTH = S::DEPTH, NB = S::NB, PA = S::PA, PB = S::PB, Q_ALL = S::PA + S::PB;
    static_assert(DEPTH % 2 == 0 && DEPTH >= 2, "set and fragment indices repeat with period DEPTH");
    static_assert(S::A_PLANE % 64 == 0 && S::LINE == 20, "the store offsets below are written for these strides");
    A += (size_t)blockIdx.y * a_batch_stride;
    B += (size_t)blockIdx.y * b_batch_stride;
    if (HAS_C) Cin += (size_t)blockIdx.y * c_batch_stride;
    D += (size_t)blockIdx.y * d_batch_stride;
    extern __shared__ __attribute__((aligned(16))) float lds[];      // LDS_BYTES
    float* As = lds;                                     // [3][4 slots][BM][LINE]
    float* Bs = lds + S::LDS_BUFFERS * S::A_FLOATS;      // [3][4 slots][BN][LINE] (+4 per plane)

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int bm0 = ((int)blockIdx.x / tiles_n) * S::BM, bn0 = ((int)blockIdx.x % tiles_n) * S::BN;
    const int chunks = (K + S::BK - 1) / S::BK, full_chunks = K / S::BK;
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    // Both roles run the same sequence of barriers: one after the prologue (when there is a whole chunk), one per whole
    // chunk, one for a ragged last chunk.
    if (wave >= S::COMPUTE_WAVES) {
        // =============================== moving waves ===============================
        // per chunk PA quads of A (row, 4 consecutive k) and PB of B (k, 4 consecutive columns) per thread; quads 0 .. PA-1
        // are A's, the rest B's.  32 consecutive lanes hold, of A, 16 quads of rows r and r + 4 (banks 20 r + kq and 16
        // further), of B, 16 consecutive k of two neighbouring column quads (banks 4 (k % 4) + k / 4 and 16 further).
        const int pt = tid - 64 * S::COMPUTE_WAVES;
        const float* src[Q_ALL];
        unsigned dst[Q_ALL];                      // LDS byte address, buffer 0, of element 0 of the quad
        int quad_k[Q_ALL];                        // k of the quad inside its chunk (first element for A)
#pragma unroll
        for (int p = 0; p < PA; ++p) {
            const int q = pt + p * S::MOVE_THREADS, rest = q / 32;
            const int row = rest % 4 + 4 * ((q / 16) % 2) + 8 * (rest / 4), kq = q % 16;
            int m = bm0 + row;
            if (m >= M) m = M - 1;                // rows past the end are computed and never stored
            quad_k[p] = 4 * kq;
            src[p] = A + (size_t)m * lda + 4 * kq;
            dst[p] = lds_byte_address(As) + 4u * (unsigned)(row * S::LINE + kq);      // element e: plane e, j = kq
        }
#pragma unroll
        for (int p = 0; p < PB; ++p) {
            const int q = pt + p * S::MOVE_THREADS;
            const int k = (q / 4) % 64, cq = 4 * (q / 256) + q % 4;
            int col = bn0 + 4 * cq;
            col = clamp_group_col(col, N, 4);     // stay inside the operand; such columns are never stored
            quad_k[PA + p] = k;
            src[PA + p] = B + (size_t)k * ldb + col;
            dst[PA + p] = lds_byte_address(Bs) + 4u * (unsigned)((k % 4) * S::B_PLANE + (4 * cq) * S::LINE + k / 4);   // element e: line 4cq + e
        }
        auto store_quad = [&](const f32x4& v, auto quad_tag, int buf) {
            constexpr int Q = decltype(quad_tag)::value;
            if constexpr (Q < PA) {
                const unsigned addr = dst[Q] + (unsigned)buf * (S::A_FLOATS * 4u);
                lds_write2_st64<0, S::A_PLANE / 64>(addr, v[0], v[1]);
                lds_write2_st64<2 * S::A_PLANE / 64, 3 * S::A_PLANE / 64>(addr, v[2], v[3]);
            } else {
                const unsigned addr = dst[Q] + (unsigned)buf * (S::B_FLOATS * 4u);
                lds_write2<0, S::LINE>(addr, v[0], v[1]);
                lds_write2<2 * S::LINE, 3 * S::LINE>(addr, v[2], v[3]);
            }
        };

        // the ragged last chunk, fetched first (it is the only load with per-lane conditions)
        f32x4 tail_stage[Q_ALL];
        if (chunks > full_chunks) {
            const int k0 = full_chunks * S::BK;
#pragma unroll
            for (int p = 0; p < Q_ALL; ++p) {
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                const int k = k0 + quad_k[p];
                if (k < K) {
                    if (p < PA) {
                        v = *reinterpret_cast<const f32x4*>(src[p] + k0);        // lda % 4 == 0 keeps the quad inside the pitch
                        if (k + 1 >= K) v[1] = 0.f;
                        if (k + 2 >= K) v[2] = 0.f;
                        if (k + 3 >= K) v[3] = 0.f;
                    } else {
                        v = *reinterpret_cast<const f32x4*>(src[p] + (size_t)k0 * ldb);
                    }
                }
                tail_stage[p] = v;
            }
        }

        // DEPTH register sets: chunk x travels through set x % DEPTH, fetched DEPTH chunks ahead of its use
        f32x4 stage[DEPTH][Q_ALL];
        int fetch_chunk = 0;                      // the chunk the fetch pointers stand on
        auto fetch = [&](auto set_tag) {
            constexpr int SET = decltype(set_tag)::value;
            const bool more = fetch_chunk + 1 < full_chunks;      // the pointers stop on the last whole chunk
            const long a_step = more ? S::BK : 0, b_step = more ? (long)S::BK * ldb : 0;
            fetch_chunk += more ? 1 : 0;
            static_for<0, Q_ALL>([&](auto q_tag) {
                constexpr int Q = decltype(q_tag)::value;
                stage[SET][Q] = *reinterpret_cast<const f32x4*>(src[Q]);
                src[Q] += Q < PA ? a_step : b_step;
            });
        };
        if (full_chunks > 0) {
            // chunks 0 .. DEPTH-1 are fetched; chunks 0 and 1 go to LDS buffers 0 and 1 and their sets are refilled
            static_for<0, DEPTH>([&](auto d) { fetch(d); });
            static_for<0, Q_ALL>([&](auto q) { store_quad(stage[0][decltype(q)::value], q, 0); });
            static_for<0, Q_ALL>([&](auto q) { store_quad(stage[1][decltype(q)::value], q, 1); });
            lds_sync();
            fetch(I0{});
            fetch(I1{});
            // while chunk c is computed: chunk c+2 goes into buffer (c+2) % 3 (it held chunk c-1, which nobody reads any
            // more), and once the stores have left the registers, the set is refilled with chunk c+2+DEPTH
            int buf_store = 2;
            auto chunk = [&](auto d) {
                constexpr int SET = (decltype(d)::value + 2) % DEPTH;
                static_for<0, Q_ALL>([&](auto q) { store_quad(stage[SET][decltype(q)::value], q, buf_store); });
                lds_sync();
                fetch(std::integral_constant<int, SET>{});
                buf_store = buf_store == 2 ? 0 : buf_store + 1;
            };
            int c0 = 0;
            for (; c0 + DEPTH <= full_chunks; c0 += DEPTH) static_for<0, DEPTH>([&](auto d) { chunk(d); });
            // c0 is a multiple of DEPTH, so the set indices continue with the same period
            static_for<0, DEPTH>([&](auto d) {
                if (c0 + decltype(d)::value < full_chunks) chunk(d);
            });
        }
        if (chunks > full_chunks) {
            // every computing wave is past the last barrier and has all its LDS reads back: any buffer is free
            static_for<0, Q_ALL>([&](auto q) { store_quad(tail_stage[decltype(q)::value], q, 0); });
            lds_sync();
        }
        return;
    }

    // =============================== computing waves ===============================
    constexpr int WAVES_N = S::BN / (16 * NB);
    const int wm0 = (wave / WAVES_N) * 16, wn0 = (wave % WAVES_N) * 16 * NB;
    const int lr = lane % 16, ls = lane / 16;     // row (of A) or column (of B) inside a block, and k-slot
    // accumulators: lane holds D[4*ls + r][lr] of each of its blocks, r = 0..3; the chains start at C when there is one
    f32x4 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
        const int n_out = bn0 + wn0 + 16 * b + lr;
        if (HAS_C) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = bm0 + wm0 + 4 * ls + r;
                if (m < M && n_out < N) acc[b][r] = Cin[(size_t)m * ldc + n_out];
            }
        }
    }
    chain16_consume<S>(As, Bs, wm0, wn0, lr, ls, full_chunks, chunks, acc);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int n_out = bn0 + wn0 + 16 * b + lr;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int m = bm0 + wm0 + 4 * ls + r;
            if (m < M && n_out < N) D[(size_t)m * ldd + n_out] = relu ? relu_by_sign(acc[b][r]) : acc[b][r];
        }
    }
}

}  // namespace decx_hip
