// The fused im2col convolution on the one-wave-per-16x16-block kernel of sgemm_chain16.hpp, for small images.
//
// A convolution of a 14x14x512 image with 512 filters is a 196 x 4608 x 512 product: two tiles of the big kernel, on
// two of 256 CUs.  The block-chain kernel gives every 16x16 block of the result a wave and is bound by the walk over K
// alone; its moving waves are off that walk, so the im2col address arithmetic (tap decoding, bounds tests) costs the
// chains nothing.  Same arithmetic as everywhere: one fused chain per output over k = (ki*kw + kj)*dpitch + c ascending,
// then bias and ReLU -- results are bit-identical to the tile kernel's and to the reference's.
//
// Moving waves: a quad of A is 4 channels of one tap of one pixel (one 16-byte buffer load; out-of-image taps and k >= K
// get an out-of-range offset, which the hardware answers with zeros, so there is no ragged last chunk to treat apart);
// a quad of B is 4 consecutive k of one filter, which is contiguous in the filter bank: both go into LDS the way A does
// in the dense kernel (element e to k-slot plane e).  All quads of a thread share their place inside the chunk, so one
// tap walk per operand serves them all.
#pragma once
#include "sgemm_chain16.hpp"

namespace decx_hip {

template <int OFF_BYTES>
__device__ __forceinline__ void lds_write1(unsigned byte_addr, float x) {
    asm volatile("ds_write_b32 %0, %1 offset:%2" : : "v"(byte_addr), "v"(x), "n"(OFF_BYTES) : "memory");
}

template <class S>
__global__ __launch_bounds__(S::NT, S::WAVES_PER_SIMD) void conv_chain16_kernel(Im2colA<false> img, FilterB<false> fb,
                                                                                const float* bias, float* dst, TensorOut out,
                                                                                int M, int N, int K, int tiles_n) {
    constexpr int DEPTH = S::DEPTH, NB = S::NB, PA = S::PA, PB = S::PB, Q_ALL = S::PA + S::PB;
    static_assert(DEPTH % 2 == 0 && DEPTH >= 2, "set and fragment indices repeat with period DEPTH");
    static_assert(S::A_PLANE % 64 == 0 && S::LINE == 20 && S::MOVE_THREADS % 32 == 0, "the store offsets below are written for these strides");
    extern __shared__ __attribute__((aligned(16))) float lds[];      // LDS_BYTES
    float* As = lds;                                     // [3][4 slots][BM][LINE]
    float* Bs = lds + S::LDS_BUFFERS * S::A_FLOATS;      // [3][4 slots][BN][LINE] (+4 per plane)

    const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
    const int bm0 = ((int)blockIdx.x / tiles_n) * S::BM, bn0 = ((int)blockIdx.x % tiles_n) * S::BN;
    const int chunks = (K + S::BK - 1) / S::BK;          // every chunk is a whole one: what lies past K reads as zero
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;

    if (wave >= S::COMPUTE_WAVES) {
        // =============================== moving waves ===============================
        // quad q of an operand: row (pixel, or filter) as in the dense kernel -- 32 consecutive lanes hold 16 quads of
        // rows r and r + 4 --, place q % 16 inside the chunk; MOVE_THREADS is a multiple of 16, so the place is the
        // same for every quad of a thread
        const int pt = tid - 64 * S::COMPUTE_WAVES, kq = pt % 16;
        Im2colA<false>::RowState pix[PA];
        int filter_base[PB];
        unsigned dst_lds[Q_ALL];                  // LDS byte address, buffer 0, of element 0 of the quad
#pragma unroll
        for (int p = 0; p < (PA > PB ? PA : PB); ++p) {
            const int q = pt + p * S::MOVE_THREADS, rest = q / 32;
            const int row = rest % 4 + 4 * ((q / 16) % 2) + 8 * (rest / 4);
            if (p < PA) {
                pix[p] = img.row_state(bm0 + row);                     // clamps pixels past the end: computed, never stored
                dst_lds[p] = lds_byte_address(As) + 4u * (unsigned)(row * S::LINE + kq);
            }
            if (p < PB) {
                int n = bn0 + row;
                if (n >= N) n = N - 1;
                filter_base[p] = 4 * n * fb.filt_stride;
                dst_lds[PA + p] = lds_byte_address(Bs) + 4u * (unsigned)(row * S::LINE + kq);
            }
        }
        TapWalk wa, wb;                           // this thread's place in the chunk to fetch next: in the image, in a filter
        wa.init(4 * kq, img.dpitch, img.kw, img.row_stride);
        wb.init(4 * kq, fb.dpitch, fb.kw, fb.filt_row_stride);
        const TapStep sa = TapStep::make(S::BK, img.dpitch, img.kw, img.row_stride);
        const TapStep sb = TapStep::make(S::BK, fb.dpitch, fb.kw, fb.filt_row_stride);

        f32x4 stage[DEPTH][Q_ALL];
        auto fetch = [&](auto set_tag) {
            constexpr int SET = decltype(set_tag)::value;
            const bool k_ok = wb.k < K;
#pragma unroll
            for (int p = 0; p < PA; ++p)
                stage[SET][p] = buffer_load_quad(make_rsrc(img.src, img.bytes), img.template quad_offset<true>(pix[p], wa));
#pragma unroll
            for (int p = 0; p < PB; ++p)
                stage[SET][PA + p] = buffer_load_quad(make_rsrc(fb.filt, fb.bytes), k_ok ? (unsigned)(filter_base[p] + wb.off) : kOutOfRange);
            wa.advance(sa, img.dpitch, img.kw);
            wb.advance(sb, fb.dpitch, fb.kw);
        };
        auto store_quad = [&](const f32x4& v, auto quad_tag, int buf) {
            constexpr int Q = decltype(quad_tag)::value;
            if constexpr (Q < PA) {
                const unsigned addr = dst_lds[Q] + (unsigned)buf * (S::A_FLOATS * 4u);
                lds_write2_st64<0, S::A_PLANE / 64>(addr, v[0], v[1]);
                lds_write2_st64<2 * S::A_PLANE / 64, 3 * S::A_PLANE / 64>(addr, v[2], v[3]);
            } else {
                const unsigned addr = dst_lds[Q] + (unsigned)buf * (S::B_FLOATS * 4u);
                lds_write1<0>(addr, v[0]);
                lds_write1<4 * S::B_PLANE>(addr, v[1]);
                lds_write1<8 * S::B_PLANE>(addr, v[2]);
                lds_write1<12 * S::B_PLANE>(addr, v[3]);
            }
        };
        // the schedule of the dense kernel: chunks 0 .. DEPTH-1 fetched, 0 and 1 stored and their sets refilled; then per
        // chunk c the stores of chunk c+2, the barrier, and the refill of that set with chunk c+2+DEPTH
        static_for<0, DEPTH>([&](auto d) { fetch(d); });
        static_for<0, Q_ALL>([&](auto q) { store_quad(stage[0][decltype(q)::value], q, 0); });
        static_for<0, Q_ALL>([&](auto q) { store_quad(stage[1][decltype(q)::value], q, 1); });
        lds_sync();
        fetch(I0{});
        fetch(I1{});
        int buf_store = 2;
        auto chunk = [&](auto d) {
            constexpr int SET = (decltype(d)::value + 2) % DEPTH;
            static_for<0, Q_ALL>([&](auto q) { store_quad(stage[SET][decltype(q)::value], q, buf_store); });
            lds_sync();
            fetch(std::integral_constant<int, SET>{});
            buf_store = buf_store == 2 ? 0 : buf_store + 1;
        };
        int c0 = 0;
        for (; c0 + DEPTH <= chunks; c0 += DEPTH) static_for<0, DEPTH>([&](auto d) { chunk(d); });
        static_for<0, DEPTH>([&](auto d) {
            if (c0 + decltype(d)::value < chunks) chunk(d);
        });
        return;
    }

    // =============================== computing waves ===============================
    constexpr int WAVES_N = S::BN / (16 * NB);
    const int wm0 = (wave / WAVES_N) * 16, wn0 = (wave % WAVES_N) * 16 * NB;
    const int lr = lane % 16, ls = lane / 16;
    f32x4 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    chain16_consume<S>(As, Bs, wm0, wn0, lr, ls, chunks, chunks, acc);
    // lane holds dst(pixel bm0 + wm0 + 4 ls + r, filter bn0 + wn0 + 16 b + lr); a bias joins the finished sum
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int m = bm0 + wm0 + 4 * ls + r;
        if (m < M) {
            float* pixel = dst + out.offset(m);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int n = bn0 + wn0 + 16 * b + lr;
                if (n < N) pixel[n] = out.finish(bias != nullptr ? acc[b][r] + bias[n] : acc[b][r]);
            }
        }
    }
}

}  // namespace decx_hip
