// fp16 convolution (fp32 accumulate) as a GEMM whose A tile is read straight from the image: the fp16 twin of the fused
// im2col path of sgemm_tile.hpp, on v_mfma_f32_32x32x16_f16.
//
//   dst(y, x, n) = sum over k = (ki*kw + kj)*dpitch + c  of  src(y + ki - oy, x + kj - ox, c) * filt(n, ki, kj, c)
//
// Both operands are contiguous along k: 8 consecutive channels of one tap are one 16-byte unit of the image (the
// channel pitch of a binary16 tensor is a multiple of 8, Tensor.h:214-235) and of filter n.  So there is no transpose
// anywhere: a staging unit is one 16-byte buffer load (out-of-image taps and the K tail get an out-of-range offset,
// which the hardware answers with zeros), LDS holds A as [pixel][k-unit] and B as [filter][k-unit] with the unit index
// XOR-swizzled by the row (a_unit_slot), and both MFMA operands -- 8 consecutive k of one row per lane -- are plain
// ds_read_b128.  The walk over k reuses TapWalk in units of 4 bytes (two halves): positions, pitches and strides of a
// binary16 tensor are all even.
//
// Products are accumulated in fp32 in the MFMA's own order (not the scalar chain of the fp32 path: there is no binary16
// reference result to be bit-identical to) and rounded to binary16, nearest even, once, after the optional bias and ReLU.
#pragma once
#include "hgemm_tile.hpp"
#include "sgemm_tile.hpp"

namespace decx_hip {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct HconvShape {
    static constexpr int BM = BM_, BN = BN_, BK = 64, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NT = WAVES_M * WAVES_N * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int U = BK / 8;                          // 16-byte units per row and K step
    static constexpr int A_UNITS = BM * U, B_UNITS = BN * U;
    static constexpr int A_PASSES = A_UNITS / NT, B_PASSES = B_UNITS / NT, ROWS_PER_PASS = NT / U;
    static constexpr size_t LDS_BYTES = 2 * (size_t)(A_UNITS + B_UNITS) * 16;
    static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(A_UNITS % NT == 0 && B_UNITS % NT == 0 && NT % U == 0, "staging must divide evenly");
};

// the image: all strides in 4-byte words (pairs of halves)
struct HalfImage {
    const void* src;
    int H, W, kh, kw, oy, ox, Wout, Mtot;
    int dpitch_w, row_stride_w;
    unsigned bytes;
};
// the filter bank: filter n starts n*filt_stride_w words in, its tap rows are row_stride_w words apart
struct HalfFilters {
    const void* filt;
    int N, dpitch_w, kw, filt_stride_w, row_stride_w;
    unsigned bytes;
};
struct HalfTensorOut {
    _Float16* dst;
    int Wout, dpitch;            // halves per pixel of dst
    size_t row_stride;           // halves between image rows of dst
    const _Float16* bias;        // N values or nullptr
    bool relu;
};

template <class S>
__global__ __launch_bounds__(S::NT) void hconv_tile_kernel(HalfImage img, HalfFilters fb, HalfTensorOut out, int M, int N,
                                                           int Kw /* K in words */, int tiles_n) {
    constexpr int BM = S::BM, BN = S::BN, NT = S::NT, U = S::U, MI = S::MI, NI = S::NI;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    u32x4* As = reinterpret_cast<u32x4*>(lds_raw);            // [2][A_UNITS]
    u32x4* Bs = As + 2 * S::A_UNITS;                          // [2][B_UNITS]

    const int bm0 = ((int)blockIdx.x / tiles_n) * BM, bn0 = ((int)blockIdx.x % tiles_n) * BN;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;

    // staging: this thread moves unit q of rows r0, r0 + ROWS_PER_PASS, ... of either operand
    const int q = tid % U, r0 = tid / U;
    int a_y[S::A_PASSES], a_x[S::A_PASSES], a_base[S::A_PASSES];      // image position of tap (0,0) and its byte offset
#pragma unroll
    for (int p = 0; p < S::A_PASSES; ++p) {
        int m = bm0 + r0 + p * S::ROWS_PER_PASS;
        if (m >= M) m = M - 1;                                       // rows past the end are computed and never stored
        a_y[p] = m / img.Wout - img.oy;
        a_x[p] = m % img.Wout - img.ox;
        a_base[p] = 4 * (a_y[p] * img.row_stride_w + a_x[p] * img.dpitch_w);
    }
    int b_base[S::B_PASSES];
#pragma unroll
    for (int p = 0; p < S::B_PASSES; ++p) {
        int n = bn0 + r0 + p * S::ROWS_PER_PASS;
        if (n >= N) n = N - 1;
        b_base[p] = 4 * n * fb.filt_stride_w;
    }
    TapWalk wa, wb;                                                   // position of this thread's unit: in the image, in a filter
    wa.init(4 * q, img.dpitch_w, img.kw, img.row_stride_w);
    wb.init(4 * q, fb.dpitch_w, fb.kw, fb.row_stride_w);
    const TapStep sa = TapStep::make(S::BK / 2, img.dpitch_w, img.kw, img.row_stride_w);
    const TapStep sb = TapStep::make(S::BK / 2, fb.dpitch_w, fb.kw, fb.row_stride_w);

    u32x4 a_stage[S::A_PASSES], b_stage[S::B_PASSES];
    auto load_stage = [&]() {
        const bool k_ok = wa.k < Kw;                                  // a unit never straddles the end of K (K % 8 == 0 halves)
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) {
            const bool inside = k_ok && (unsigned)(a_y[p] + wa.ki) < (unsigned)img.H && (unsigned)(a_x[p] + wa.kj) < (unsigned)img.W;
            const f32x4 v = buffer_load_quad(make_rsrc(img.src, img.bytes), inside ? (unsigned)(a_base[p] + wa.off) : kOutOfRange);
            a_stage[p] = __builtin_bit_cast(u32x4, v);
        }
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) {
            const f32x4 v = buffer_load_quad(make_rsrc(fb.filt, fb.bytes), k_ok ? (unsigned)(b_base[p] + wb.off) : kOutOfRange);
            b_stage[p] = __builtin_bit_cast(u32x4, v);
        }
        wa.advance(sa, img.dpitch_w, img.kw);
        wb.advance(sb, fb.dpitch_w, fb.kw);
    };
    auto store_stage = [&](int buf) {
        u32x4* Ab = As + buf * S::A_UNITS;
        u32x4* Bb = Bs + buf * S::B_UNITS;
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) Ab[a_unit_slot(r0 + p * S::ROWS_PER_PASS, q, U)] = a_stage[p];
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) Bb[a_unit_slot(r0 + p * S::ROWS_PER_PASS, q, U)] = b_stage[p];
    };

    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    const int steps = (Kw + S::BK / 2 - 1) / (S::BK / 2);
    load_stage();
    store_stage(0);
    __syncthreads();
    for (int t = 0; t < steps; ++t) {
        const int buf = t & 1;
        if (t + 1 < steps) load_stage();
        const u32x4* Ab = As + buf * S::A_UNITS;
        const u32x4* Bb = Bs + buf * S::B_UNITS;
#pragma unroll
        for (int ks = 0; ks < S::BK / 16; ++ks) {
            f16x8 af[MI], bf[NI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) af[mi] = __builtin_bit_cast(f16x8, Ab[a_unit_slot(wm0 + mi * 32 + li, 2 * ks + lh, U)]);
#pragma unroll
            for (int ni = 0; ni < NI; ++ni) bf[ni] = __builtin_bit_cast(f16x8, Bb[a_unit_slot(wn0 + ni * 32 + li, 2 * ks + lh, U)]);
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

    float bias_v[NI];
#pragma unroll
    for (int ni = 0; ni < NI; ++ni) {
        const int n = bn0 + wn0 + ni * 32 + li;
        bias_v[ni] = (out.bias != nullptr && n < N) ? (float)out.bias[n] : 0.f;
    }
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
            if (m < M) {
                _Float16* pix = out.dst + (size_t)(m / out.Wout) * out.row_stride + (size_t)(m % out.Wout) * out.dpitch;
#pragma unroll
                for (int ni = 0; ni < NI; ++ni) {
                    const int n = bn0 + wn0 + ni * 32 + li;
                    float v = acc[mi][ni][r];
                    if (out.bias != nullptr) v += bias_v[ni];
                    if (out.relu) v = relu_by_sign(v);
                    if (n < N) pix[n] = (_Float16)v;
                }
            }
        }
}

}  // namespace decx_hip
