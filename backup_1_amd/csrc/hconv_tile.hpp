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
// K steps are short (16 MFMAs per wave), so the loads run DEPTH steps ahead through DEPTH register sets.  The filters
// are the MFMA's row operand and the pixels its column operand: a lane then holds, for ONE pixel, runs of four
// consecutive filters, which is how dst is laid out -- bias, ReLU and the rounding happen on those runs in registers,
// they go to LDS as 8-byte pieces and leave it as 16-byte ones.  Everything else is kept off the VALU (which shares
// its issue slots with the matrix pipe): LDS addresses are per-lane constants plus immediates, divisions by the image
// width use a float reciprocal while the pixel count allows it.
//
// Products are accumulated in fp32 in the MFMA's own order (not the scalar chain of the fp32 path: there is no binary16
// reference result to be bit-identical to) and rounded to binary16, nearest even, once, after the optional bias and ReLU.
#pragma once
#include "hgemm_tile.hpp"
#include "sgemm_tile.hpp"

namespace decx_hip {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int DEPTH_>
struct HconvShape {
    static constexpr int BM = BM_, BN = BN_, BK = 64, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int DEPTH = DEPTH_;                      // register sets: K steps in flight from global memory
    static constexpr int NT = WAVES_M * WAVES_N * kWave;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int U = BK / 8;                          // 16-byte units per row and K step
    static constexpr int A_UNITS = BM * U, B_UNITS = BN * U;
    static constexpr int A_PASSES = A_UNITS / NT, B_PASSES = B_UNITS / NT, ROWS_PER_PASS = NT / U;
    static constexpr int OUT_ROW = BN + 4;                    // halves per pixel of the result tile in LDS: rows 66 words apart,
                                                              // so the 8-byte writes of 16 lanes (16 pixels) cover all banks
    static constexpr size_t STAGE_BYTES = 2 * (size_t)(A_UNITS + B_UNITS) * 16;
    static constexpr size_t OUT_BYTES = (size_t)BM * OUT_ROW * 2 + (size_t)BN * 4;      // result tile + bias as floats
    static constexpr size_t LDS_BYTES = STAGE_BYTES > OUT_BYTES ? STAGE_BYTES : OUT_BYTES;
    static_assert(DEPTH_ % 2 == 0, "the LDS buffer of a step is a compile-time index of the unrolled loop");
    static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(A_UNITS % NT == 0 && B_UNITS % NT == 0 && NT % U == 0, "staging must divide evenly");
    static_assert(BN % 8 == 0 && (BM * (BN / 8)) % NT == 0, "the result tile leaves in whole 16-byte units");
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

// Epilogue of the fp16 convolution kernels.  Lane (li, lh) holds for pixel wm0 + 32 mi + li the filters
// wn0 + 32 ni + 8 j + 4 lh + e (e = 0..3) in acc[mi][ni][4 j + e]: bias, ReLU and one rounding to binary16 per run of
// four, then through LDS (which must be free: no reader of the operand buffers left, no load into them in flight) so
// that the tile leaves in 16-byte pieces.
template <class S, class PixelOf>
__device__ __forceinline__ void hconv_store_tile(const f32x16 (&acc)[S::MI][S::NI], unsigned char* lds_raw, const HalfTensorOut& out,
                                                 int M, int N, int bm0, int bn0, int wm0, int wn0, int tid, const PixelOf& pixel_of) {
    constexpr int BM = S::BM, BN = S::BN, NT = S::NT, MI = S::MI, NI = S::NI;
    const int lane = tid % kWave, li = lane & 31, lh = lane >> 5;
    typedef _Float16 f16x4v __attribute__((ext_vector_type(4)));
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    _Float16* tile = reinterpret_cast<_Float16*>(lds_raw);                                   // [BM][OUT_ROW]
    float* bias_lds = reinterpret_cast<float*>(lds_raw + (size_t)BM * S::OUT_ROW * 2);         // [BN]
    if (out.bias != nullptr) {
        for (int i = tid; i < BN; i += NT) bias_lds[i] = bn0 + i < N ? (float)out.bias[bn0 + i] : 0.f;
        __syncthreads();
    }
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n_local = wn0 + ni * 32 + 8 * j + 4 * lh;
                f32x4 v = {acc[mi][ni][4 * j], acc[mi][ni][4 * j + 1], acc[mi][ni][4 * j + 2], acc[mi][ni][4 * j + 3]};
                if (out.bias != nullptr) v += *reinterpret_cast<const f32x4*>(bias_lds + n_local);
                if (out.relu) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = relu_by_sign(v[e]);
                }
                const f16x4v h = __builtin_convertvector(v, f16x4v);
                *reinterpret_cast<u32x2*>(tile + (wm0 + mi * 32 + li) * S::OUT_ROW + n_local) = __builtin_bit_cast(u32x2, h);
            }
    __syncthreads();
    constexpr int UNITS_PER_ROW = BN / 8, OUT_PASSES = BM * UNITS_PER_ROW / NT;
    // whole 16-byte units when dst allows it (pixel pitch a multiple of 8 halves, 16-byte aligned base), else half by half
    const bool vec = out.dpitch % 8 == 0 && out.row_stride % 8 == 0 && (reinterpret_cast<size_t>(out.dst) & 15) == 0;
    // a whole tile of a tensor whose pixels lie back to back: pixel m starts at m * dpitch -- no bounds branches, no
    // division per piece (one scalar test per workgroup)
    if (vec && out.row_stride == (size_t)out.Wout * out.dpitch && bm0 + BM <= M && bn0 + BN <= N) {
#pragma unroll
        for (int p = 0; p < OUT_PASSES; ++p) {
            const int id = tid + p * NT, row = id / UNITS_PER_ROW, u = id % UNITS_PER_ROW;
            const _Float16* t8 = tile + row * S::OUT_ROW + 8 * u;
            const u32x2 lo = *reinterpret_cast<const u32x2*>(t8), hi = *reinterpret_cast<const u32x2*>(t8 + 4);
            *reinterpret_cast<u32x4*>(out.dst + (size_t)(bm0 + row) * out.dpitch + bn0 + 8 * u) = u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
        return;
    }
#pragma unroll
    for (int p = 0; p < OUT_PASSES; ++p) {
        const int id = tid + p * NT, row = id / UNITS_PER_ROW, u = id % UNITS_PER_ROW;
        const int m = bm0 + row, n = bn0 + 8 * u;
        if (m < M && n < N) {
            int y, x;
            pixel_of(m, y, x);
            _Float16* pix = out.dst + (size_t)y * out.row_stride + (size_t)x * out.dpitch + n;
            const _Float16* t8 = tile + row * S::OUT_ROW + 8 * u;          // 8-byte aligned
            if (vec && n + 8 <= N) {
                const u32x2 lo = *reinterpret_cast<const u32x2*>(t8), hi = *reinterpret_cast<const u32x2*>(t8 + 4);
                *reinterpret_cast<u32x4*>(pix) = u32x4{lo[0], lo[1], hi[0], hi[1]};
            } else {
                for (int e = 0; e < 8 && n + e < N; ++e) pix[e] = t8[e];
            }
        }
    }
}

// TAP_UNIFORM (channel pitch a multiple of 64 halves, i.e. of a K step): a K step lies inside one tap, so the walk over
// (tap row, tap column, channel) is the same for every lane up to a constant and runs on the scalar unit; a load then
// costs the vector unit one add (plus the column check of an image load), and a filter load nothing at all.
// SPLIT_K (small images: few tiles, many K steps): blockIdx.y selects a range of steps_per_split K steps; the tile's fp32
// partial sums go to a workspace of dense M x N fp32 planes: range y stores into plane y (partial_plane floats apart;
// nothing to zero), or, with partial_plane == 0, all ranges add into one zeroed plane with atomics.
// hconv_split_finish_kernel adds the planes in range order, applies bias and ReLU and writes the binary16 tensor.
template <class S, bool TAP_UNIFORM, bool SPLIT_K = false>
__global__ __launch_bounds__(S::NT, 2) void hconv_tile_kernel(HalfImage img, HalfFilters fb, HalfTensorOut out, int M, int N,
                                                           int Kw /* K in words */, int tiles_n, float* partial,
                                                           int steps_per_split, size_t partial_plane) {
    constexpr int BM = S::BM, BN = S::BN, NT = S::NT, U = S::U, MI = S::MI, NI = S::NI;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    constexpr int A_BYTES = S::A_UNITS * 16, B_BYTES = S::B_UNITS * 16;     // one buffer of either operand
    unsigned char* As = lds_raw;                              // [2][A_UNITS] units of 16 bytes
    unsigned char* Bs = lds_raw + 2 * A_BYTES;                // [2][B_UNITS]

    // each XCD gets one contiguous run of tiles: neighbouring tiles share their halo rows in that XCD's L2
    const TileCoord tc = xcd_grouped_tile((int)blockIdx.x, (int)gridDim.x / tiles_n, tiles_n, 8);
    const int all_steps = (Kw + S::BK / 2 - 1) / (S::BK / 2);
    const int first_step = SPLIT_K ? (int)blockIdx.y * steps_per_split : 0;
    const int steps = SPLIT_K ? (all_steps - first_step < steps_per_split ? all_steps - first_step : steps_per_split) : all_steps;
    const int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;
    const bool small_m = M < (1 << 22);
    const float rcp_wout = 1.0f / (float)img.Wout;
    auto pixel_of = [&](int m, int& y, int& x) {
        if (small_m) small_divmod(m, img.Wout, rcp_wout, y, x);
        else { y = m / img.Wout; x = m - y * img.Wout; }
    };

    // staging: this thread moves unit q of rows r0, r0 + ROWS_PER_PASS, ... of either operand
    const int q = tid % U, r0 = tid / U;
    int a_y[S::A_PASSES], a_x[S::A_PASSES], a_base[S::A_PASSES];      // image position of tap (0,0) and its byte offset
#pragma unroll
    for (int p = 0; p < S::A_PASSES; ++p) {
        int m = bm0 + r0 + p * S::ROWS_PER_PASS;
        if (m >= M) m = M - 1;                                       // rows past the end are computed and never stored
        int y, x;
        pixel_of(m, y, x);
        a_y[p] = y - img.oy;
        a_x[p] = x - img.ox;
        a_base[p] = 4 * (a_y[p] * img.row_stride_w + a_x[p] * img.dpitch_w);
    }
    int b_base[S::B_PASSES];
#pragma unroll
    for (int p = 0; p < S::B_PASSES; ++p) {
        int n = bn0 + r0 + p * S::ROWS_PER_PASS;
        if (n >= N) n = N - 1;
        b_base[p] = 4 * n * fb.filt_stride_w;
    }
    // position of this thread's unit in the image and in a filter; with TAP_UNIFORM the walk starts at unit 0 for all
    // lanes (scalar registers) and the lane's own 16 q bytes are part of its base offsets
    TapWalk wa, wb;
    wa.init(first_step * (S::BK / 2) + (TAP_UNIFORM ? 0 : 4 * q), img.dpitch_w, img.kw, img.row_stride_w);
    wb.init(first_step * (S::BK / 2) + (TAP_UNIFORM ? 0 : 4 * q), fb.dpitch_w, fb.kw, fb.row_stride_w);
    const TapStep sa = TapStep::make(S::BK / 2, img.dpitch_w, img.kw, img.row_stride_w);
    const TapStep sb = TapStep::make(S::BK / 2, fb.dpitch_w, fb.kw, fb.row_stride_w);
    if (TAP_UNIFORM) {
#pragma unroll
        for (int p = 0; p < S::A_PASSES; ++p) a_base[p] += 16 * q;
#pragma unroll
        for (int p = 0; p < S::B_PASSES; ++p) b_base[p] += 16 * q;
    }

    // LDS addresses.  Unit (row, u) of a buffer lies at row*U + (u ^ ((row / 2) % U)) (a_unit_slot); rows that are a
    // multiple of 16 apart share the swizzle term, so per lane it is one value for all staging passes and one for all
    // fragment reads, and everything else is an immediate.
    static_assert(U == 8 && S::ROWS_PER_PASS % 16 == 0, "swizzle terms are shared between passes and blocks");
    const int stage_off = (r0 * U + (q ^ ((r0 / 2) % U))) * 16;      // + p * ROWS_PER_PASS * 128
    int frag_x[S::BK / 16];                                           // ((2 ks + lh) ^ swizzle) * 16
#pragma unroll
    for (int ks = 0; ks < S::BK / 16; ++ks) frag_x[ks] = ((2 * ks + lh) ^ ((li / 2) % U)) * 16;
    const int a_frag_row = (wm0 + li) * U * 16, b_frag_row = (wn0 + li) * U * 16;

    // DEPTH register sets: the loads of K step t travel through set t % DEPTH and are issued DEPTH steps before they are
    // needed -- one step is only 16 MFMAs per wave, a load takes several times that.  Loads past the end of K ask for an
    // out-of-range offset: zeros, no memory traffic, never used.
    constexpr int DEPTH = S::DEPTH;
    u32x4 a_stage[DEPTH][S::A_PASSES], b_stage[DEPTH][S::B_PASSES];
    auto load_stage = [&](auto set_tag) {
        constexpr int SET = decltype(set_tag)::value;
        if constexpr (TAP_UNIFORM) {
            // Rows above and below the image need no test: their offsets are negative or past the end of the tensor.  K
            // is a whole number of steps here; the loads that run past it fetch something that is never used.
#pragma unroll
            for (int p = 0; p < S::A_PASSES; ++p) {
                const bool inside = (unsigned)(a_x[p] + wa.kj) < (unsigned)img.W;
                const unsigned off = inside ? (unsigned)(a_base[p] + wa.off) : kOutOfRange;
                a_stage[SET][p] = __builtin_bit_cast(u32x4, buffer_load_quad(make_rsrc(img.src, img.bytes), off));
            }
#pragma unroll
            for (int p = 0; p < S::B_PASSES; ++p)
                b_stage[SET][p] = __builtin_bit_cast(
                    u32x4, __builtin_amdgcn_raw_buffer_load_b128(make_rsrc(fb.filt, fb.bytes), b_base[p], wb.off, 0));
        } else {
            const bool k_ok = wa.k < Kw;                              // a unit never straddles the end of K (K % 8 == 0 halves)
#pragma unroll
            for (int p = 0; p < S::A_PASSES; ++p) {
                const bool inside = k_ok && (unsigned)(a_y[p] + wa.ki) < (unsigned)img.H && (unsigned)(a_x[p] + wa.kj) < (unsigned)img.W;
                const f32x4 v = buffer_load_quad(make_rsrc(img.src, img.bytes), inside ? (unsigned)(a_base[p] + wa.off) : kOutOfRange);
                a_stage[SET][p] = __builtin_bit_cast(u32x4, v);
            }
#pragma unroll
            for (int p = 0; p < S::B_PASSES; ++p) {
                const f32x4 v = buffer_load_quad(make_rsrc(fb.filt, fb.bytes), k_ok ? (unsigned)(b_base[p] + wb.off) : kOutOfRange);
                b_stage[SET][p] = __builtin_bit_cast(u32x4, v);
            }
        }
        wa.advance(sa, img.dpitch_w, img.kw);
        wb.advance(sb, fb.dpitch_w, fb.kw);
    };
    // staging pass P (0 .. A_PASSES-1: image, then the filters) of a register set into LDS buffer BUF
    constexpr int PASSES = S::A_PASSES + S::B_PASSES;
    auto store_pass = [&](auto set_tag, auto buf_tag, auto pass_tag) {
        constexpr int SET = decltype(set_tag)::value, BUF = decltype(buf_tag)::value, P = decltype(pass_tag)::value;
        if constexpr (P < S::A_PASSES)
            *reinterpret_cast<u32x4*>(As + BUF * A_BYTES + P * S::ROWS_PER_PASS * U * 16 + stage_off) = a_stage[SET][P];
        else
            *reinterpret_cast<u32x4*>(Bs + BUF * B_BYTES + (P - S::A_PASSES) * S::ROWS_PER_PASS * U * 16 + stage_off) = b_stage[SET][P - S::A_PASSES];
    };

    // acc[mi][ni]: rows of the MFMA result are filters, columns are pixels
    f32x16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    typedef std::integral_constant<int, 0> I0;
    static_for<0, DEPTH>([&](auto d) { load_stage(d); });
    static_for<0, PASSES>([&](auto p) { store_pass(I0{}, I0{}, p); });
    __syncthreads();
    load_stage(I0{});                                          // step DEPTH
    // Step t: MFMAs from LDS buffer t % 2; between them the loads of step t+1 (set (t+1) % DEPTH, issued DEPTH-1 steps
    // ago) go to the other buffer, which everybody finished reading before the last barrier -- LDS stores are slow (a
    // 16-byte store of a wave takes 13 cycles) and must not form a phase of their own; then the barrier, and the set is
    // refilled with step t+1+DEPTH.  Past the end of K all of this moves zeros that nobody reads.
    constexpr int KS = S::BK / 16;
    auto k_step = [&](auto d) {
        constexpr int DD = decltype(d)::value, BUF = DD & 1;
        typedef std::integral_constant<int, (DD + 1) % DEPTH> NextSet;
        typedef std::integral_constant<int, BUF ^ 1> NextBuf;
        static_for<0, KS>([&](auto ks_tag) {
            constexpr int ks = decltype(ks_tag)::value;
            f16x8 pf[MI], ff[NI];
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
                pf[mi] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(As + BUF * A_BYTES + mi * 32 * U * 16 + a_frag_row + frag_x[ks]));
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
                ff[ni] = __builtin_bit_cast(f16x8, *reinterpret_cast<const u32x4*>(Bs + BUF * B_BYTES + ni * 32 * U * 16 + b_frag_row + frag_x[ks]));
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int ni = 0; ni < NI; ++ni)
                    // split-K keeps the GEMM orientation (pixels as rows): a lane's atomic adds then run along the filters,
                    // i.e. along consecutive addresses of the workspace
                    acc[mi][ni] = SPLIT_K ? __builtin_amdgcn_mfma_f32_32x32x16_f16(pf[mi], ff[ni], acc[mi][ni], 0, 0, 0)
                                          : __builtin_amdgcn_mfma_f32_32x32x16_f16(ff[ni], pf[mi], acc[mi][ni], 0, 0, 0);
            static_for<ks * PASSES / KS, (ks + 1) * PASSES / KS>([&](auto p) { store_pass(NextSet{}, NextBuf{}, p); });
        });
        __syncthreads();
        load_stage(NextSet{});
    };
    for (int t0 = 0; t0 < steps; t0 += DEPTH)
        static_for<0, DEPTH>([&](auto d) {
            if (t0 + decltype(d)::value < steps) k_step(d);
        });

    if (SPLIT_K) {
        const bool ordered = partial_plane != 0;                 // uniform over the launch
        float* plane = partial + (size_t)blockIdx.y * partial_plane;
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
    __syncthreads();                                           // everybody is done reading the last operand buffer
    hconv_store_tile<S>(acc, lds_raw, out, M, N, bm0, bn0, wm0, wn0, tid, pixel_of);
}

// dst(pixel m, filter n) = half(relu(plane 0 + plane 1 + ... + bias[n])), added in that order: the end of a split-K
// convolution.  partial holds `planes` dense M x N fp32 planes, `plane` floats apart.
static __global__ __launch_bounds__(256) void hconv_split_finish_kernel(const float* __restrict__ partial, int planes, size_t plane,
                                                                 HalfTensorOut out, int M, int N) {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int m = (int)(i / N), n = (int)(i - (size_t)m * N);
        float v = ordered_plane_sum(partial, planes, plane, i);
        if (out.bias != nullptr) v += (float)out.bias[n];
        if (out.relu) v = relu_by_sign(v);
        out.dst[(size_t)(m / out.Wout) * out.row_stride + (size_t)(m % out.Wout) * out.dpitch + n] = (_Float16)v;
    }
}

}  // namespace decx_hip
