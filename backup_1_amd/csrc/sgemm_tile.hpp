// fp32 MFMA contraction tile for gfx950, shared by the dense GEMM and the fused im2col convolution.
//
// One workgroup owns a BM x BN tile of the result and walks K in steps of BK.  Its waves are laid out WAVES_M x
// WAVES_N, each owning a (BM/WAVES_M) x (BN/WAVES_N) sub-tile as a grid of 32x32 v_mfma_f32_32x32x2_f32 blocks
// whose accumulators stay in registers for the whole K walk.
//
// Staging: global -> registers -> LDS, two LDS buffers, one barrier per K step; the loads run one or two K steps ahead
// of the MFMAs.  A is kept in LDS as float4 "k-quads":
//   A quad (p, m) = A[m][8s+par+{0,2,4,6}], p = 2s+par,  at  As[p][m]
// so that one ds_read_b128 per 32-row block feeds four MFMAs.
// Summation order.  v_mfma_f32_32x32x2_f32 computes, per output element, fma(a1, b1, fma(a0, b0, c)) with operand 0 from
// lanes 0-31 and operand 1 from lanes 32-63 (checked bit for bit on the hardware), i.e. it IS two steps of the
// reference's single-accumulator fused chain.  The k indices are therefore laid out so that every output sees them in
// ascending order: of each group of 8 consecutive k (8s .. 8s+7) the even ones go to plane 2s, the odd ones to plane
// 2s+1 (de-interleaved while staging), lanes 0-31 read plane 2s and lanes 32-63 plane 2s+1, and MFMA e of the group
// multiplies k = 8s+2e and 8s+2e+1.  The result equals fmaf over k = 0 .. K-1 from a single accumulator -- the
// arithmetic of every fp32 path of the reference -- bit for bit, whatever the tile shape.
// B has two LDS layouts, chosen by its source:
//   * a row-major K x N matrix (DenseB) stays row-major, Bs[k][n], exactly as loaded -- no transpose, no VALU work.
//     The wave's 32x32 blocks then take INTERLEAVED columns: lane li of block ni owns column NI*li + ni of the wave's
//     strip, so the NI operands a lane needs at one k are NI consecutive floats of one row (one ds_read_b128 for
//     NI = 4) and the NI results it holds per row are consecutive too (one 16-byte store).
//   * a filter bank (FilterB), whose k runs contiguously per column, is kept as k-quads like A:
//       B quad (p, n) = B[8s+par+{0,2,4,6}][n] at  Bs[p][b_slot(n)];  block ni takes columns 32*ni + li.
// Every instruction that is not an MFMA costs the matrix pipe cycles (measured: 3-8 per VALU instruction; a wave's VALU
// and MFMA work do not overlap), so the K loop is kept as free of address arithmetic and data shuffling as the layouts
// allow, and two waves share a SIMD where the registers permit (a lone wave leaves ~3.5 idle cycles between MFMAs).
//
// Ragged edges: rows >= M and columns >= N are read from clamped (valid) addresses and never stored; only the last,
// partial K step zero-fills (both operands, so that 0 * Inf cannot appear).  No padded copies exist anywhere.
#pragma once
#include <type_traits>
#include "tile_common.hpp"

namespace decx_hip {

// ---------------------------------------------------------------------------------------------------------------
// A-operand sources.  Interface:
//   RowState row_state(int m)                       per-row values that do not change along K
//   KState k_state(k) / KStep k_step(dk) / advance(ks, step)
//                                                   position of the first quad of a k-group (8 consecutive k), moved on
//                                                   by whole K steps
//   template<bool TAIL> load_pair(rs, ks, step, lo, hi)
//                                                   A[m][k..k+3] and A[m][k+4..k+7], branch-free; what lies outside the
//                                                   operand (image border, K tail when TAIL) comes back as zeros
// ---------------------------------------------------------------------------------------------------------------
// Slot of column n inside a B plane: bits 3-4 of n are folded onto bits 0-1.
// Measured on gfx950 (two active lanes hitting the same banks, SQ_LDS_BANK_CONFLICT): ds_read_b128 services a wave in
// four phases -- lanes {0-3, 12-15, 20-23, 24-27} and {4-11, 16-19, 28-31} of each half-wave -- and a phase is
// conflict-free when its 16-byte accesses fall into distinct slots mod 16; ds_write_b128 goes in eight phases of 8
// consecutive lanes, conflict-free when the slots are distinct mod 8.  With this fold the fragment reads (32
// consecutive columns per half-wave) qualify.  Rows of A need no fold: consecutive slots are read.
__device__ __forceinline__ int b_slot(int n) { return n ^ ((n >> 3) & 3); }

// 16 bytes through a buffer resource: offsets at or beyond the resource's size read as zeros, which is how taps
// outside the image, rows of a ragged last tile and the K tail are zero-filled without a select per element.
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
constexpr unsigned kOutOfRange = 0x80000000u;      // resources are kept below 2 GiB
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ f32x4 buffer_load_quad(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_offset) {
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 0));
}

// Two floats from any two registers to two consecutive-pair LDS dwords: halves 0 and 1 fill dwords (0,1) and (2,3) of a
// 16-byte quad.  This is how 8 consecutive k are de-interleaved into an even-k and an odd-k quad without first gathering
// the values into consecutive registers (which costs a register move per float, and every VALU instruction takes cycles
// from the matrix pipe).  Issued from inline asm: the compiler does not count these stores in its LDS wait counts, which
// is safe (a wait computed without them only ever waits for more), and the barrier code waits for lgkmcnt(0) itself.
template <int HALF>
__device__ __forceinline__ void lds_write_pair(unsigned byte_addr, float x, float y) {
    if (HALF == 0) asm volatile("ds_write2_b32 %0, %1, %2 offset0:0 offset1:1" : : "v"(byte_addr), "v"(x), "v"(y) : "memory");
    else asm volatile("ds_write2_b32 %0, %1, %2 offset0:2 offset1:3" : : "v"(byte_addr), "v"(x), "v"(y) : "memory");
}
// 8 consecutive k held as two quads (lo = k0..k3, hi = k4..k7); part 0, 1: even k to the quad at even_addr; 2, 3: odd k
template <int PART>
__device__ __forceinline__ void lds_write_deinterleaved(unsigned even_addr, unsigned odd_addr, const f32x4& lo, const f32x4& hi) {
    if (PART == 0) lds_write_pair<0>(even_addr, lo[0], lo[2]);
    if (PART == 1) lds_write_pair<1>(even_addr, hi[0], hi[2]);
    if (PART == 2) lds_write_pair<0>(odd_addr, lo[1], lo[3]);
    if (PART == 3) lds_write_pair<1>(odd_addr, hi[1], hi[3]);
}
__device__ __forceinline__ unsigned lds_byte_address(const void* p) {
    return (unsigned)(size_t)(__attribute__((address_space(3))) const char*)p;
}
// Workgroup barrier that first waits for this wave's own LDS traffic, stated explicitly because the compiler's wait
// counting does not see the inline-asm stores above.
__device__ __forceinline__ void lds_sync() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// A K step of dk as an increment of the im2col position (c, kj, ki): dk = (dki*kw + dkj)*dpitch + dc, and of the byte
// offset of that position inside a tensor whose rows are row_stride floats apart.  Worked out once per kernel so that
// advancing is a handful of adds and selects.
struct TapStep {
    int dk, dc, dkj, dki;
    int step_bytes;      // offset change of the raw increments
    int wrap_bytes;      // extra change when kj wraps into the next tensor row (a c -> kj carry changes nothing: the
                         // channels of consecutive taps of one row are contiguous)
    __device__ __forceinline__ static TapStep make(int dk, int dpitch, int kw, int row_stride) {
        const int taps = dk / dpitch, rows = taps / kw;
        const int dc = dk - taps * dpitch, dkj = taps - rows * kw;
        return TapStep{dk, dc, dkj, rows, 4 * (rows * row_stride + dkj * dpitch + dc), 4 * (row_stride - kw * dpitch)};
    }
};

// Position of one k index inside the im2col ordering k = (ki*kw + kj)*dpitch + c, with its byte offset
// 4*(ki*row_stride + kj*dpitch + c).  Decoded once (two integer divisions), then advanced by whole K steps without
// divisions, loops or branches (control flow inside the K loop would split its body into basic blocks and undo the
// instruction schedule).
struct TapWalk {
    int k, c, ki, kj, off;
    __device__ __forceinline__ void init(int k_, int dpitch, int kw, int row_stride) {
        k = k_;
        const int tap = k_ / dpitch;
        c = k_ - tap * dpitch;
        ki = tap / kw;
        kj = tap - ki * kw;
        off = 4 * (ki * row_stride + kj * dpitch + c);
    }
    __device__ __forceinline__ void advance(const TapStep& st, int dpitch, int kw) {
        k += st.dk;
        c += st.dc;
        const bool carry_c = c >= dpitch;                 // c < 2*dpitch: one carry at most
        c -= carry_c ? dpitch : 0;
        kj += st.dkj + (carry_c ? 1 : 0);
        const bool carry_kj = kj >= kw;                   // kj <= 2*kw - 1: one carry at most
        kj -= carry_kj ? kw : 0;
        ki += st.dki + (carry_kj ? 1 : 0);
        off += st.step_bytes + (carry_kj ? st.wrap_bytes : 0);
    }
    // the position 4 further on (c and dpitch are multiples of 4, so c + 4 never exceeds dpitch)
    __device__ __forceinline__ TapWalk next_quad(const TapStep& st, int dpitch, int kw) const {
        TapWalk w;
        w.k = k + 4;
        const bool carry_c = c + 4 >= dpitch;
        w.c = carry_c ? 0 : c + 4;
        const bool carry_kj = carry_c && kj + 1 >= kw;
        w.kj = carry_c ? (carry_kj ? 0 : kj + 1) : kj;
        w.ki = ki + (carry_kj ? 1 : 0);
        w.off = off + 16 + (carry_kj ? st.wrap_bytes : 0);
        return w;
    }
};

template <bool VEC>
struct DenseA {
    const float* A;
    int lda, M, K;
    size_t batch_stride;      // elements between consecutive matrices of a batch (blockIdx.y walks the batch)
    __device__ __forceinline__ void select_batch(int b) { A += (size_t)b * batch_stride; }
    __device__ __forceinline__ void set_k_end(int k_end) { K = k_end; }      // split-K: this workgroup's K range ends here
    struct RowState {
        const float* row;
    };
    struct KState {
        int k;
    };
    struct KStep {
        int dk;
    };
    __device__ __forceinline__ KState k_state(int k) const { return KState{k}; }
    __device__ __forceinline__ KStep k_step(int dk) const { return KStep{dk}; }
    __device__ __forceinline__ void advance(KState& ks, const KStep& st) const { ks.k += st.dk; }
    // the 8 consecutive k of one staging task: two quads
    template <bool TAIL>
    __device__ __forceinline__ void load_pair(const RowState& rs, const KState& ks, const KStep&, f32x4& lo, f32x4& hi) const {
        lo = load<TAIL>(rs, ks);
        hi = load<TAIL>(rs, KState{ks.k + 4});
    }
    __device__ __forceinline__ RowState row_state(int m) const {
        RowState rs;
        rs.row = A + (size_t)(m < M ? m : M - 1) * lda;
        return rs;
    }
    template <bool TAIL>
    __device__ __forceinline__ f32x4 load(const RowState& rs, const KState& ks) const {
        const int k = ks.k;
        f32x4 v = {0.f, 0.f, 0.f, 0.f};
        if (VEC) {
            if (!TAIL) {
                v = *reinterpret_cast<const f32x4*>(rs.row + k);
            } else if (k < K) {
                v = *reinterpret_cast<const f32x4*>(rs.row + k);   // lda % 4 == 0 keeps the quad inside the pitch
                if (k + 1 >= K) v[1] = 0.f;
                if (k + 2 >= K) v[2] = 0.f;
                if (k + 3 >= K) v[3] = 0.f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (k + e < K) v[e] = rs.row[k + e];
        }
        return v;
    }
};

// The im2col view of a channel-innermost tensor: row m = (y, x) of the output, column k = (ki*kw + kj)*dpitch + c.
// Everything is 32-bit byte-offset arithmetic against one buffer resource (tensors stay below 2 GiB): per row the offset
// of its top-left tap is kept, per K step the tap's offset is added, and a tap outside the image gets an out-of-range
// offset instead, which the hardware answers with zeros.
// PAIRED (dpitch % 8 == 0): the two quads of a staging task (8 consecutive k) always lie in the same tap, so one bounds
// check and one offset serve both; otherwise the second quad's position is derived from the first.
template <bool PAIRED>
struct Im2colA {
    const float* src;
    int H, W, dpitch, kh, kw, oy, ox, Wout, Mtot, K;
    int row_stride;            // floats between image rows
    unsigned bytes;            // extent of the tensor
    __device__ __forceinline__ void select_batch(int) {}
    __device__ __forceinline__ void set_k_end(int k_end) { K = k_end; }
    struct RowState {
        int y, x;          // output pixel shifted by (-oy, -ox): the image position of tap (0, 0)
        int base;          // 4*(y*row_stride + x*dpitch); may be negative, only used together with an in-image tap
    };
    __device__ __forceinline__ RowState row_state(int m) const {
        if (m >= Mtot) m = Mtot - 1;
        RowState rs;
        rs.y = m / Wout - oy;
        rs.x = m % Wout - ox;
        rs.base = 4 * (rs.y * row_stride + rs.x * dpitch);
        return rs;
    }
    typedef TapWalk KState;
    typedef TapStep KStep;
    __device__ __forceinline__ KState k_state(int k) const {
        KState ks;
        ks.init(k, dpitch, kw, row_stride);
        return ks;
    }
    __device__ __forceinline__ KStep k_step(int dk) const { return TapStep::make(dk, dpitch, kw, row_stride); }
    __device__ __forceinline__ void advance(KState& ks, const KStep& st) const { ks.advance(st, dpitch, kw); }
    template <bool TAIL>
    __device__ __forceinline__ unsigned quad_offset(const RowState& rs, const KState& ks) const {
        // K = kh*kw*dpitch is a multiple of 4 (of 8 when PAIRED): quads (pairs) never straddle it
        const bool inside = (unsigned)(rs.y + ks.ki) < (unsigned)H && (unsigned)(rs.x + ks.kj) < (unsigned)W && (!TAIL || ks.k < K);
        return inside ? (unsigned)(rs.base + ks.off) : kOutOfRange;
    }
    template <bool TAIL>
    __device__ __forceinline__ void load_pair(const RowState& rs, const KState& ks, const KStep& st, f32x4& lo, f32x4& hi) const {
        const unsigned o = quad_offset<TAIL>(rs, ks);
        lo = buffer_load_quad(make_rsrc(src, bytes), o);
        if (PAIRED) hi = buffer_load_quad(make_rsrc(src, bytes), o + 16u);      // out of range stays out of range
        else hi = buffer_load_quad(make_rsrc(src, bytes), quad_offset<TAIL>(rs, ks.next_quad(st, dpitch, kw)));
    }
};

// Im2colA for a channel pitch that is a multiple of the K step (16 floats): a K step then lies inside one tap, so the
// walk over (tap row, tap column, channel) is the same for every lane up to the lane's own 0 or 8 floats and runs on
// the scalar unit.  Rows above and below the image need no test -- their offsets are negative or past the end of the
// tensor, and the buffer answers those with zeros -- which leaves one column test per task on the vector unit.
struct Im2colAUniform : Im2colA<true> {
    struct KState {
        TapWalk walk;          // of the K step's first float; held in scalar registers
        int lane_bytes;        // this lane's offset inside the step
    };
    __device__ __forceinline__ KState k_state(int k) const {
        KState ks;
        const int lane_k = k & 15;
        ks.walk.init(__builtin_amdgcn_readfirstlane(k - lane_k), dpitch, kw, row_stride);
        ks.lane_bytes = 4 * lane_k;
        return ks;
    }
    __device__ __forceinline__ void advance(KState& ks, const KStep& st) const { ks.walk.advance(st, dpitch, kw); }
    template <bool TAIL>
    __device__ __forceinline__ void load_pair(const RowState& rs, const KState& ks, const KStep&, f32x4& lo, f32x4& hi) const {
        const bool inside = (unsigned)(rs.x + ks.walk.kj) < (unsigned)W && (!TAIL || ks.walk.k < K);
        const unsigned o = inside ? (unsigned)(rs.base + ks.lane_bytes + ks.walk.off) : kOutOfRange;
        lo = buffer_load_quad(make_rsrc(src, bytes), o);
        hi = buffer_load_quad(make_rsrc(src, bytes), o + 16u);
    }
};

// Result addressing: dense matrices (row m at m*ld) or the convolution's output tensor (pixel (y,x) at
// y*row_stride + x*dpitch).  relu: apply relu_by_sign to every result element before it is stored.
struct DenseOut {
    static constexpr bool PRELOAD_C = true;      // "+ C" enters the accumulators before the K walk
    static constexpr bool STREAM_OUT = false;    // (non-temporal stores lose 1.5 % on the ragged 3000x1500x4500 product)
    int ld;
    bool relu = false;
    bool vec = false;      // every row of the result starts 16-byte aligned: runs of consecutive columns go out as one store
    __device__ __forceinline__ size_t offset(int m) const { return (size_t)m * ld; }
    __device__ __forceinline__ bool rows_at_pitch() const { return true; }      // row m starts at pitched_offset(m)
    __device__ __forceinline__ size_t pitched_offset(int m) const { return (size_t)m * ld; }
    __device__ __forceinline__ float finish(float v) const { return relu ? relu_by_sign(v) : v; }
};
struct TensorOut {
    int Wout, dpitch;
    size_t row_stride;
    bool dense;      // row_stride == Wout*dpitch: pixel m simply starts at m*dpitch, no division needed
    bool relu = false;
    static constexpr bool vec = false;
    static constexpr bool PRELOAD_C = false;     // the "+ C" operand is a bias row, added to the finished sum
    static constexpr bool STREAM_OUT = true;     // the result is written once and not read by this launch: non-temporal stores
    __device__ __forceinline__ float finish(float v) const { return relu ? relu_by_sign(v) : v; }
    __device__ __forceinline__ bool rows_at_pitch() const { return dense; }
    __device__ __forceinline__ size_t pitched_offset(int m) const { return (size_t)m * dpitch; }
    __device__ __forceinline__ size_t offset(int m) const {
        if (dense) return (size_t)m * dpitch;
        const int y = m / Wout, x = m - y * Wout;
        return (size_t)y * row_stride + (size_t)x * dpitch;
    }
};

// ---------------------------------------------------------------------------------------------------------------
// B-operand sources.  Interface (S = SgemmShape):
//   ROW_MAJOR_LDS, lds_floats<S>()               which LDS layout the source keeps, and the size of one buffer of it
//   quads<S>()                                   staging registers (float4) per thread and K step
//   k_state<S>(tid, k_begin, bn0, lds_buf0) / k_step<S>() / advance(ks, step)
//                                                position of the K step to fetch next (plus whatever per-thread
//                                                constants the source wants to keep: filter offsets, LDS addresses)
//   load<S, TAIL>(stage, tid, ks, bn0, step)     fetch this thread's share of B[k0 .. k0+BK) x [bn0 .. bn0+BN)
//   writes<S>() / write_one<S>(buf0, buf, stage, tid, ks, W)
//                                                LDS store instructions per thread and step, and the W-th of them
//   frag_reads<S>() / read_frags<S>(buf, s, lh, li, wn0, frag)
//                                                LDS reads per k-group, and the operands of k-group s for this lane
//   strip_col<S>(ni, li)                         column (within the wave's strip) that lane li holds in block ni
// ---------------------------------------------------------------------------------------------------------------
// B as a row-major K x N matrix.  Staging copies 16-byte pieces of rows straight through: task t of a K step is
// row t / (BN/4), column group t % (BN/4), so a wave reads and writes whole kilobytes of consecutive addresses.  Rows
// are BN + 8 floats apart in LDS (BN + 32 when a lane reads a single float, where both half-waves of a fragment read,
// touching adjacent rows, are serviced together and have to land on opposite halves of the 64 banks).
template <bool VEC>
struct DenseB {
    const float* B;
    int ldb, N, K;
    size_t batch_stride;
    static constexpr bool ROW_MAJOR_LDS = true;
    __device__ __forceinline__ void select_batch(int b) { B += (size_t)b * batch_stride; }
    __device__ __forceinline__ void set_k_end(int k_end) { K = k_end; }
    template <class S>
    static constexpr int row_floats() { return S::BN + (S::NI == 1 ? 32 : 8); }
    template <class S>
    static constexpr int lds_floats() { return S::BK * row_floats<S>(); }      // one buffer
    template <class S>
    static constexpr int quads() {
        static_assert((S::BK * S::BN / 4) % S::NT == 0, "B staging must divide evenly over the threads");
        return S::BK * S::BN / 4 / S::NT;
    }
    template <class S>
    static constexpr int frag_reads() { return 4; }                           // LDS reads per quad pair: one per k-slot pair
    struct KState {
        int k0;
    };
    struct KStep {
        int dk;
    };
    template <class S>
    __device__ __forceinline__ KState k_state(int tid, int k_begin, int bn0, const float*) const { return KState{k_begin}; }
    template <class S>
    __device__ __forceinline__ KStep k_step() const { return KStep{S::BK}; }
    __device__ __forceinline__ void advance(KState& ks, const KStep& st) const { ks.k0 += st.dk; }

    template <class S, bool TAIL>
    __device__ __forceinline__ void load(f32x4* st, int tid, const KState& ks, int bn0, const KStep&) const {
        constexpr int CG = S::BN / 4;
#pragma unroll
        for (int p = 0; p < quads<S>(); ++p) {
            const int task = tid + p * S::NT;
            const int k = ks.k0 + task / CG, col = bn0 + 4 * (task % CG);
            f32x4 v = {0.f, 0.f, 0.f, 0.f};
            if (!TAIL || k < K) {
                if (VEC) {
                    const int cc = clamp_group_col(col, N, 4);   // stay inside the operand; such columns are never stored
                    v = *reinterpret_cast<const f32x4*>(B + (size_t)k * ldb + cc);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < N) v[e] = B[(size_t)k * ldb + col + e];
                }
            }
            st[p] = v;
        }
    }
    // LDS store instructions per thread and step, and store number W of them (W a compile-time tag)
    template <class S>
    static constexpr int writes() { return quads<S>(); }
    template <class S, class KS, class WTag>
    __device__ __forceinline__ void write_one(float* buf0, int buf, const f32x4* st, int tid, const KS&, WTag) const {
        constexpr int CG = S::BN / 4, W = WTag::value;
        const int task = tid + W * S::NT;
        *reinterpret_cast<f32x4*>(buf0 + buf * lds_floats<S>() + (task / CG) * row_floats<S>() + 4 * (task % CG)) = st[W];
    }
    // operands of k-group s for this lane: frag[e][ni] = B[k(s, e, lh)][wn0 + NI*li + ni], k = 8s + 2e + lh
    template <class S>
    __device__ __forceinline__ void read_frags(const float* buf, int s, int lh, int li, int wn0, float (*frag)[S::NI]) const {
        typedef float vec_t __attribute__((ext_vector_type(S::NI)));
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float* at = buf + (8 * s + 2 * e + lh) * row_floats<S>() + wn0 + S::NI * li;
            if constexpr (S::NI == 3) {
                // 12-byte runs are not aligned for a vector read; three single reads (lanes 3 floats apart: no bank conflict)
#pragma unroll
                for (int ni = 0; ni < 3; ++ni) frag[e][ni] = at[ni];
            } else {
                const vec_t v = *reinterpret_cast<const vec_t*>(at);
#pragma unroll
                for (int ni = 0; ni < S::NI; ++ni) frag[e][ni] = v[ni];
            }
        }
    }
    // column (relative to the wave's strip) held by lane li in block ni
    template <class S>
    __device__ __forceinline__ static int strip_col(int ni, int li) { return S::NI * li + ni; }
    // (half blocks of 16 rows exist for the filter-bank layout only; never called)
    template <class S>
    __device__ __forceinline__ void read_half_frags(const float*, int, int, int, float (*)[2]) const {}
};

// B as a bank of N filters, filter n holding its taps channel-innermost: column n of the lowered GEMM is filter n and
// four consecutive k (same tap, four channels) are already contiguous in memory, so a k-quad is one 16-byte load.
// Same 32-bit offsets against a buffer resource as Im2colA (the bank stays below 2 GiB), same meaning of PAIRED.
template <bool PAIRED>
struct FilterB {
    const float* filt;
    int N, K, dpitch, kw;
    int filt_stride, filt_row_stride;      // floats between filters / between tap rows of one filter
    unsigned bytes;
    static constexpr bool ROW_MAJOR_LDS = false;
    __device__ __forceinline__ void select_batch(int) {}
    __device__ __forceinline__ void set_k_end(int k_end) { K = k_end; }
    // a staging task is 8 consecutive k (one k-group s) of one filter n: two 16-byte loads, de-interleaved into the
    // even-k and odd-k planes.  Task id = tid + j*NT: group s = id % GROUPS, filter (id / GROUPS) % BN -- when there are
    // more threads than tasks the surplus repeats earlier tasks, which is harmless and keeps the loop branch-free.
    template <class S>
    static constexpr int tasks() { return (S::BN * (S::KQ / 2) + S::NT - 1) / S::NT; }
    template <class S>
    static constexpr int quads() { return 2 * tasks<S>(); }
    template <class S>
    static constexpr int lds_floats() { return 4 * S::KQ * S::B_ROW; }          // one buffer
    template <class S>
    static constexpr int frag_reads() { return S::NI; }                        // one k-quad per 32-column block
    template <int TASKS>
    struct KStateT {
        TapWalk walk;                 // the first quad of this thread's k-group (the same group for all its tasks)
        int filter_base[TASKS];       // byte offset of each task's filter
        unsigned store_addr[2][TASKS][2];   // LDS byte address of each task's even-k / odd-k quad, per buffer
    };
    typedef TapStep KStep;
    template <class S>
    __device__ __forceinline__ KStateT<tasks<S>()> k_state(int tid, int k_begin, int bn0, const float* lds_buf0) const {
        constexpr int G = S::KQ / 2;
        static_assert(S::NT % G == 0, "every task of a thread must fall into the same k-group");
        KStateT<tasks<S>()> ks;
        ks.walk.init(k_begin + 8 * (tid % G), dpitch, kw, filt_row_stride);
        const unsigned base = lds_byte_address(lds_buf0);
#pragma unroll
        for (int j = 0; j < tasks<S>(); ++j) {
            const int id = tid + j * S::NT;
            const int s = id % G, col = (id / G) % S::BN;
            int n = bn0 + col;
            if (n >= N) n = N - 1;
            ks.filter_base[j] = 4 * n * filt_stride;
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int par = 0; par < 2; ++par)
                    ks.store_addr[b][j][par] = base + 4u * (unsigned)(b * lds_floats<S>()) + 16u * (unsigned)((2 * s + par) * S::B_ROW + b_slot(col));
        }
        return ks;
    }
    template <class S>
    __device__ __forceinline__ KStep k_step() const { return TapStep::make(S::BK, dpitch, kw, filt_row_stride); }
    template <class KS>
    __device__ __forceinline__ void advance(KS& ks, const KStep& st) const { ks.walk.advance(st, dpitch, kw); }

    template <class S, bool TAIL, class KS>
    __device__ __forceinline__ void load(f32x4* st, int tid, const KS& ks, int bn0, const KStep& step) const {
        const bool ok0 = !TAIL || ks.walk.k < K;
        if (PAIRED) {
#pragma unroll
            for (int j = 0; j < tasks<S>(); ++j) {
                const unsigned o = ok0 ? (unsigned)(ks.filter_base[j] + ks.walk.off) : kOutOfRange;
                st[2 * j] = buffer_load_quad(make_rsrc(filt, bytes), o);
                st[2 * j + 1] = buffer_load_quad(make_rsrc(filt, bytes), o + 16u);
            }
        } else {
            const TapWalk second = ks.walk.next_quad(step, dpitch, kw);
            const bool ok1 = !TAIL || second.k < K;
#pragma unroll
            for (int j = 0; j < tasks<S>(); ++j) {
                st[2 * j] = buffer_load_quad(make_rsrc(filt, bytes), ok0 ? (unsigned)(ks.filter_base[j] + ks.walk.off) : kOutOfRange);
                st[2 * j + 1] = buffer_load_quad(make_rsrc(filt, bytes), ok1 ? (unsigned)(ks.filter_base[j] + second.off) : kOutOfRange);
            }
        }
    }
    template <class S>
    static constexpr int writes() { return 4 * tasks<S>(); }
    template <class S, class KS, class WTag>
    __device__ __forceinline__ void write_one(float*, int buf, const f32x4* st, int tid, const KS& ks, WTag) const {
        constexpr int W = WTag::value, J = W / 4;
        lds_write_deinterleaved<W % 4>(buf ? ks.store_addr[1][J][0] : ks.store_addr[0][J][0],
                                       buf ? ks.store_addr[1][J][1] : ks.store_addr[0][J][1], st[2 * J], st[2 * J + 1]);
    }
    // operands of k-group s for this lane: frag[e][ni] = B[8s + 2e + lh][wn0 + 32*ni + li] (plane 2s+lh, element e)
    template <class S>
    __device__ __forceinline__ void read_frags(const float* buf, int s, int lh, int li, int wn0, float (*frag)[S::NI]) const {
        const f32x4* plane = reinterpret_cast<const f32x4*>(buf) + (2 * s + lh) * S::B_ROW;
#pragma unroll
        for (int ni = 0; ni < S::NI; ++ni) {
            const f32x4 v = plane[b_slot(wn0 + ni * 32 + li)];
#pragma unroll
            for (int e = 0; e < 4; ++e) frag[e][ni] = v[e];
        }
    }
    // operands of k-group s for a 16-row half block (v_mfma_f32_16x16x4_f32, lane = 16 * slot + i): bh[c][j] =
    // B[8s + 4j + slot][wn0 + 16c + i] -- plane 2s + slot % 2, elements slot / 2 and 2 + slot / 2 of the column's quad
    template <class S>
    __device__ __forceinline__ void read_half_frags(const float* buf, int s, int lane, int wn0, float (*bh)[2]) const {
        const int slot = lane >> 4, i = lane & 15;
        const f32x4* plane = reinterpret_cast<const f32x4*>(buf) + (2 * s + (slot & 1)) * S::B_ROW;
#pragma unroll
        for (int c = 0; c < 2 * S::NI; ++c) {
            const float* q = reinterpret_cast<const float*>(plane + b_slot(wn0 + 16 * c + i)) + (slot >> 1);
            bh[c][0] = q[0];
            bh[c][1] = q[2];
        }
    }
    template <class S>
    __device__ __forceinline__ static int strip_col(int ni, int li) { return 32 * ni + li; }
};

// FilterB for a channel pitch that is a multiple of the K step, the companion of Im2colAUniform: the walk runs on the
// scalar unit and enters each load as its scalar offset; the lane's own share (its filter, its 0 or 8 floats inside
// the step) is a constant vector offset.  A filter load then costs the vector unit nothing.
struct FilterBUniform : FilterB<true> {
    template <class S>
    __device__ __forceinline__ KStateT<tasks<S>()> k_state(int tid, int k_begin, int bn0, const float* lds_buf0) const {
        constexpr int G = S::KQ / 2;
        KStateT<tasks<S>()> ks = FilterB<true>::template k_state<S>(tid, k_begin, bn0, lds_buf0);
        ks.walk.init(__builtin_amdgcn_readfirstlane(k_begin), dpitch, kw, filt_row_stride);
#pragma unroll
        for (int j = 0; j < tasks<S>(); ++j) ks.filter_base[j] += 32 * (tid % G);
        return ks;
    }
    template <class S, bool TAIL, class KS>
    __device__ __forceinline__ void load(f32x4* st, int tid, const KS& ks, int bn0, const KStep&) const {
        const bool ok = !TAIL || ks.walk.k < K;
#pragma unroll
        for (int j = 0; j < tasks<S>(); ++j) {
            const int v = ok ? ks.filter_base[j] : (int)kOutOfRange;
            st[2 * j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(make_rsrc(filt, bytes), v, ks.walk.off, 0));
            st[2 * j + 1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(make_rsrc(filt, bytes), v + 16, ks.walk.off, 0));
        }
    }
};

template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int WAVES_PER_SIMD_ = 1,
          int STAGE_SETS_ = (WAVES_PER_SIMD_ == 1 ? 2 : 1), bool UNEVEN_M_ = false, bool HALF_BLOCK_ = false>
struct SgemmShape {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int WAVES_PER_SIMD = WAVES_PER_SIMD_;   // occupancy the register budget is held to
    // Staging register sets = how many K steps ahead of the MFMAs the global loads run.  Two sets hide more latency but
    // cost A_PASSES + B quads more float4 registers per lane, which only the 512-register budget of one wave per SIMD
    // holds without spilling.
    static constexpr int STAGE_SETS = STAGE_SETS_;
    static_assert(STAGE_SETS == 1 || STAGE_SETS == 2, "one or two K steps of prefetch");
    static constexpr int NT = WAVES_M * WAVES_N * kWave;
    // UNEVEN_M: two rows of waves share an odd number of 32-row blocks, the upper row taking one more than the lower
    // (224 rows = 4 + 3 blocks).  Waves w and w + WAVES_N land on the same SIMD, so every SIMD carries one wave of
    // each kind and the same number of MFMAs per K step.
    static constexpr bool UNEVEN_M = UNEVEN_M_;
    // HALF_BLOCK (with UNEVEN_M, filter-bank B only): BM is an odd multiple of 16 and what the upper wave row has more
    // than the lower one is a block of 16 rows, computed with v_mfma_f32_16x16x4_f32 (208 rows = 3 1/2 + 3 blocks): tiles
    // a sixteenth finer, for results whose rows divide badly over the CUs in steps of 32.
    static constexpr bool HALF_BLOCK = HALF_BLOCK_;
    static constexpr int MI = HALF_BLOCK ? BM / 64 : UNEVEN_M ? (BM / 32 + 1) / 2 : BM / WAVES_M / 32;      // 32-row blocks of the upper wave row
    static constexpr int MI_LOW = HALF_BLOCK ? MI : UNEVEN_M ? BM / 32 - MI : MI;    // blocks of the other wave rows
    static constexpr int WM = MI * 32 + (HALF_BLOCK ? 16 : 0), WN = BN / WAVES_N;
    static constexpr int NI = WN / 32;
    static constexpr int KQ = BK / 4;                         // k-quads per step
    static constexpr int KGROUPS = KQ / 2;                    // groups of 8 consecutive k per step
    // An A staging task is one k-group of one row (two float4 loads); a thread takes A_TASKS of them per step.
    // When BM*KGROUPS is not a multiple of NT the last pass covers rows past BM: they are staged like any other (loaded
    // from the tile's first row, stored to plane rows BM .. A_STAGED_ROWS-1 that no wave reads), which keeps the K loop
    // free of branches -- a divergent skip would split the loop body into basic blocks and undo its instruction schedule.
    static constexpr int A_TASKS = (BM * KGROUPS + NT - 1) / NT;
    static constexpr int A_PASSES = 2 * A_TASKS;              // float4 global loads of A per thread per step
    static constexpr int A_STAGED_ROWS = A_TASKS * (NT / KGROUPS);
    static constexpr int A_ROW = A_STAGED_ROWS + 2;           // quads per A plane (planes 2 slots out of step mod 8)
    static constexpr int B_ROW = BN + 2;                      // quads per B plane (k-quad layout only)
    static constexpr bool A_PARTIAL = (BM * KGROUPS) % NT != 0;
    template <class BSrc>
    static constexpr size_t lds_bytes() {
        return 2 * ((size_t)KQ * A_ROW * sizeof(f32x4) + (size_t)BSrc::template lds_floats<SgemmShape>() * sizeof(float));
    }
    static_assert(HALF_BLOCK ? (UNEVEN_M && WAVES_M == 2 && BM % 32 == 16 && MI >= 1 && WAVES_N % 4 == 0)
                  : UNEVEN_M ? (WAVES_M == 2 && BM % 32 == 0 && MI_LOW >= 1 && WAVES_N % 4 == 0) : BM % (WAVES_M * 32) == 0,
                  "wave tile must be whole 32x32 blocks (plus one block of 16 rows with HALF_BLOCK)");
    static_assert(BN % (WAVES_N * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(BK % 8 == 0, "a K step is whole quad pairs");
    static_assert(NT % KGROUPS == 0, "A staging: KGROUPS lanes per row");
};

// SPLIT_K: blockIdx.z selects a K range of k_split_len (a multiple of BK); every range adds its partial products to dst
// with fp32 atomics, so dst must hold zeros beforehand and the summation order over ranges is not fixed.  C, if any, is
// added by range 0.
template <bool HAS_C, class Out>
struct HAS_C_PRELOAD_GUARD { static constexpr bool value = HAS_C && Out::PRELOAD_C; };

template <class S, class ASrc, class BSrc, class Out, bool HAS_C, bool SPLIT_K = false>
__global__ __launch_bounds__(S::NT, S::WAVES_PER_SIMD) void sgemm_tile_kernel(ASrc a_src, BSrc b_src, const float* Cin, int ldc, float* D,
                                                           Out out, int M, int N, int K, int tiles_m, int tiles_n,
                                                           int group_m, size_t c_batch_stride, size_t d_batch_stride,
                                                           int k_split_len) {
    const int k_begin = SPLIT_K ? (int)blockIdx.z * k_split_len : 0;
    if (SPLIT_K) {
        const int k_end = k_begin + k_split_len < K ? k_begin + k_split_len : K;
        a_src.set_k_end(k_end);
        b_src.set_k_end(k_end);
        K = k_end - k_begin;          // from here on K is the length of this workgroup's range
    }
    // blockIdx.y walks a batch of independent problems of the same shape
    a_src.select_batch(blockIdx.y);
    b_src.select_batch(blockIdx.y);
    if (HAS_C) Cin += (size_t)blockIdx.y * c_batch_stride;
    D += (size_t)blockIdx.y * d_batch_stride;
    constexpr int BM = S::BM, BN = S::BN, BK = S::BK, NT = S::NT, KQ = S::KQ, NI = S::NI;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    f32x4* As = reinterpret_cast<f32x4*>(lds_raw);                       // [2][KQ][A_ROW]
    float* Bs = reinterpret_cast<float*>(As + 2 * KQ * S::A_ROW);        // [2][layout of the B source]
    constexpr int B_BUF = BSrc::template lds_floats<S>();

    const TileCoord tc = xcd_grouped_tile(blockIdx.x, tiles_m, tiles_n, group_m);
    const int bm0 = tc.tm * BM, bn0 = tc.tn * BN;
    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int wm0 = (wave / S::WAVES_N) * S::WM, wn0 = (wave % S::WAVES_N) * S::WN;
    const int li = lane & 31, lh = lane >> 5;

    // ---- staging assignment -------------------------------------------------------------------------------
    // A: KGROUPS consecutive lanes cover one row's BK floats, 8 consecutive k (two 16-byte quads) each
    constexpr int G = S::KGROUPS;
    const int a_s = tid % G, a_r = tid / G;
    constexpr int A_RSTEP = NT / G;
    typename ASrc::RowState a_rs[S::A_TASKS];
#pragma unroll
    for (int p = 0; p < S::A_TASKS; ++p) {
        const int r = a_r + p * A_RSTEP;
        a_rs[p] = a_src.row_state(bm0 + (S::A_PARTIAL && r >= BM ? 0 : r));
    }
    // With two staging register sets the K step fetched during step t is the one after next (t+2), so a global load
    // has almost two steps of MFMAs to land before its data is moved into LDS; with one set it is step t+1.
    constexpr int B_QUADS = BSrc::template quads<S>();
    constexpr int SETS = S::STAGE_SETS;
    f32x4 a_stage[SETS][S::A_PASSES];
    f32x4 b_stage[SETS][B_QUADS];
    typename ASrc::KState a_ks = a_src.k_state(k_begin + 8 * a_s);   // first quad of this thread's k-group in the next step to fetch
    auto b_ks = b_src.template k_state<S>(tid, k_begin, bn0, Bs);
    // LDS byte addresses of this thread's A staging stores: [buffer][task][even-k plane, odd-k plane]
    unsigned a_waddr[2][S::A_TASKS][2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int p = 0; p < S::A_TASKS; ++p)
#pragma unroll
            for (int par = 0; par < 2; ++par)
                a_waddr[b][p][par] = lds_byte_address(As) + 16u * (unsigned)(b * KQ * S::A_ROW + (2 * a_s + par) * S::A_ROW + a_r + p * A_RSTEP);
    const typename ASrc::KStep a_step = a_src.k_step(BK);
    const typename BSrc::KStep b_step = b_src.template k_step<S>();

    // fetches the next K step (steps are always taken in order) into register set SET and moves the k positions on
    auto load_stage = [&](auto set_tag, auto tail_tag) {
        constexpr int SET = decltype(set_tag)::value;
        constexpr bool TAIL = decltype(tail_tag)::value;
#pragma unroll
        for (int p = 0; p < S::A_TASKS; ++p)
            a_src.template load_pair<TAIL>(a_rs[p], a_ks, a_step, a_stage[SET][2 * p], a_stage[SET][2 * p + 1]);
        b_src.template load<S, TAIL>(b_stage[SET], tid, b_ks, bn0, b_step);
        a_src.advance(a_ks, a_step);
        b_src.advance(b_ks, b_step);
    };

    // LDS store number W of a step (A's first, then B's).  A's 8 consecutive k are de-interleaved on the way: even k to
    // plane 2s, odd k to plane 2s+1.
    constexpr int A_WRITES = 4 * S::A_TASKS, B_WRITES = BSrc::template writes<S>(), WRITE_OPS = A_WRITES + B_WRITES;
    auto write_one = [&](auto set_tag, int buf, auto w_tag) {
        constexpr int SET = decltype(set_tag)::value, W = decltype(w_tag)::value;
        if constexpr (W < A_WRITES) {
            constexpr int P = W / 4;
            lds_write_deinterleaved<W % 4>(buf ? a_waddr[1][P][0] : a_waddr[0][P][0], buf ? a_waddr[1][P][1] : a_waddr[0][P][1],
                                           a_stage[SET][2 * P], a_stage[SET][2 * P + 1]);
        } else {
            b_src.template write_one<S>(Bs, buf, b_stage[SET], tid, b_ks, std::integral_constant<int, W - A_WRITES>{});
        }
    };
    auto store_stage = [&](auto set_tag, int buf) {
        static_for<0, WRITE_OPS>([&](auto w_tag) { write_one(set_tag, buf, w_tag); });
    };

    // Everything from here on depends on how many 32-row blocks the wave owns, a compile-time count: one instance of the
    // K walk and the epilogue per count, chosen per wave below.
    auto run = [&](auto mi_tag, auto half_tag) {
        constexpr int MI = decltype(mi_tag)::value;
        // HALF: this wave also owns the 16 rows below its MI blocks, as 2 NI blocks of 16 x 16 (v_mfma_f32_16x16x4_f32:
        // lane 16 slot + i feeds row i / column i at k-slot slot, per element fma over slots 0..3 in ascending order, and
        // holds rows 4 slot .. 4 slot + 3 of column i) -- two of them per k-group and column block, k ascending
        constexpr bool HALF = decltype(half_tag)::value;
        constexpr int HC = HALF ? 2 * NI : 0;
        static_assert(!HALF || (!BSrc::ROW_MAJOR_LDS && !HAS_C_PRELOAD_GUARD<HAS_C, Out>::value), "half blocks: filter-bank B, C added at the end");
        const int hs = lane >> 4, hi = lane & 15;                 // k-slot and row / column inside a 16 x 16 block
        const int hm0 = wm0 + MI * 32;                            // first row of the half block inside the tile
        // Accumulators start at zero, or at C for dst = A*B + C on dense matrices: the reference's chain starts from C
        // (GEMM.cuh:223), and starting anywhere else would round differently.  A convolution's bias is added at the end.
        constexpr bool PRELOAD_C = HAS_C && Out::PRELOAD_C;
        f32x16 acc[MI][NI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
            for (int ni = 0; ni < NI; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;
        f32x4 acc_h[HC > 0 ? HC : 1];
#pragma unroll
        for (int c = 0; c < HC; ++c) acc_h[c] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (PRELOAD_C && (!SPLIT_K || blockIdx.z == 0)) {
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
#pragma unroll
                    for (int ni = 0; ni < NI; ++ni) {
                        const int n = bn0 + wn0 + BSrc::template strip_col<S>(ni, li);
                        if (m < M && n < N) acc[mi][ni][r] = Cin[(size_t)m * ldc + n];
                    }
                }
        }

        // Fragments of one quad pair s: A, per 32-row block one float4 = four consecutive k of this lane's k-slot; B, per
        // k of the pair (e) and block (ni) one float, fetched as the B source's LDS layout dictates.
        // The half block's operands of a quad pair: ah[j] = A[hm0 + hi][8s + 4j + hs], bh[c][j] = B[8s + 4j + hs][16c + hi],
        // j = 0, 1 -- elements hs / 2 and 2 + hs / 2 of the quad in plane 2s + hs % 2.
        struct Frags {
            f32x4 af[MI];
            float bf[4][NI];
            float ah[2];
            float bh[HC > 0 ? HC : 1][2];
        };
        auto read_frags = [&](int buf, int s, Frags& f) {
            const f32x4* Ab = As + buf * KQ * S::A_ROW;
            const int q = 2 * s + lh;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi) f.af[mi] = Ab[q * S::A_ROW + wm0 + mi * 32 + li];
            b_src.template read_frags<S>(Bs + buf * B_BUF, s, lh, li, wn0, f.bf);
            if constexpr (HALF) {
                const float* aq = reinterpret_cast<const float*>(Ab + (2 * s + (hs & 1)) * S::A_ROW + hm0 + hi) + (hs >> 1);
                f.ah[0] = aq[0];
                f.ah[1] = aq[2];
                b_src.template read_half_frags<S>(Bs + buf * B_BUF, s, lane, wn0, f.bh);
            }
        };
        // MFMAs number lo .. hi-1 of a quad pair: the 4*MI*NI of the 32-row blocks in the order (e, mi, ni), with the HC
        // of the half block for k = 8s .. 8s+3 (j = 0) after those of e = 1 and the HC for k = 8s+4 .. 8s+7 after e = 3.
        constexpr int FULL_MFMAS = 4 * MI * NI, PAIR_MFMAS = FULL_MFMAS + 2 * HC, HALF_PAIR = FULL_MFMAS / 2 + HC;
        auto mfma_range = [&](const Frags& f, auto lo_tag, auto hi_tag) {
            constexpr int LO = decltype(lo_tag)::value, HI = decltype(hi_tag)::value;
#pragma unroll
            for (int i = LO; i < HI; ++i) {
                const int j = i / HALF_PAIR, within = i % HALF_PAIR;      // which half of the pair's k, position inside it
                if (within < FULL_MFMAS / 2) {
                    const int x = j * (FULL_MFMAS / 2) + within;
                    const int e = x / (MI * NI), mi = (x / NI) % MI, ni = x % NI;
                    acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.af[mi][e], f.bf[e][ni], acc[mi][ni], 0, 0, 0);
                } else if constexpr (HALF) {
                    const int c = within - FULL_MFMAS / 2;
                    acc_h[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(f.ah[j], f.bh[c][j], acc_h[c], 0, 0, 0);
                }
            }
        };
        auto compute_stage = [&](int buf) {      // unpipelined: used for the peeled steps only
#pragma unroll
            for (int s = 0; s < KQ / 2; ++s) {
                Frags f;
                read_frags(buf, s, f);
                mfma_range(f, std::integral_constant<int, 0>{}, std::integral_constant<int, PAIR_MFMAS>{});
            }
        };

        // K walk over T steps (the last one partial when K % BK != 0; its loader zero-fills, so computing it is no
        // different).  Step t lives in LDS buffer t&1.  Two sets: step t came through register set t&1; while it is
        // computed, step t+2 is fetched into set t&1 (free since step t went to LDS during step t-1) and step t+1 moves from
        // set (t+1)&1 into the other LDS buffer.  One set: step t+1 is fetched at the start of step t and moved to LDS in its
        // second half.  The bulk of the steps (all whose fetch is a full step) run the software-pipelined body; the last
        // few, with the masking loader, run a plain one.
        const int full_steps = K / BK;
        const int T = full_steps + (full_steps * BK < K ? 1 : 0);
        typedef std::integral_constant<int, 0> Set0;
        typedef std::integral_constant<int, 1> Set1;

        // prologue: the loads of steps 0 and 1 go out back to back, so the tile pays one global round trip, not two
        if (full_steps > 0) load_stage(Set0{}, std::false_type{});
        else load_stage(Set0{}, std::true_type{});
        if constexpr (SETS == 2) {
            if (T > 1) {
                if (full_steps > 1) load_stage(Set1{}, std::false_type{});
                else load_stage(Set1{}, std::true_type{});
            }
        }
        store_stage(Set0{}, 0);
        lds_sync();

        static_assert(KQ == 4, "the pipelined loop is written for two quad pairs per K step");
        constexpr int VMEM_OPS = S::A_PASSES + B_QUADS;     // global loads per thread and step
        constexpr int FRAG_OPS = MI + BSrc::template frag_reads<S>() + (HALF ? 1 + HC : 0);   // LDS reads per quad pair
        Frags f0, f1;

        // Steady state of one K step t (fragments of its first quad pair are in af0/bf0):
        //   pair 0 MFMAs   interleaved with: global loads of step t+SETS, LDS reads of pair 1
        //   pair 1 MFMAs   interleaved with: LDS writes of step t+1 into the other buffer
        //   barrier, then the LDS reads of step t+1's pair 0 hide behind the last few MFMAs of pair 1.
        // Every memory instruction sits between MFMAs, so the matrix pipe is never starved by an in-order wait.
        auto pipelined_step = [&](auto set_tag, int buf) {
            constexpr int SET = decltype(set_tag)::value;
            load_stage(set_tag, std::false_type{});
            read_frags(buf, 1, f1);
            mfma_range(f0, std::integral_constant<int, 0>{}, std::integral_constant<int, PAIR_MFMAS>{});
            // scheduling-group masks: 0x002 VALU, 0x008 MFMA, 0x020 VMEM read, 0x100 DS read, 0x200 DS write
            constexpr int G0 = PAIR_MFMAS / (VMEM_OPS + FRAG_OPS) > 0 ? PAIR_MFMAS / (VMEM_OPS + FRAG_OPS) : 1;
#pragma unroll
            for (int i = 0; i < VMEM_OPS; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, G0, 0);
            }
#pragma unroll
            for (int i = 0; i < FRAG_OPS; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, G0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);

            constexpr int LATE = MI * NI < PAIR_MFMAS / 4 ? MI * NI : PAIR_MFMAS / 4;   // MFMAs kept for after the barrier
            constexpr int EARLY = PAIR_MFMAS - LATE;
            // step t+1 sits in the other set when there are two; buffer buf^1 was last read before the previous barrier.
            // Its LDS stores are spread evenly between the MFMAs, each placement pinned (the de-interleaving stores are
            // inline asm, which the scheduling-group masks cannot name).
            typedef std::integral_constant<int, SETS == 2 ? 1 - SET : 0> StoreSet;
            static_for<0, WRITE_OPS>([&](auto w_tag) {
                constexpr int W = decltype(w_tag)::value;
                write_one(StoreSet{}, buf ^ 1, w_tag);
                mfma_range(f1, std::integral_constant<int, W * EARLY / WRITE_OPS>{}, std::integral_constant<int, (W + 1) * EARLY / WRITE_OPS>{});
                __builtin_amdgcn_sched_barrier(0);
            });
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            read_frags(buf ^ 1, 0, f0);
            mfma_range(f1, std::integral_constant<int, EARLY>{}, std::integral_constant<int, PAIR_MFMAS>{});
            __builtin_amdgcn_sched_group_barrier(0x100, FRAG_OPS, 2);
            __builtin_amdgcn_sched_group_barrier(0x008, LATE, 2);
            __builtin_amdgcn_sched_barrier(0);
        };

        int t = 0;
        if constexpr (SETS == 2) {
            if (full_steps > 2) {
                read_frags(0, 0, f0);
                for (; t + 3 < full_steps; t += 2) {      // steps t and t+1 both fetch a full step (t+2, t+3 < full_steps)
                    pipelined_step(Set0{}, 0);
                    pipelined_step(Set1{}, 1);
                }
                if (t + 2 < full_steps) {
                    pipelined_step(Set0{}, 0);
                    ++t;
                }
            }
            // the remaining steps: at most one more fetch, and that one is the partial step
            for (; t < T; ++t) {
                const int buf = t & 1;
                if (t + 2 < T) {
                    if (buf == 0) load_stage(Set0{}, std::true_type{});
                    else load_stage(Set1{}, std::true_type{});
                }
                compute_stage(buf);
                if (t + 1 < T) {
                    if (buf == 0) store_stage(Set1{}, 1);
                    else store_stage(Set0{}, 0);
                    lds_sync();
                }
            }
        } else {
            if (full_steps > 1) {
                read_frags(0, 0, f0);
                for (; t + 1 < full_steps; ++t) pipelined_step(Set0{}, t & 1);   // fetches step t+1, a full one
            }
            for (; t < T; ++t) {
                const int buf = t & 1;
                if (t + 1 < T) load_stage(Set0{}, std::true_type{});
                compute_stage(buf);
                if (t + 1 < T) {
                    store_stage(Set0{}, buf ^ 1);
                    lds_sync();
                }
            }
        }

        // ---- epilogue.  Lane li holds, per row, the columns strip_col(ni, li) of its wave's strip: NI consecutive ones when B
        // came from a row-major matrix (one vector store per row where alignment and the edge allow), 32 apart otherwise.
        // dst = A*B + C adds C here (C may alias dst: every element is read and written by the same lane).
        // FULL: the whole tile lies inside the result and row m starts at m times the pitch -- no bounds checks (each
        // one is a branch around its store) and no division per row; the choice is one scalar branch per workgroup.
        auto store_rows = [&](auto full_tag) {
            constexpr bool FULL = decltype(full_tag)::value;
#pragma unroll
            for (int mi = 0; mi < MI; ++mi)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = bm0 + wm0 + mi * 32 + (r >> 2) * 8 + lh * 4 + (r & 3);
                    if (FULL || m < M) {
                        float* drow = D + (FULL ? out.pitched_offset(m) : out.offset(m));
                        const float* crow = HAS_C ? Cin + (size_t)m * ldc : nullptr;
                        const bool add_c = HAS_C && !PRELOAD_C && (!SPLIT_K || blockIdx.z == 0);
                        if (BSrc::ROW_MAJOR_LDS && !SPLIT_K && NI > 1 && NI != 3) {      // runs of 3 floats are not aligned for one store
                            const int n0 = bn0 + wn0 + NI * li;
                            if (out.vec && (FULL || n0 + NI <= N)) {
                                typedef float vec_t __attribute__((ext_vector_type(NI)));
                                vec_t v;
#pragma unroll
                                for (int ni = 0; ni < NI; ++ni) v[ni] = out.finish(add_c ? acc[mi][ni][r] + crow[n0 + ni] : acc[mi][ni][r]);
                                *reinterpret_cast<vec_t*>(drow + n0) = v;
                                continue;
                            }
                        }
#pragma unroll
                        for (int ni = 0; ni < NI; ++ni) {
                            const int n = bn0 + wn0 + BSrc::template strip_col<S>(ni, li);
                            if (FULL || n < N) {
                                const float v = add_c ? acc[mi][ni][r] + crow[n] : acc[mi][ni][r];
                                if (SPLIT_K) unsafeAtomicAdd(drow + n, v);      // hardware fp32 add in L2
                                else if constexpr (Out::STREAM_OUT) __builtin_nontemporal_store(out.finish(v), drow + n);
                                else drow[n] = out.finish(v);
                            }
                        }
                    }
                }
        };
        if (!SPLIT_K && out.rows_at_pitch() && bm0 + BM <= M && bn0 + BN <= N) store_rows(std::true_type{});
        else store_rows(std::false_type{});
        if constexpr (HALF) {
            // the half block: lane (hs, hi) holds rows 4 hs .. 4 hs + 3 of column 16 c + hi
            const bool full = out.rows_at_pitch() && bm0 + BM <= M && bn0 + BN <= N;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = bm0 + hm0 + 4 * hs + r;
                if (full || m < M) {
                    float* drow = D + (full ? out.pitched_offset(m) : out.offset(m));
                    const float* crow = HAS_C ? Cin + (size_t)m * ldc : nullptr;
#pragma unroll
                    for (int c = 0; c < HC; ++c) {
                        const int n = bn0 + wn0 + 16 * c + hi;
                        if (full || n < N) __builtin_nontemporal_store(out.finish(HAS_C ? acc_h[c][r] + crow[n] : acc_h[c][r]), drow + n);
                    }
                }
            }
        }
    };
    if constexpr (S::UNEVEN_M) {
        // a branch on the scalar unit: the two wave rows run different instances, with the same sequence of barriers
        if (__builtin_amdgcn_readfirstlane(wave) < S::WAVES_N) run(std::integral_constant<int, S::MI>{}, std::integral_constant<bool, S::HALF_BLOCK>{});
        else run(std::integral_constant<int, S::MI_LOW>{}, std::false_type{});
    } else {
        run(std::integral_constant<int, S::MI>{}, std::false_type{});
    }
}

}  // namespace decx_hip
