// Shared pieces of the gfx950 contraction kernels: vector types, the XCD-aware tile walk, status codes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace decx_hip {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;      // CDNA wavefront width
constexpr int kXcds = 8;       // MI355X: 8 accelerator complex dies, 32 CUs and one 4 MiB L2 each

// ReLU exactly as the reference's element-wise kernel computes it (nn/operators/ReLU.h:57-82): the value times
// float(sign bit clear).  Hence a negative input gives -0.0f, -inf gives NaN, NaN stays NaN.
__device__ __forceinline__ float relu_by_sign(float v) {
    return (float)((~__float_as_uint(v)) >> 31) * v;
}

// Where a loader fetches the `unit`-wide column group that starts at column `col` (a multiple of `unit`) of a
// row-major B with N valid columns: groups that start at or beyond N rounded up to `unit` are moved back onto the last
// group that holds a valid column.  Such columns are computed and never stored.  The bound is the extent of the
// operand the caller described, not its pitch: B may be a column range of a wider matrix (pointer moved right, parent
// pitch), and then B + ldb of the last row lies beyond the parent's allocation.  With B 16-byte aligned and ldb a
// multiple of `unit`, N rounded up to `unit` never exceeds the parent's pitch.
__host__ __device__ __forceinline__ constexpr int clamp_group_col(int col, int N, int unit) {
    const int last = (N + unit - 1) / unit * unit - unit;
    return col < last ? col : last;
}

// m / d and m % d for 0 <= m < 2^22 and d > 0 by a float reciprocal and one correction step either way
__device__ __forceinline__ void small_divmod(int m, int d, float rcp_d, int& quot, int& rem) {
    int qv = (int)((float)m * rcp_d);
    int r = m - qv * d;
    if (r < 0) { r += d; --qv; }
    if (r >= d) { r -= d; ++qv; }
    quot = qv;
    rem = r;
}

// f(integral_constant<int, I>) for I = I0 .. N-1, unrolled at compile time
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// plane 0 + plane 1 + ... of element i of `planes` fp32 planes `plane` floats apart, added in that order (the fixed
// order is what makes a split-K result the same on every run); the loads of 8 planes are issued together, the
// additions stay sequential
__device__ __forceinline__ float ordered_plane_sum(const float* __restrict__ partial, int planes, size_t plane, size_t i) {
    float v = partial[i];
    int s = 1;
    for (; s + 8 <= planes; s += 8) {
        float p[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) p[j] = __builtin_nontemporal_load(partial + (size_t)(s + j) * plane + i);
#pragma unroll
        for (int j = 0; j < 8; ++j) v += p[j];
    }
    for (; s < planes; ++s) v += partial[(size_t)s * plane + i];
    return v;
}

// One 16-byte-per-lane load from global memory (wave-uniform base + per-lane byte offset) straight into LDS at
// lds_base + 16*lane (lds_base wave-uniform).
__device__ __forceinline__ void dma_load16(const void* sbase, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 : : "v"(lane_off), "s"(sbase), "s"(lds_base) : "memory", "m0");
}

// The same with a tag in the instruction text.  Copies of a code sequence that issue the same loads (two instances of an
// unrolled pass, two branches of a dispatch) are otherwise merged by the compiler into one sequence whose operands are
// selected per copy -- in vector registers, which the scalar operands of this instruction do not accept; texts that
// differ cannot be merged.
template <int TAG>
__device__ __forceinline__ void dma_load16_tagged(const void* sbase, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 ; load %3"
                 : : "v"(lane_off), "s"(sbase), "s"(lds_base), "n"(TAG) : "memory", "m0");
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

// raw buffer resource over [base, base + bytes): stride 0, offsets in bytes, out-of-range reads give zeros
__device__ __forceinline__ i32x4 raw_buffer_words(const void* base, unsigned bytes) {
    const uint64_t b = reinterpret_cast<uint64_t>(base);
    return i32x4{(int)(uint32_t)b, (int)(uint32_t)((b >> 32) & 0xffffu), (int)bytes, 0x00020000};
}

// One 16-byte-per-lane load from a buffer (per-lane byte offset + wave-uniform byte offset) straight into LDS at
// lds_base + 16*lane (lds_base wave-uniform).
__device__ __forceinline__ void dma_buffer_load16(i32x4 rsrc, uint32_t lane_off, uint32_t uniform_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
                 : : "v"(lane_off), "s"(rsrc), "s"(uniform_off), "s"(lds_base) : "memory", "m0");
}

// The same with a tag in the instruction text (see dma_load16_tagged).
template <int TAG>
__device__ __forceinline__ void dma_buffer_load16_tagged(i32x4 rsrc, uint32_t lane_off, uint32_t uniform_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds ; load %4"
                 : : "v"(lane_off), "s"(rsrc), "s"(uniform_off), "s"(lds_base), "n"(TAG) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_dma_then_barrier() {
    // my loads older than the N most recent have landed; my LDS reads are done; then everybody meets
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" : : "n"(N) : "memory");
}

struct TileCoord {
    int tm, tn;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Re-number them so that the ids living on one XCD
// form one contiguous run of a "grouped" raster (group_m tile-rows tall, walked column by column): the tiles that
// are resident on an XCD at the same time then share A row-panels and B column-panels in that XCD's private L2.
__device__ __forceinline__ TileCoord xcd_grouped_tile(int pid, int tiles_m, int tiles_n, int group_m) {
    const int total = tiles_m * tiles_n;
    const int xcd = pid % kXcds;
    const int local = pid / kXcds;
    const int base = total / kXcds, rem = total % kXcds;
    const int start = xcd * base + (xcd < rem ? xcd : rem);
    const int id = start + local;
    const int per_group = group_m * tiles_n;
    const int group = id / per_group;
    const int first_m = group * group_m;
    const int rows = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
    const int in_group = id - group * per_group;
    TileCoord t;
    t.tm = first_m + in_group % rows;
    t.tn = in_group / rows;
    return t;
}

}  // namespace decx_hip
