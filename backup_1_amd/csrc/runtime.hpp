// State and helpers shared by the translation units of libdecx_hip.so (each .hip file instantiates one family of
// kernels, so that they compile side by side): the library's runtime record, the status-code helpers, the launch
// description of a batch and the enqueue functions the C ABI calls.
#pragma once
#include "../../include/decx_hip.h"

#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

namespace decx_hip {

struct Runtime {
    bool is_init = false;
    int device = -1;
    int compute_units = 0;
    int clock_khz = 0;
    size_t hbm_bytes = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    int sgemm_variant = 0;
    int hgemm_variant = 0;
    float* partial = nullptr;      // fp32 workspace of the fp16 split-K path, grown on demand, kept until the process ends
    size_t partial_bytes = 0;
    int splitk_atomic = 0;         // fp16 split-K: 0 = one workspace plane per K range, added in range order (the same
                                   // result on every run); 1 = all ranges add into one plane with atomics
    int spin_wait_us = 2000;       // a blocking compute call polls its completion word this long before it waits in
                                   // hipStreamSynchronize (env DECX_HIP_SPIN_WAIT_US overrides; 0 = wait there at once)
    unsigned* done_flag = nullptr; // pinned, host-coherent word a one-lane kernel behind the work stores done_seq to
    unsigned done_seq = 0;
    int group_m = 8;   // tile-rows per raster group of the XCD-aware tile walk (env DECX_HIP_GROUP_M overrides, for tuning)
};
extern Runtime g_rt;

// sets the calling thread's error string (decx_hip_last_error) and returns `code`
int fail(int code, const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e_ = (expr);                         \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

int need_init();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int cdiv(int a, int b) { return (a + b - 1) / b; }

// The convolution kernels on patch-shaped tiles (sconv_dma.hpp, hconv_mfma16.hpp) address the image with 32-bit byte
// offsets through a buffer resource and throw a load out of the tensor's range by adding 2^31 to its offset.  That works
// while every offset they form stays below 2^31 before the addition and wraps past 2^32 - (apron) after it: the tensor's
// bytes, plus the apron's negative offsets (oy rows and ox pixels before the first, and a 16-byte unit), plus the
// patches' reach past the output (up to 16 rows and 16 columns) and the taps' (kh rows, kw pixels) must stay below 2^31.
// Strides and pitches in elements of elem_bytes.
inline bool conv_patch_offsets_fit(size_t src_bytes, size_t row_stride, size_t dpitch, int kh, int kw, int oy, int ox, size_t elem_bytes) {
    const size_t apron_bytes = ((size_t)oy * row_stride + (size_t)ox * dpitch) * elem_bytes + 16;
    const size_t reach_bytes = ((size_t)(16 + kh) * row_stride + (size_t)(16 + kw) * dpitch) * elem_bytes;
    return src_bytes + apron_bytes + reach_bytes < 0x80000000ull;
}

// A batch of `count` independent, equally shaped problems; the strides are in elements between consecutive problems.
// Every launcher enqueues on `stream`.
struct Batch {
    int count = 1;
    size_t stride_a = 0, stride_b = 0, stride_c = 0, stride_d = 0;
    hipStream_t stream = nullptr;
};

int check_gemm_args(const void* A, int lda, const void* B, int ldb, const void* Cin, int ldc, const void* D, int ldd, int M,
                    int N, int K, const Batch& batch);

// zero-fills the M x N region of a pitched matrix on `stream` (the split-K kernels accumulate into it)
void enqueue_zero_region(float* D, int ldd, int M, int N, hipStream_t stream);

// the fp32 workspace of the fp16 split-K paths (g_rt.partial): grown on demand, kept until the process ends
int ensure_partial(size_t need);

// Enqueue functions, one family per translation unit.  Each checks its arguments, picks a kernel and launches it on
// the given stream (the library's, where none is passed) without waiting.
int sgemm_enqueue(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                  int N, int K, const Batch& batch, bool relu = false);
int sgemm_splitk_enqueue(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                         int N, int K, int splits);
int conv_enqueue(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt, int N, int kh,
                 int kw, size_t filt_stride, size_t filt_row_stride, float* dst, int dst_dpitch, size_t dst_row_stride,
                 int flag, const float* bias = nullptr, bool relu = false);
int hgemm_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                  int ldd, int M, int N, int K, const Batch& batch);
// host-only: which kernel the two entry points above take for a product of these sizes and pitches (no device call)
int sgemm_plan(int M, int N, int K, int batch, long lda, long ldb, bool aligned);
int conv_plan_split(int Hout, int Wout, int N, int K, int* shape);
int sgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, bool aligned, int* shape, int* by_columns);
int hgemm_plan(int M, int N, int K, int batch, long lda, long ldb, bool aligned, int* splits);
int hgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, bool aligned, int* by_columns);
// the K-range route of hgemm_enqueue on the library's static device workspace (no allocation); splits <= 0: automatic
int hgemm_splitk_static_enqueue(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                uint16_t* D, int ldd, int M, int N, int K, int splits);
// looks up the device address of the static workspace for the current device and prepares the kernels that use it
int hgemm_static_scratch_init(int device);
int hconv_enqueue(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt, int N, int kh,
                  int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst, int dst_dpitch, size_t dst_row_stride,
                  int flag, const uint16_t* bias, bool relu);

}  // namespace decx_hip
