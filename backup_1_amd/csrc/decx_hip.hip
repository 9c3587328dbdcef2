// C ABI of libdecx_hip.so: device bring-up, memory, host-resident pipelines, ReLU, and the entry points that call the
// enqueue functions of the kernel families (sgemm_dense.hip, sgemm_conv.hip, hgemm.hip, hconv.hip).
// Declarations and the reference interface each entry point stands in for: include/decx_hip.h.
#include "runtime.hpp"

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "tile_common.hpp"

namespace decx_hip {

Runtime g_rt;

namespace {
thread_local char g_err[512] = "No error\n";   // SUCCESS string of the reference, core/error.h:61
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char* what) {
    return fail(DECX_HIP_FAIL_HIP_BASE + (int)e, "%s: %s\n", what, hipGetErrorString(e));
}

int need_init() { return fail(DECX_HIP_FAIL_NOT_INIT, "CUDA should be initialized first\n"); }   // core/error.h:60

// zero-fills the M x N region of a pitched matrix (the split-K kernel accumulates into it)
__global__ __launch_bounds__(256) void zero_region_kernel(float* D, int ldd, int M, int N) {
    const size_t total = (size_t)M * N;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        D[(i / N) * ldd + i % N] = 0.f;
}
void enqueue_zero_region(float* D, int ldd, int M, int N, hipStream_t stream) {
    const size_t total = (size_t)M * N;
    const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(zero_region_kernel, dim3(blocks), dim3(256), 0, stream, D, ldd, M, N);
}

int check_gemm_args(const void* A, int lda, const void* B, int ldb, const void* Cin, int ldc, const void* D, int ldd, int M,
                    int N, int K, const Batch& batch) {
    if (!g_rt.is_init) return need_init();
    if (!A || !B || !D) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null matrix pointer\n");
    if (M <= 0 || N <= 0 || K <= 0 || batch.count <= 0) return fail(DECX_HIP_FAIL_DIMS, "Matrix Dims don't match each other");
    if (lda < K || ldb < N || ldd < N || (Cin && ldc < N))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "leading dimension smaller than the row length\n");
    if (batch.count > 1 && (batch.stride_a < (size_t)(M - 1) * lda + K || batch.stride_b < (size_t)(K - 1) * ldb + N ||
                            batch.stride_d < (size_t)(M - 1) * ldd + N || (Cin && batch.stride_c < (size_t)(M - 1) * ldc + N)))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "batch stride smaller than one matrix\n");
    return 0;
}

// the fp32 workspace of the fp16 split-K paths: reserved by decx_hip_init for every split the library chooses by itself
// (at most one 128x128 tile and range per CU, twice that in the atomic mode's tile count), grown only for larger forced
// splits, kept until the process ends
int ensure_partial(size_t need) {
    if (need <= g_rt.partial_bytes) return 0;
    HIP_TRY(hipDeviceSynchronize());               // earlier launches may still use the old workspace
    if (g_rt.partial) HIP_TRY(hipFree(g_rt.partial));
    g_rt.partial = nullptr;
    g_rt.partial_bytes = 0;
    if (hipMalloc(&g_rt.partial, need) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    }
    g_rt.partial_bytes = need;
    return 0;
}

}  // namespace decx_hip

using namespace decx_hip;

namespace {

Batch single_on_library_stream() {
    Batch b;
    b.stream = g_rt.stream;
    return b;
}
Batch batch_on_library_stream(int count, size_t sa, size_t sb, size_t sc, size_t sd) {
    Batch b;
    b.count = count;
    b.stride_a = sa;
    b.stride_b = sb;
    b.stride_c = sc;
    b.stride_d = sd;
    b.stream = g_rt.stream;
    return b;
}

// ---------------------------------------------------------------------------------------------------------------
// What the host-matrix pipelines keep between calls, like the reference keeps its device blocks in a pool
// (core/memory_management/MemoryPool_D.h) until de::release_all_tmp (Memory_pool.h:23-37): device blocks, the copy
// streams and the events.  Allocating and freeing three 256 MiB blocks and creating the streams costs 2 ms of a
// 14 ms call at 8192^3.  Every pipeline call ends with all of its work complete, so whatever it used is free again
// when it returns; decx_hip_release_tmp gives the blocks back to the runtime.
// ---------------------------------------------------------------------------------------------------------------
struct TmpBlock {
    void* ptr;
    size_t bytes;
    bool in_use;
};
constexpr int kMaxTmpBlocks = 16, kPipeEvents = 40;
TmpBlock g_tmp[kMaxTmpBlocks];
int g_tmp_count = 0;
struct PipeObjects {
    hipStream_t up = nullptr, down = nullptr;                    // uploads, downloads (kernels run on the library's stream)
    hipEvent_t ev[kPipeEvents] = {};
    bool ready = false;
} g_pipe;

int free_idle_tmp_blocks() {
    int kept = 0;
    hipError_t first = hipSuccess;
    for (int i = 0; i < g_tmp_count; ++i) {
        if (g_tmp[i].in_use) {
            g_tmp[kept++] = g_tmp[i];
        } else {
            const hipError_t e = hipFree(g_tmp[i].ptr);
            if (e != hipSuccess && first == hipSuccess) first = e;
        }
    }
    g_tmp_count = kept;
    return first == hipSuccess ? 0 : hip_fail(first, "hipFree");
}

// the smallest idle block that holds `bytes` without being more than twice as large (+ 16 MiB); else a new one
void* tmp_acquire(size_t bytes) {
    int best = -1;
    for (int i = 0; i < g_tmp_count; ++i)
        if (!g_tmp[i].in_use && g_tmp[i].bytes >= bytes && g_tmp[i].bytes <= 2 * bytes + ((size_t)16 << 20) &&
            (best < 0 || g_tmp[i].bytes < g_tmp[best].bytes))
            best = i;
    if (best >= 0) {
        g_tmp[best].in_use = true;
        return g_tmp[best].ptr;
    }
    if (g_tmp_count == kMaxTmpBlocks) (void)free_idle_tmp_blocks();
    if (g_tmp_count == kMaxTmpBlocks) return nullptr;
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();
        (void)free_idle_tmp_blocks();                  // make room and try once more
        if (hipMalloc(&p, bytes) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
    }
    g_tmp[g_tmp_count++] = TmpBlock{p, bytes, true};
    return p;
}
void tmp_release(void* p) {
    for (int i = 0; i < g_tmp_count; ++i)
        if (g_tmp[i].ptr == p) g_tmp[i].in_use = false;
}

int pipe_objects() {
    if (g_pipe.ready) return 0;
    HIP_TRY(hipStreamCreateWithFlags(&g_pipe.up, hipStreamNonBlocking));
    HIP_TRY(hipStreamCreateWithFlags(&g_pipe.down, hipStreamNonBlocking));
    for (hipEvent_t& e : g_pipe.ev) HIP_TRY(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    g_pipe.ready = true;
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Host-resident batches (the MatrixArray GEMM3 of the reference): one matrix triple per pipeline step, two device
// buffer sets, uploads / kernel / downloads on three streams chained by events, so that the copies of steps i+1 and
// i-1 run under the kernel of step i.
// ---------------------------------------------------------------------------------------------------------------
template <typename T, class Enqueue>
int gemm3_host_pipeline(const T* hA, int lda, size_t plane_a, const T* hB, int ldb, size_t plane_b, const T* hC, int ldc,
                        size_t plane_c, T* hD, int ldd, size_t plane_d, int M, int N, int K, int count, Enqueue enqueue) {
    if (!g_rt.is_init) return need_init();
    if (!hA || !hB || !hD) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null matrix pointer\n");
    if (M <= 0 || N <= 0 || K <= 0 || count <= 0) return fail(DECX_HIP_FAIL_DIMS, "Matrix Dims don't match each other");
    if (lda < K || ldb < N || ldd < N || (hC && ldc < N))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "leading dimension smaller than the row length\n");
    const size_t bytes_a = (size_t)M * lda * sizeof(T), bytes_b = (size_t)K * ldb * sizeof(T), bytes_d = (size_t)M * ldd * sizeof(T);
    struct Set { T *a = nullptr, *b = nullptr, *d = nullptr; hipEvent_t up = nullptr, done = nullptr, down = nullptr; } set[2];
    if (int rc0 = pipe_objects()) return rc0;
    const hipStream_t s_up = g_pipe.up, s_down = g_pipe.down;
    int rc = 0;
    auto cleanup = [&] {
        (void)hipDeviceSynchronize();
        for (Set& s : set) {
            if (s.a) tmp_release(s.a);
            if (s.b) tmp_release(s.b);
            if (s.d) tmp_release(s.d);
        }
    };
#define PIPE_TRY(expr)                                   \
    do {                                                 \
        hipError_t e_ = (expr);                          \
        if (e_ != hipSuccess) { rc = hip_fail(e_, #expr); cleanup(); return rc; } \
    } while (0)
    for (int i = 0; i < 2; ++i) {
        Set& s = set[i];
        s.a = static_cast<T*>(tmp_acquire(bytes_a));
        s.b = static_cast<T*>(tmp_acquire(bytes_b));
        s.d = static_cast<T*>(tmp_acquire(bytes_d));
        if (!s.a || !s.b || !s.d) {
            cleanup();
            return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
        }
        s.up = g_pipe.ev[3 * i], s.done = g_pipe.ev[3 * i + 1], s.down = g_pipe.ev[3 * i + 2];
    }
    auto upload = [&](int i) -> hipError_t {
        Set& s = set[i & 1];
        hipError_t e;
        if (i >= 2 && (e = hipStreamWaitEvent(s_up, s.done, 0)) != hipSuccess) return e;    // kernel i-2 has read a, b
        if (hC && i >= 2 && (e = hipStreamWaitEvent(s_up, s.down, 0)) != hipSuccess) return e;   // and d was drained
        if ((e = hipMemcpyAsync(s.a, hA + (size_t)i * plane_a, bytes_a, hipMemcpyHostToDevice, s_up)) != hipSuccess) return e;
        if ((e = hipMemcpyAsync(s.b, hB + (size_t)i * plane_b, bytes_b, hipMemcpyHostToDevice, s_up)) != hipSuccess) return e;
        if (hC && (e = hipMemcpy2DAsync(s.d, (size_t)ldd * sizeof(T), hC + (size_t)i * plane_c, (size_t)ldc * sizeof(T),
                                        (size_t)N * sizeof(T), M, hipMemcpyHostToDevice, s_up)) != hipSuccess) return e;
        return hipEventRecord(s.up, s_up);
    };
    PIPE_TRY(upload(0));
    for (int i = 0; i < count; ++i) {
        Set& s = set[i & 1];
        if (i + 1 < count) PIPE_TRY(upload(i + 1));
        PIPE_TRY(hipStreamWaitEvent(g_rt.stream, s.up, 0));
        if (i >= 2) PIPE_TRY(hipStreamWaitEvent(g_rt.stream, s.down, 0));                   // result i-2 has left d
        Batch one;
        one.stream = g_rt.stream;
        rc = enqueue(s.a, s.b, hC ? s.d : nullptr, s.d, one);
        if (rc) { cleanup(); return rc; }
        PIPE_TRY(hipEventRecord(s.done, g_rt.stream));
        PIPE_TRY(hipStreamWaitEvent(s_down, s.done, 0));
        PIPE_TRY(hipMemcpy2DAsync(hD + (size_t)i * plane_d, (size_t)ldd * sizeof(T), s.d, (size_t)ldd * sizeof(T),
                                  (size_t)N * sizeof(T), M, hipMemcpyDeviceToHost, s_down));
        PIPE_TRY(hipEventRecord(s.down, s_down));
    }
    PIPE_TRY(hipStreamSynchronize(s_down));
    PIPE_TRY(hipStreamSynchronize(g_rt.stream));
    PIPE_TRY(hipStreamSynchronize(s_up));
#undef PIPE_TRY
    for (Set& s_ : set) {
        tmp_release(s_.a);
        tmp_release(s_.b);
        tmp_release(s_.d);
    }
    return 0;
}

// One GEMM on HOST-resident matrices (the Matrix<T> overloads of de::cuda::GEMM, GEMM.h:56-131, :139-228).  The link to
// the host is the bottleneck (8192^3 fp32: 0.54 GB up at 57 GB/s = 9.3 ms against 7.3 ms of kernel), so the uploads never
// pause and the kernel follows them as closely as the data allows: A goes up in row panels, B in column panels, taking
// turns; a new row panel of A is multiplied at once with all column panels of B already there, a new column panel of B
// with all row panels of A already there (one GEMM launch each, on sub-matrices of the device copies), and each finished
// region of the result goes down on a third stream.  Every output is still one whole walk over K: same bits as the
// device-resident call.  Device copies keep the host pitches.  Overlap needs pinned host memory (decx_hip_host_malloc);
// pageable memory works but serialises.
template <typename T, class Enqueue>
int gemm_host_pipeline(const T* hA, int lda, const T* hB, int ldb, const T* hC, int ldc, T* hD, int ldd, int M, int N, int K,
                       Enqueue enqueue) {
    if (!g_rt.is_init) return need_init();
    if (!hA || !hB || !hD) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null matrix pointer\n");
    if (M <= 0 || N <= 0 || K <= 0) return fail(DECX_HIP_FAIL_DIMS, "Matrix Dims don't match each other");
    if (lda < K || ldb < N || ldd < N || (hC && ldc < N))
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "leading dimension smaller than the row length\n");
    // panels of whole 256-wide tiles, at least 512 wide, at most 8 per operand (measured at 2048^3 ... 8192^3: 4 panels
    // per operand 6 % slower at 8192^3, 12 and 16 equal; panels of at least 1024 4 % slower at 2048^3 and 4096^3)
    constexpr int MAX_PANELS = 8, MAX_STEPS = 2 * MAX_PANELS;
    auto panel_extent = [](int extent) {
        int p = cdiv(cdiv(extent, MAX_PANELS), 256) * 256;
        return p < 512 ? 512 : p;
    };
    const int pm = panel_extent(M), pn = panel_extent(N);
    const int panels_a = cdiv(M, pm), panels_b = cdiv(N, pn), steps = panels_a + panels_b;
    static_assert(2 * MAX_STEPS <= kPipeEvents, "an upload and a kernel event per step");
    if (int rc0 = pipe_objects()) return rc0;
    T *dA = nullptr, *dB = nullptr, *dD = nullptr;
    const hipStream_t s_up = g_pipe.up, s_down = g_pipe.down;
    hipEvent_t* const up = g_pipe.ev;
    hipEvent_t* const done = g_pipe.ev + MAX_STEPS;
    int rc = 0;
    auto release_blocks = [&] {
        if (dA) tmp_release(dA);
        if (dB) tmp_release(dB);
        if (dD) tmp_release(dD);
    };
    auto cleanup = [&] {           // after an error: whatever was enqueued must be over before the blocks are used again
        (void)hipDeviceSynchronize();
        release_blocks();
    };
#define PIPE_TRY(expr)                                   \
    do {                                                 \
        hipError_t e_ = (expr);                          \
        if (e_ != hipSuccess) { rc = hip_fail(e_, #expr); cleanup(); return rc; } \
    } while (0)
    dA = static_cast<T*>(tmp_acquire((size_t)M * lda * sizeof(T)));
    dB = static_cast<T*>(tmp_acquire((size_t)K * ldb * sizeof(T)));
    dD = static_cast<T*>(tmp_acquire((size_t)M * ldd * sizeof(T)));
    if (!dA || !dB || !dD) {
        cleanup();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    }
    int a_up = 0, b_up = 0;      // panels of A / B on the device (or on their way, in stream order)
    for (int step = 0; step < steps; ++step) {
        // whichever operand is behind goes next; A first
        const bool next_is_a = b_up == panels_b || (a_up < panels_a && (long)a_up * panels_b <= (long)b_up * panels_a);
        int r0, rows, c0, cols;      // the region of the result that this panel completes the operands of
        if (next_is_a) {
            r0 = a_up * pm, rows = M - r0 < pm ? M - r0 : pm;
            c0 = 0, cols = b_up * pn < N ? b_up * pn : N;
            PIPE_TRY(hipMemcpy2DAsync(dA + (size_t)r0 * lda, (size_t)lda * sizeof(T), hA + (size_t)r0 * lda, (size_t)lda * sizeof(T),
                                      (size_t)K * sizeof(T), rows, hipMemcpyHostToDevice, s_up));
            ++a_up;
        } else {
            c0 = b_up * pn, cols = N - c0 < pn ? N - c0 : pn;
            r0 = 0, rows = a_up * pm < M ? a_up * pm : M;
            PIPE_TRY(hipMemcpy2DAsync(dB + c0, (size_t)ldb * sizeof(T), hB + c0, (size_t)ldb * sizeof(T), (size_t)cols * sizeof(T), K,
                                      hipMemcpyHostToDevice, s_up));
            ++b_up;
        }
        if (rows == 0 || cols == 0) continue;      // the very first panel: its partner is not there yet
        if (hC)   // C goes into the result buffer and is accumulated onto in place, as the reference does (GEMM.h:196-206)
            PIPE_TRY(hipMemcpy2DAsync(dD + (size_t)r0 * ldd + c0, (size_t)ldd * sizeof(T), hC + (size_t)r0 * ldc + c0,
                                      (size_t)ldc * sizeof(T), (size_t)cols * sizeof(T), rows, hipMemcpyHostToDevice, s_up));
        PIPE_TRY(hipEventRecord(up[step], s_up));
        // (the strips of consecutive steps are disjoint and could run side by side on two streams; measured, two
        // kernels sharing the chip slow each other by what the overlap gains)
        PIPE_TRY(hipStreamWaitEvent(g_rt.stream, up[step], 0));
        Batch one;
        one.stream = g_rt.stream;
        T* d_region = dD + (size_t)r0 * ldd + c0;
        rc = enqueue(dA + (size_t)r0 * lda, dB + c0, hC ? d_region : nullptr, d_region, rows, cols, one);
        if (rc) { cleanup(); return rc; }
        PIPE_TRY(hipEventRecord(done[step], g_rt.stream));
        PIPE_TRY(hipStreamWaitEvent(s_down, done[step], 0));
        PIPE_TRY(hipMemcpy2DAsync(hD + (size_t)r0 * ldd + c0, (size_t)ldd * sizeof(T), d_region, (size_t)ldd * sizeof(T),
                                  (size_t)cols * sizeof(T), rows, hipMemcpyDeviceToHost, s_down));
    }
    PIPE_TRY(hipStreamSynchronize(s_down));            // every download waits for its kernel, every kernel for its uploads
    PIPE_TRY(hipStreamSynchronize(g_rt.stream));
#undef PIPE_TRY
    release_blocks();
    return 0;
}

// Element-wise ReLU family of nn/operators/ReLU.h.  MODE 0: forward; 1: forward + record; 2: backward (dst = src where
// the recorded bit is set, else 0 * src; ReLU.h:131-165).  The bit map has one byte per 8 consecutive floats: bits 4..7
// = the first 16-byte quad's x,y,z,w, bits 0..3 = the second quad's (ReLU.h:86-123).
// One quad per lane, no loop, streaming (non-temporal) accesses: every byte is touched once, consecutive lanes take
// consecutive 16 bytes, and short-lived workgroups keep more loads in flight across the chip than a few long-lived ones
// (measured: 6.7 TB/s against 5.2-5.8 TB/s for grid-stride loops of any unroll depth).  A map byte is assembled from
// the two lanes of a quad pair with one lane exchange; the even lane stores it.
template <int MODE>
__global__ __launch_bounds__(256) void relu_kernel(const f32x4* __restrict__ src, f32x4* __restrict__ dst,
                                                   unsigned char* __restrict__ rec_map, size_t quads) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const bool live = i < quads;              // quads is even in modes 1 and 2, so both lanes of a pair are live together
    f32x4 q = {0.f, 0.f, 0.f, 0.f};
    if (live) q = __builtin_nontemporal_load(src + i);
    unsigned nibble = 0;
    if (MODE == 2 && live) {
        const unsigned byte = rec_map[i >> 1];
        nibble = (i & 1) ? (byte & 15u) : (byte >> 4);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (MODE == 2) {
            q[e] = (float)((nibble >> e) & 1u) * q[e];
        } else {
            const unsigned s = (~__float_as_uint(q[e])) >> 31;
            q[e] = (float)s * q[e];
            nibble |= s << e;
        }
    }
    if (MODE == 1) {
        const unsigned other = (unsigned)__shfl_xor((int)nibble, 1);
        if (live && (i & 1) == 0) rec_map[i >> 1] = (unsigned char)((nibble << 4) | other);
    }
    if (live) __builtin_nontemporal_store(q, dst + i);
}
// the last n % 4 floats of the plain forward form
__global__ void relu_tail_kernel(const float* __restrict__ src, float* __restrict__ dst, int n) {
    const int i = threadIdx.x;
    if (i < n) dst[i] = relu_by_sign(src[i]);
}

template <int MODE>
int relu_enqueue(const float* src, float* dst, unsigned char* rec_map, size_t n) {
    if (!g_rt.is_init) return need_init();
    if (!src || !dst || (MODE != 0 && !rec_map)) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null pointer\n");
    if (!aligned16(src) || !aligned16(dst)) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "ReLU needs 16-byte aligned buffers\n");
    if (MODE != 0 && n % 8 != 0)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "the recorded forms work on whole groups of 8 floats (one map byte each)\n");
    const size_t quads = MODE == 0 ? n / 4 : n / 8 * 2;
    if (quads > 0) {
        const size_t blocks = (quads + 255) / 256;
        if (blocks > 0x7fffffffull) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "buffer too large for one launch\n");
        hipLaunchKernelGGL(relu_kernel<MODE>, dim3((unsigned)blocks), dim3(256), 0, g_rt.stream,
                           reinterpret_cast<const f32x4*>(src), reinterpret_cast<f32x4*>(dst), rec_map, quads);
        HIP_TRY(hipGetLastError());
    }
    if (MODE == 0 && n % 4 != 0) {
        hipLaunchKernelGGL(relu_tail_kernel, dim3(1), dim3(64), 0, g_rt.stream, src + quads * 4, dst + quads * 4, (int)(n % 4));
        HIP_TRY(hipGetLastError());
    }
    return 0;
}

// One lane stores `value` to a word of pinned, host-coherent memory (system scope, release).
__global__ __launch_bounds__(64) void completion_flag_kernel(unsigned* host_flag, unsigned value) {
    if (threadIdx.x == 0) __atomic_store_n(host_flag, value, __ATOMIC_RELEASE);
}

// Waits until the compute work enqueued on the library's stream is complete.  Every call of the reference's API blocks
// (cudaDeviceSynchronize, GEMM.h:122, :450; conv2_mk_im2col.h:268), so this is on the path of every drop-in call, and
// most of them are kernels of tens of microseconds.  Measured on an MI355X around a 60 us kernel: launch +
// hipStreamSynchronize returns 11.4 us after the kernel's own time, polling hipStreamQuery or an event no sooner; a
// one-lane kernel enqueued behind it that stores a sequence number to a word of host-coherent pinned memory, which
// the host polls, 7.9 us.  The stream runs kernels in order, each starting after the one before has completed and
// released its writes, so when the number arrives every kernel enqueued before it is complete.  The host polls for
// a bounded time only (spin_wait_us; a faulting kernel never delivers the number) and then, as for spin_wait_us = 0,
// waits in hipStreamSynchronize.
int wait_compute() {
    if (g_rt.spin_wait_us > 0 && g_rt.done_flag) {
        const unsigned seq = ++g_rt.done_seq;
        hipLaunchKernelGGL(completion_flag_kernel, dim3(1), dim3(64), 0, g_rt.stream, g_rt.done_flag, seq);
        HIP_TRY(hipGetLastError());
        const auto t0 = std::chrono::steady_clock::now();
        for (unsigned polls = 1;; ++polls) {
            if (__atomic_load_n(g_rt.done_flag, __ATOMIC_ACQUIRE) == seq) return 0;
            if ((polls & 255u) == 0 && std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(g_rt.spin_wait_us)) break;
        }
    }
    HIP_TRY(hipStreamSynchronize(g_rt.stream));
    return 0;
}

// copies and fills: the host may read what they wrote the moment the call returns, so these wait in the runtime
int wait_stream() {
    HIP_TRY(hipStreamSynchronize(g_rt.stream));
    return 0;
}

int finish(int rc) {
    if (rc != 0) return rc;
    return wait_compute();
}

}  // namespace

extern "C" {

int decx_hip_init(int* device) {
    if (!g_rt.is_init) {
        int count = 0;
        HIP_TRY(hipGetDeviceCount(&count));
        if (count <= 0) return fail(DECX_HIP_FAIL_NOT_INIT, "no HIP device visible\n");
        int dev = 0;
        HIP_TRY(hipGetDevice(&dev));
        hipDeviceProp_t prop;
        HIP_TRY(hipGetDeviceProperties(&prop, dev));
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return fail(DECX_HIP_FAIL_NOT_INIT, "device %d is %s; this library carries gfx950 code only\n", dev,
                        prop.gcnArchName);
        g_rt.device = dev;
        g_rt.compute_units = prop.multiProcessorCount;
        g_rt.clock_khz = prop.clockRate;
        g_rt.hbm_bytes = prop.totalGlobalMem;
        HIP_TRY(hipStreamCreateWithFlags(&g_rt.stream, hipStreamNonBlocking));
        HIP_TRY(hipEventCreate(&g_rt.ev_start));
        HIP_TRY(hipEventCreate(&g_rt.ev_stop));
        if (const char* gm = getenv("DECX_HIP_GROUP_M")) { int v = atoi(gm); if (v > 0) g_rt.group_m = v; }
        if (const char* sw = getenv("DECX_HIP_SPIN_WAIT_US")) { int v = atoi(sw); if (v >= 0) g_rt.spin_wait_us = v; }
        {
            void* flag = nullptr;                              // the word the completion kernel writes and wait_compute polls
            if (hipHostMalloc(&flag, 64, hipHostMallocCoherent) != hipSuccess) {
                (void)hipGetLastError();
                flag = nullptr;                                // blocking calls then wait in hipStreamSynchronize
            } else {
                *static_cast<unsigned*>(flag) = 0;
            }
            g_rt.done_flag = static_cast<unsigned*>(flag);
            g_rt.done_seq = 0;
        }
        if (int rc = hgemm_static_scratch_init(dev)) return rc;
        // so that the _async fp16 entry points never synchronise the device to grow the workspace
        if (int rc = ensure_partial((size_t)2 * (size_t)(g_rt.compute_units > 0 ? g_rt.compute_units : 256) * 128 * 128 * sizeof(float))) return rc;
        g_rt.is_init = true;
    }
    if (device) *device = g_rt.device;
    return 0;
}

int decx_hip_is_init(void) { return g_rt.is_init ? 1 : 0; }

int decx_hip_device_info(int* compute_units, int* clock_khz, size_t* hbm_bytes) {
    if (!g_rt.is_init) return need_init();
    if (compute_units) *compute_units = g_rt.compute_units;
    if (clock_khz) *clock_khz = g_rt.clock_khz;
    if (hbm_bytes) *hbm_bytes = g_rt.hbm_bytes;
    return 0;
}

int decx_hip_malloc(void** dptr, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    if (!dptr) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null output pointer\n");
    *dptr = nullptr;
    if (hipMalloc(dptr, bytes ? bytes : 1) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");   // core/error.h:65
    }
    return 0;
}

int decx_hip_free(void* dptr) {
    if (!dptr) return 0;
    HIP_TRY(hipFree(dptr));
    return 0;
}

int decx_hip_memset(void* dptr, int value, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipMemsetAsync(dptr, value, bytes, g_rt.stream));
    return wait_stream();
}

int decx_hip_host_malloc(void** hptr, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    if (!hptr) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null output pointer\n");
    *hptr = nullptr;
    if (hipHostMalloc(hptr, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess) {
        (void)hipGetLastError();
        return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    }
    return 0;
}

int decx_hip_host_free(void* hptr) {
    if (!hptr) return 0;
    HIP_TRY(hipHostFree(hptr));
    return 0;
}

static hipMemcpyKind copy_kind(int direction) {
    switch (direction) {
        case DECX_HIP_H2D: return hipMemcpyHostToDevice;
        case DECX_HIP_D2H: return hipMemcpyDeviceToHost;
        default: return hipMemcpyDeviceToDevice;
    }
}

int decx_hip_memcpy2d(void* dst, size_t dst_pitch_bytes, const void* src, size_t src_pitch_bytes, size_t width_bytes,
                      size_t rows, int direction) {
    if (!g_rt.is_init) return need_init();
    if (direction < DECX_HIP_H2D || direction > DECX_HIP_D2D) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "bad copy direction\n");
    if (width_bytes == 0 || rows == 0) return 0;
    if (dst_pitch_bytes < width_bytes || src_pitch_bytes < width_bytes)
        return fail(DECX_HIP_FAIL_ERROR_PARAMS, "pitch smaller than the row width\n");
    HIP_TRY(hipMemcpy2DAsync(dst, dst_pitch_bytes, src, src_pitch_bytes, width_bytes, rows, copy_kind(direction),
                             g_rt.stream));
    return wait_stream();
}

int decx_hip_memcpy(void* dst, const void* src, size_t bytes, int direction) {
    if (!g_rt.is_init) return need_init();
    if (direction < DECX_HIP_H2D || direction > DECX_HIP_D2D) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "bad copy direction\n");
    if (bytes == 0) return 0;
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, copy_kind(direction), g_rt.stream));
    return wait_stream();
}

int decx_hip_sync(void) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipDeviceSynchronize());
    return 0;
}

int decx_hip_sgemm_async(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd,
                         int M, int N, int K) {
    return sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream());
}
int decx_hip_sgemm(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                   int N, int K) {
    return finish(sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream()));
}
int decx_hip_sgemm_relu(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                        int N, int K) {
    return finish(sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream(), true));
}
int decx_hip_sgemm_splitk(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                          int N, int K, int splits) {
    return finish(sgemm_splitk_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, splits));
}
int decx_hip_sgemm_batched(const float* A, int lda, size_t stride_a, const float* B, int ldb, size_t stride_b,
                           const float* Cin, int ldc, size_t stride_c, float* D, int ldd, size_t stride_d, int M, int N, int K,
                           int batch) {
    return finish(sgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K,
                                batch_on_library_stream(batch, stride_a, stride_b, stride_c, stride_d)));
}

int decx_hip_hgemm_f32acc_async(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                uint16_t* D, int ldd, int M, int N, int K) {
    return hgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream());
}
int decx_hip_hgemm_f32acc(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                          int ldd, int M, int N, int K) {
    return finish(hgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, single_on_library_stream()));
}
int decx_hip_hgemm_f32acc_noalloc(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                  uint16_t* D, int ldd, int M, int N, int K, int splits) {
    return finish(hgemm_splitk_static_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K, splits));
}
int decx_hip_hgemm_f32acc_batched(const uint16_t* A, int lda, size_t stride_a, const uint16_t* B, int ldb, size_t stride_b,
                                  const uint16_t* Cin, int ldc, size_t stride_c, uint16_t* D, int ldd, size_t stride_d, int M,
                                  int N, int K, int batch) {
    return finish(hgemm_enqueue(A, lda, B, ldb, Cin, ldc, D, ldd, M, N, K,
                                batch_on_library_stream(batch, stride_a, stride_b, stride_c, stride_d)));
}

int decx_hip_gemm3_host_f32(const float* hA, int lda, size_t plane_a, const float* hB, int ldb, size_t plane_b,
                            const float* hC, int ldc, size_t plane_c, float* hD, int ldd, size_t plane_d, int M, int N, int K,
                            int count) {
    return gemm3_host_pipeline<float>(hA, lda, plane_a, hB, ldb, plane_b, hC, ldc, plane_c, hD, ldd, plane_d, M, N, K, count,
                                      [&](const float* a, const float* b, const float* c, float* d, const Batch& one) {
                                          return sgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, M, N, K, one);
                                      });
}
int decx_hip_gemm3_host_f16(const uint16_t* hA, int lda, size_t plane_a, const uint16_t* hB, int ldb, size_t plane_b,
                            const uint16_t* hC, int ldc, size_t plane_c, uint16_t* hD, int ldd, size_t plane_d, int M, int N,
                            int K, int count) {
    return gemm3_host_pipeline<uint16_t>(hA, lda, plane_a, hB, ldb, plane_b, hC, ldc, plane_c, hD, ldd, plane_d, M, N, K, count,
                                         [&](const uint16_t* a, const uint16_t* b, const uint16_t* c, uint16_t* d, const Batch& one) {
                                             return hgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, M, N, K, one);
                                         });
}

int decx_hip_gemm_host_f32(const float* hA, int lda, const float* hB, int ldb, const float* hC, int ldc, float* hD, int ldd,
                           int M, int N, int K) {
    return gemm_host_pipeline<float>(hA, lda, hB, ldb, hC, ldc, hD, ldd, M, N, K,
                                     [&](const float* a, const float* b, const float* c, float* d, int rows, int cols, const Batch& one) {
                                         return sgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, rows, cols, K, one);
                                     });
}
int decx_hip_gemm_host_f16(const uint16_t* hA, int lda, const uint16_t* hB, int ldb, const uint16_t* hC, int ldc, uint16_t* hD,
                           int ldd, int M, int N, int K) {
    return gemm_host_pipeline<uint16_t>(hA, lda, hB, ldb, hC, ldc, hD, ldd, M, N, K,
                                        [&](const uint16_t* a, const uint16_t* b, const uint16_t* c, uint16_t* d, int rows, int cols, const Batch& one) {
                                            return hgemm_enqueue(a, lda, b, ldb, c, ldd, d, ldd, rows, cols, K, one);
                                        });
}

int decx_hip_conv2_im2col_f32_async(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag) {
    return conv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst, dst_dpitch,
                        dst_row_stride, flag);
}
int decx_hip_conv2_im2col_f32(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt, int N,
                              int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst, int dst_dpitch,
                              size_t dst_row_stride, int flag) {
    return finish(conv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst,
                               dst_dpitch, dst_row_stride, flag));
}

int decx_hip_conv2_im2col_f32_fused(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag, const float* bias, int relu) {
    return finish(conv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst,
                               dst_dpitch, dst_row_stride, flag, bias, relu != 0));
}

int decx_hip_conv2_im2col_f16_async(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag, const uint16_t* bias, int relu) {
    return hconv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst, dst_dpitch,
                         dst_row_stride, flag, bias, relu != 0);
}
int decx_hip_conv2_im2col_f16(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt, int N,
                              int kh, int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst, int dst_dpitch,
                              size_t dst_row_stride, int flag, const uint16_t* bias, int relu) {
    return finish(hconv_enqueue(src, H, W, dpitch, src_row_stride, filt, N, kh, kw, filt_stride, filt_row_stride, dst,
                                dst_dpitch, dst_row_stride, flag, bias, relu != 0));
}

int decx_hip_relu_f32(const float* src, float* dst, size_t n) { return finish(relu_enqueue<0>(src, dst, nullptr, n)); }
int decx_hip_relu_f32_async(const float* src, float* dst, size_t n) { return relu_enqueue<0>(src, dst, nullptr, n); }
int decx_hip_relu_f32_rec(const float* src, float* dst, unsigned char* rec_map, size_t n) {
    return finish(relu_enqueue<1>(src, dst, rec_map, n));
}
int decx_hip_relu_f32_backward(const float* src, float* dst, const unsigned char* rec_map, size_t n) {
    return finish(relu_enqueue<2>(src, dst, const_cast<unsigned char*>(rec_map), n));
}

int decx_hip_tmp_malloc(void** dptr, size_t bytes) {
    if (!g_rt.is_init) return need_init();
    if (!dptr || bytes == 0) return fail(DECX_HIP_FAIL_ERROR_PARAMS, "null pointer or empty block\n");
    *dptr = tmp_acquire(bytes);
    if (!*dptr) return fail(DECX_HIP_FAIL_ALLOCATION, "Fail to allocate memory\n");
    return 0;
}

int decx_hip_tmp_free(void* dptr) {
    if (!dptr) return 0;
    for (int i = 0; i < g_tmp_count; ++i)
        if (g_tmp[i].ptr == dptr && g_tmp[i].in_use) {
            g_tmp[i].in_use = false;
            return 0;
        }
    return fail(DECX_HIP_FAIL_ERROR_PARAMS, "not a block of decx_hip_tmp_malloc in use\n");
}

int decx_hip_release_tmp(void) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipDeviceSynchronize());
    return free_idle_tmp_blocks();
}

void* decx_hip_stream(void) { return g_rt.is_init ? static_cast<void*>(g_rt.stream) : nullptr; }

int decx_hip_timer_start(void) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipEventRecord(g_rt.ev_start, g_rt.stream));
    return 0;
}

int decx_hip_timer_stop(float* milliseconds) {
    if (!g_rt.is_init) return need_init();
    HIP_TRY(hipEventRecord(g_rt.ev_stop, g_rt.stream));
    HIP_TRY(hipEventSynchronize(g_rt.ev_stop));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, g_rt.ev_start, g_rt.ev_stop));
    if (milliseconds) *milliseconds = ms;
    return 0;
}

const char* decx_hip_last_error(void) { return g_err; }

int decx_hip_set_sgemm_variant(int variant) {
    int prev = g_rt.sgemm_variant;
    g_rt.sgemm_variant = variant;
    return prev;
}
int decx_hip_set_hgemm_variant(int variant) {
    int prev = g_rt.hgemm_variant;
    g_rt.hgemm_variant = variant;
    return prev;
}

int decx_hip_set_splitk_mode(int mode) {
    int prev = g_rt.splitk_atomic;
    g_rt.splitk_atomic = mode ? 1 : 0;
    return prev;
}

int decx_hip_sgemm_plan(int M, int N, int K, int batch, long lda, long ldb, int aligned) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || lda < K || ldb < N) return -1;
    return sgemm_plan(M, N, K, batch, lda, ldb, aligned != 0);
}

int decx_hip_sgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, int aligned, int* shape, int* by_columns) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || lda < K || ldb < N) return -1;
    return sgemm_plan_split(M, N, K, batch, lda, ldb, aligned != 0, shape, by_columns);
}

int decx_hip_conv_plan_split(int H, int W, int dpitch, int N, int kh, int kw, int flag, int* shape) {
    if (H <= 0 || W <= 0 || dpitch <= 0 || N <= 0 || kh <= 0 || kw <= 0) return -1;
    const int Hout = flag ? H : H - 2 * (kh / 2), Wout = flag ? W : W - 2 * (kw / 2);
    const long K = (long)kh * kw * dpitch;
    if (Hout <= 0 || Wout <= 0 || K > 0x7fffffffL) return -1;
    return conv_plan_split(Hout, Wout, N, (int)K, shape);
}

int decx_hip_hgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, int aligned, int* by_columns) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || lda < K || ldb < N) return -1;
    return hgemm_plan_split(M, N, K, batch, lda, ldb, aligned != 0, by_columns);
}

int decx_hip_hgemm_plan(int M, int N, int K, int batch, long lda, long ldb, int aligned, int* splits) {
    if (M <= 0 || N <= 0 || K <= 0 || batch <= 0 || lda < K || ldb < N) return -1;
    return hgemm_plan(M, N, K, batch, lda, ldb, aligned != 0, splits);
}

int decx_hip_conv_patch_offsets_fit(int H, int W, int dpitch, size_t src_row_stride, int kh, int kw, int flag, int elem_bytes) {
    if (H <= 0 || W <= 0 || dpitch <= 0 || kh <= 0 || kw <= 0 || (elem_bytes != 2 && elem_bytes != 4) || src_row_stride < (size_t)W * dpitch) return -1;
    const size_t src_bytes = ((size_t)(H - 1) * src_row_stride + (size_t)W * dpitch) * elem_bytes;
    if (src_bytes >= 0x80000000ull) return 0;
    return conv_patch_offsets_fit(src_bytes, src_row_stride, (size_t)dpitch, kh, kw, flag ? kh / 2 : 0, flag ? kw / 2 : 0, (size_t)elem_bytes) ? 1 : 0;
}

int decx_hip_b_read_extent(int N, int tile_n, int unit) {
    if (N <= 0 || tile_n <= 0 || unit <= 0 || tile_n % unit) return -1;
    int last = -1;
    for (int bn0 = 0; bn0 < N; bn0 += tile_n)                    // every tile column of the launch
        for (int g = 0; g < tile_n; g += unit) {                 // every column group a tile stages
            const int col = clamp_group_col(bn0 + g, N, unit) + unit - 1;
            if (col > last) last = col;
        }
    return last;
}

}  // extern "C"
