// TEST INFRASTRUCTURE ONLY.  CPU restatement of the arithmetic of DECX's dense-contraction path.
// Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this library; the
// product (backup_1_amd/) never links, imports or calls it.
//
// What the reference computes (citations relative to the reference tree):
//   * every fp32 GEMM path keeps ONE fp32 accumulator per output element and updates it with a fused
//     multiply-add over ascending k:
//       srcs/GEMM/CUDA/GEMM_kernel_def.cuh:33-55   (sfma_8x8: fmaf per element, k ascending inside GEMM.cuh:83-92)
//       srcs/GEMM/CPU/sgemm_calc_kernel.h:24-29    (_mm256_fmadd_ps per (row,k), C stored/reloaded per 64-k block)
//       srcs/convolution/CUDA/im2col/eq_GEMM.cuh:65-74, :172-193 (fmaf, k ascending)
//     `dst = A*B + C` pre-loads the accumulator from C (GEMM.cuh:223).
//   * the im2col convolution orders k as (ki*kw + kj)*dpitch + c  (srcs/convolution/CUDA/im2col/im2col.cuh:153),
//     is a cross-correlation (no filter flip, im2col.cuh:150-163), stride 1, and in the "zero compensate" mode
//     reads 0 outside the image (conv2_mk_im2col.h:167-274); output row m = y*wpitch_out + x lands at
//     dst[m*dpitch_out + n] (conv2_mk_im2col.h:185-189, :266).
//   * fp16 storage is IEEE binary16 produced by round-to-nearest-even (float_half_convert.h:32-43 uses __float2half).
//
// Pinning status (what proves each function right, see tests/test_oracle.py):
//   oracle_sgemm_chain        : reference-held known answer (test/test/CUDA_GEMM/CUDA_GEMM.cpp:24-42, 0.1*index
//                               pattern, closed form), exact small-integer products vs int64 arithmetic,
//                               permutation/identity B, A=0 => dst=C, tiny brute force in exact rational arithmetic
//                               of the fused chain (python fractions + single rounding per step).
//   oracle_sgemm_chain_fast   : bit-identical to oracle_sgemm_chain on random ragged shapes.
//   oracle_decx_cpu_sgemm     : bit-identical to oracle_sgemm_chain on shapes hitting every variant
//                               (N%16 in {0,8}, M%32, K%64, panel count %4).
//   oracle_conv2_chain        : all-ones closed form (tap counts), impulse response = reversed filter slices,
//                               fp64 7-loop brute force on tiny shapes, integer-exact vs int64.
//   oracle_gemm_f64_rows_f16  : integer-exact vs int64, numpy float64 matmul on random data.
//   oracle_conv2_f64_f16      : fp64 arithmetic on binary16 tensors, the yardstick of the fp16 convolution (the reference has
//                               none to restate; indexing as oracle_conv2_chain): numpy float16 -> float64 conversion
//                               plus a 7-loop brute force, all-ones tap counts, impulse response, equality with
//                               oracle_conv2_chain on integer data, padded strides.
//   oracle_float_to_half/back : numpy float16 casts (independent RNE implementation), IEEE known values.
//   oracle_relu_f32[_rec|_backward] : restate srcs/nn/operators/ReLU.h:57-165 (value times float(sign bit clear); one
//                               map byte per 8 floats).  The reference holds no test vectors for them; pinned by
//                               numpy max(x,0) on finite data, the IEEE special cases the multiplication implies
//                               (-x -> -0.0, -inf -> NaN, +inf kept), map bits against numpy's signbit/packbits, and
//                               backward(rec(x)) identities.
//
// Build: make -C oracle   (g++ -O2 -mavx2 -mfma, see oracle/Makefile)

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <condition_variable>
#include <functional>
#include <future>
#include <mutex>
#include <thread>
#include <vector>
#include <immintrin.h>

namespace {

// ---------------------------------------------------------------------------------------------------------------
// small helpers
// ---------------------------------------------------------------------------------------------------------------
int host_threads(int requested) {
    int hw = (int)std::thread::hardware_concurrency();
    if (hw <= 0) hw = 1;
    if (requested > 0) return requested;
    return hw;
}

template <class F>
void parallel_ranges(int nthreads, long total, F&& body) {
    nthreads = host_threads(nthreads);
    if (nthreads > total) nthreads = (int)(total > 0 ? total : 1);
    if (nthreads <= 1) { body(0L, total); return; }
    std::vector<std::thread> th;
    long per = (total + nthreads - 1) / nthreads;
    for (int t = 0; t < nthreads; ++t) {
        long lo = t * per, hi = lo + per;
        if (hi > total) hi = total;
        if (lo >= hi) break;
        th.emplace_back([=, &body] { body(lo, hi); });
    }
    for (auto& x : th) x.join();
}

// acc[0..n) = fma(a, b[0..n), acc[0..n)) with one rounding per element (AVX2 FMA lanes are IEEE fused ops,
// identical to std::fmaf per lane).
inline void row_fma(float a, const float* b, float* acc, int n) {
    __m256 va = _mm256_set1_ps(a);
    int j = 0;
    for (; j + 8 <= n; j += 8)
        _mm256_storeu_ps(acc + j, _mm256_fmadd_ps(va, _mm256_loadu_ps(b + j), _mm256_loadu_ps(acc + j)));
    for (; j < n; ++j) acc[j] = std::fmaf(a, b[j], acc[j]);
}

// ---------------------------------------------------------------------------------------------------------------
// thread pool restated from srcs/core/thread_management/thread_pool.h:30-247 and task_queue.h:23-92:
// one LIFO queue of std::packaged_task<void()> per worker, register_task() picks the first idle queue (else the
// shortest one) and returns a std::future<void>.  Differences on purpose: the worker arrays are sized to the
// worker count (the reference placement-news hardware_concurrency() workers into arrays of 16,
// thread_pool.h:18,131-136) and the queue length is read under its lock.
// ---------------------------------------------------------------------------------------------------------------
class TaskQueuePool {
    struct Worker {
        std::mutex mtx;
        std::condition_variable cv;
        std::vector<std::packaged_task<void()>> tasks;   // executed back-to-front (LIFO), as task_queue.h does
        bool shutdown = false;
        std::thread thr;
    };
    std::vector<Worker*> workers_;

    void main_loop(Worker* w) {
        for (;;) {
            std::packaged_task<void()> task;
            {
                std::unique_lock<std::mutex> lock(w->mtx);
                w->cv.wait(lock, [&] { return !w->tasks.empty() || w->shutdown; });
                if (w->tasks.empty()) return;
                task = std::move(w->tasks.back());
                w->tasks.pop_back();
            }
            task();
        }
    }

    size_t pick_queue() {
        size_t best = 0, best_len = ~size_t(0);
        for (size_t i = 0; i < workers_.size(); ++i) {
            std::lock_guard<std::mutex> g(workers_[i]->mtx);
            size_t len = workers_[i]->tasks.size();
            if (len == 0) return i;
            if (len < best_len) { best_len = len; best = i; }
        }
        return best;
    }

public:
    explicit TaskQueuePool(int n) {
        if (n < 1) n = 1;
        for (int i = 0; i < n; ++i) {
            Worker* w = new Worker();
            workers_.push_back(w);
            w->thr = std::thread(&TaskQueuePool::main_loop, this, w);
        }
    }
    ~TaskQueuePool() {
        for (Worker* w : workers_) {
            { std::lock_guard<std::mutex> g(w->mtx); w->shutdown = true; }
            w->cv.notify_one();
            w->thr.join();
            delete w;
        }
    }
    size_t size() const { return workers_.size(); }

    template <class F, class... Args>
    std::future<void> register_task(F&& f, Args&&... args) {
        std::packaged_task<void()> task(std::bind(std::forward<F>(f), std::forward<Args>(args)...));
        std::future<void> fut = task.get_future();
        Worker* w = workers_[pick_queue()];
        { std::lock_guard<std::mutex> g(w->mtx); w->tasks.emplace_back(std::move(task)); }
        w->cv.notify_one();
        return fut;
    }
};

TaskQueuePool& global_pool(int nthreads) {
    // reference: decx::thread_pool(hardware_concurrency(), true), arrays of MAX_THREAD_NUM 16 (thread_pool.h:18,244-247)
    static std::mutex m;
    static TaskQueuePool* pool = nullptr;
    static int pool_n = 0;
    std::lock_guard<std::mutex> g(m);
    int want = nthreads > 0 ? nthreads : (int)std::thread::hardware_concurrency();
    if (want < 1) want = 1;
    if (want > 16) want = 16;
    if (!pool || pool_n != want) { delete pool; pool = new TaskQueuePool(want); pool_n = want; }
    return *pool;
}

// ---------------------------------------------------------------------------------------------------------------
// DECX_cpu SGEMM restated: B panel re-pack + 32x16x64 micro-kernel + 3x4 task grid.
// ---------------------------------------------------------------------------------------------------------------
constexpr int BL_K = 64;   // sgemm_BL_Linear   sgemm_calc_kernel.h:15
constexpr int BL_M = 32;   // sgemm_BL_hA       :16
constexpr int BL_N = 16;   // sgemm_BL_wB       :17

// Re-pack columns [16p, 16p+w) of B (K x ldb) into a contiguous K x w panel, w = 16 or 8
// (sort_MatB_16 / sort_MatB_16_w8, gemm_utils.h:59-166).
void pack_panels(const float* B, long ldb, int K, int first_panel, int last_panel, int npanels, int n8,
                 float* packed) {
    for (int p = first_panel; p < last_panel; ++p) {
        int w = (p == npanels - 1 && (n8 % 16) == 8) ? 8 : 16;
        float* dst = packed + (size_t)p * 16 * K;
        const float* src = B + (size_t)p * 16;
        for (int k = 0; k < K; ++k) {
            _mm256_storeu_ps(dst, _mm256_loadu_ps(src));
            if (w == 16) _mm256_storeu_ps(dst + 8, _mm256_loadu_ps(src + 8));
            dst += w;
            src += ldb;
        }
    }
}

// One (rows x 16 | 8) x kb block update: C (+)= A_blk * B_panel.  `first` zero-initialises the accumulators
// (_avx256_sgemm_block_first, sgemm_calc_kernel.h:190-245 family); otherwise C is reloaded, exactly one fp32
// accumulator per element.  rows <= 32 covers the flexibleH variants, kb <= 64 the Lleft variants, w == 8 the w8 ones.
void micro_block(const float* A, long lda, const float* Bp, float* C, long ldc, int rows, int kb, int w, bool first) {
    if (w == 16) {
        for (int i = 0; i < rows; ++i) {
            const float* a = A + (size_t)i * lda;
            float* c = C + (size_t)i * ldc;
            __m256 c0 = first ? _mm256_setzero_ps() : _mm256_loadu_ps(c);
            __m256 c1 = first ? _mm256_setzero_ps() : _mm256_loadu_ps(c + 8);
            const float* b = Bp;
            for (int k = 0; k < kb; ++k) {
                __m256 va = _mm256_set1_ps(a[k]);
                c0 = _mm256_fmadd_ps(va, _mm256_loadu_ps(b), c0);
                c1 = _mm256_fmadd_ps(va, _mm256_loadu_ps(b + 8), c1);
                b += 16;
            }
            _mm256_storeu_ps(c, c0);
            _mm256_storeu_ps(c + 8, c1);
        }
    } else {
        for (int i = 0; i < rows; ++i) {
            const float* a = A + (size_t)i * lda;
            float* c = C + (size_t)i * ldc;
            __m256 c0 = first ? _mm256_setzero_ps() : _mm256_loadu_ps(c);
            const float* b = Bp;
            for (int k = 0; k < kb; ++k) {
                c0 = _mm256_fmadd_ps(_mm256_set1_ps(a[k]), _mm256_loadu_ps(b), c0);
                b += 8;
            }
            _mm256_storeu_ps(c, c0);
        }
    }
}

// One task of the 3x4 grid (_ST_sgemm_Dblock_*, sgemm_callers.h:219-636): row-block 32 -> column panel -> k-block 64.
void task_block(const float* A, long lda, const float* packed, float* C, long ldc, int row0, int row1, int pan0,
                int pan1, int npanels, int n8, int K) {
    for (int r = row0; r < row1; r += BL_M) {
        int rows = row1 - r < BL_M ? row1 - r : BL_M;
        for (int p = pan0; p < pan1; ++p) {
            int w = (p == npanels - 1 && (n8 % 16) == 8) ? 8 : 16;
            const float* Bp = packed + (size_t)p * 16 * K;
            for (int k0 = 0; k0 < K; k0 += BL_K) {
                int kb = K - k0 < BL_K ? K - k0 : BL_K;
                micro_block(A + (size_t)r * lda + k0, lda, Bp + (size_t)k0 * w, C + (size_t)r * ldc + (size_t)p * 16,
                            ldc, rows, kb, w, k0 == 0);
            }
        }
    }
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------------------------------------------------------
// Definitional chain: D[i][j] = fmaf-chain over k ascending, acc0 = 0 or Cin[i][j].  Scalar, single-threaded.
// ---------------------------------------------------------------------------------------------------------------
void oracle_sgemm_chain(const float* A, long lda, const float* B, long ldb, const float* Cin, long ldc, float* D,
                        long ldd, int M, int N, int K) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = Cin ? Cin[(size_t)i * ldc + j] : 0.0f;
            for (int k = 0; k < K; ++k) acc = std::fmaf(A[(size_t)i * lda + k], B[(size_t)k * ldb + j], acc);
            D[(size_t)i * ldd + j] = acc;
        }
}

// Same values, vectorised over j and threaded over i (each element still sees k = 0..K-1 in order, one fused
// rounding per step).  Used where the scalar loop would take minutes (4096^3, 8192^3 row samples).
void oracle_sgemm_chain_fast(const float* A, long lda, const float* B, long ldb, const float* Cin, long ldc, float* D,
                             long ldd, int M, int N, int K, int nthreads) {
    constexpr int JB = 1024;   // accumulator strip kept in L1
    parallel_ranges(nthreads, M, [&](long lo, long hi) {
        std::vector<float> acc(JB);
        for (long i = lo; i < hi; ++i)
            for (int j0 = 0; j0 < N; j0 += JB) {
                int n = N - j0 < JB ? N - j0 : JB;
                if (Cin) std::memcpy(acc.data(), Cin + (size_t)i * ldc + j0, sizeof(float) * n);
                else std::memset(acc.data(), 0, sizeof(float) * n);
                const float* a = A + (size_t)i * lda;
                for (int k = 0; k < K; ++k) row_fma(a[k], B + (size_t)k * ldb + j0, acc.data(), n);
                std::memcpy(D + (size_t)i * ldd + j0, acc.data(), sizeof(float) * n);
            }
    });
}

// Chain for a list of rows only: out is nrows x N (dense).  For spot checks at 8192^3.
void oracle_sgemm_chain_rows(const float* A, long lda, const float* B, long ldb, const int* rows, int nrows, float* out,
                             int N, int K, int nthreads) {
    parallel_ranges(nthreads, nrows, [&](long lo, long hi) {
        for (long r = lo; r < hi; ++r) {
            float* acc = out + (size_t)r * N;
            std::memset(acc, 0, sizeof(float) * N);
            const float* a = A + (size_t)rows[r] * lda;
            for (int j0 = 0; j0 < N; j0 += 1024) {
                int n = N - j0 < 1024 ? N - j0 : 1024;
                for (int k = 0; k < K; ++k) row_fma(a[k], B + (size_t)k * ldb + j0, acc + j0, n);
            }
        }
    });
}

// ---------------------------------------------------------------------------------------------------------------
// DECX_cpu thread-pool SGEMM (de::cpu::sgemm -> decx::sgemm_caller<3,4>, sgemm.h:28-60, sgemm_callers.h:1227-1249).
// A: M x K (pitch lda), B: K x N (pitch ldb), D: M x N (pitch ldd).  Like the reference the columns are processed
// in units of 8 up to ceil8(N) (a _Matrix pitch is a multiple of 8, Matrix.h:24-27,:260), so ldb and ldd must be
// >= ceil8(N); values in D's pitch padding are written.  Departures from the reference, all defect fixes:
// the three row groups are multiples of 32 rows (sgemm_callers.h:1120 uses M/3, which overlaps and overruns);
// K need not be a multiple of 8; dst is M x N rather than (K, K) (sgemm.h:40).
// Returns 0, or -1 for bad arguments.
// ---------------------------------------------------------------------------------------------------------------
int oracle_decx_cpu_sgemm(const float* A, long lda, const float* B, long ldb, float* D, long ldd, int M, int N, int K,
                          int nthreads) {
    if (M <= 0 || N <= 0 || K <= 0) return -1;
    int n8 = (N + 7) / 8 * 8;
    if (ldb < n8 || ldd < n8 || lda < K) return -1;
    int npanels = (n8 + 15) / 16;
    TaskQueuePool& pool = global_pool(nthreads);

    float* packed = (float*)std::aligned_alloc(64, ((size_t)npanels * 16 * K * sizeof(float) + 63) / 64 * 64);
    if (!packed) return -1;

    // B re-pack on 12 tasks (sort_MatB_16<12>, gemm_utils.h:107-134): panels split evenly, remainder to the last.
    {
        constexpr int T = 12;
        std::vector<std::future<void>> fut;
        int per = npanels / T;
        for (int t = 0; t < T; ++t) {
            int p0 = t * per, p1 = (t == T - 1) ? npanels : p0 + per;
            if (p0 >= p1) continue;
            fut.emplace_back(pool.register_task(pack_panels, B, ldb, K, p0, p1, npanels, n8, packed));
        }
        for (auto& f : fut) f.get();
    }

    // 3 x 4 task grid (sgemm_caller<3,4>): rows in 3 groups of whole 32-row blocks, panels in 4 groups.
    {
        constexpr int TR = 3, TC = 4;
        int rblocks = (M + BL_M - 1) / BL_M;
        std::vector<std::future<void>> fut;
        for (int tr = 0; tr < TR; ++tr) {
            int rb0 = (int)((long)rblocks * tr / TR), rb1 = (int)((long)rblocks * (tr + 1) / TR);
            int row0 = rb0 * BL_M, row1 = rb1 * BL_M < M ? rb1 * BL_M : M;
            if (row0 >= row1) continue;
            for (int tc = 0; tc < TC; ++tc) {
                int p0 = (int)((long)npanels * tc / TC), p1 = (int)((long)npanels * (tc + 1) / TC);
                if (p0 >= p1) continue;
                fut.emplace_back(
                    pool.register_task(task_block, A, lda, packed, D, ldd, row0, row1, p0, p1, npanels, n8, K));
            }
        }
        for (auto& f : fut) f.get();
    }
    std::free(packed);
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Convolution, chain order k = (ki*kw + kj)*dpitch + c  (im2col.cuh:153), computed as "one im2col row at a time,
// then the same chain".  src: H rows, row stride src_row_stride floats, pixel stride dpitch floats (Tensor.h:389-394).
// filt: N filters, filter n at filt + n*filt_stride, tap (ki,kj) at ki*filt_row_stride + kj*dpitch (TensorArray.h:521-525).
// dst(y,x,n) at dst[y*dst_row_stride + x*dst_dpitch + n].
// flag 1: same size, zero outside the image; flag 0: valid region only, out = (H-2*(kh/2)) x (W-2*(kw/2))
// (conv2_mk_im2col.h:63-66, :173-176).  Columns x >= W_out of dst rows are not written.
// Returns 0, -1 bad flag / sizes.
// ---------------------------------------------------------------------------------------------------------------
int oracle_conv2_chain(const float* src, int H, int W, int dpitch, long src_row_stride, const float* filt, int N, int kh,
                       int kw, long filt_stride, long filt_row_stride, float* dst, int dst_dpitch, long dst_row_stride,
                       int flag, int nthreads) {
    if (flag != 0 && flag != 1) return -1;
    int Hout = flag ? H : H - 2 * (kh / 2), Wout = flag ? W : W - 2 * (kw / 2);
    if (Hout <= 0 || Wout <= 0 || N <= 0 || dpitch <= 0) return -1;
    int oy = flag ? kh / 2 : 0, ox = flag ? kw / 2 : 0;
    int K = kh * kw * dpitch;
    // filters transposed once to [k][n] so that the chain vectorises over n
    std::vector<float> Wt((size_t)K * N);
    for (int n = 0; n < N; ++n)
        for (int ki = 0; ki < kh; ++ki)
            for (int kj = 0; kj < kw; ++kj)
                for (int c = 0; c < dpitch; ++c)
                    Wt[(size_t)((ki * kw + kj) * dpitch + c) * N + n] =
                        filt[(size_t)n * filt_stride + (size_t)ki * filt_row_stride + (size_t)kj * dpitch + c];
    parallel_ranges(nthreads, Hout, [&](long lo, long hi) {
        std::vector<float> patch(K), acc(N);
        for (long y = lo; y < hi; ++y)
            for (int x = 0; x < Wout; ++x) {
                for (int ki = 0; ki < kh; ++ki)
                    for (int kj = 0; kj < kw; ++kj) {
                        long sy = y + ki - oy, sx = x + kj - ox;
                        float* p = patch.data() + (size_t)(ki * kw + kj) * dpitch;
                        if (sy < 0 || sy >= H || sx < 0 || sx >= W) std::memset(p, 0, sizeof(float) * dpitch);
                        else std::memcpy(p, src + (size_t)sy * src_row_stride + (size_t)sx * dpitch, sizeof(float) * dpitch);
                    }
                std::memset(acc.data(), 0, sizeof(float) * N);
                for (int k = 0; k < K; ++k) row_fma(patch[k], Wt.data() + (size_t)k * N, acc.data(), N);
                std::memcpy(dst + (size_t)y * dst_row_stride + (size_t)x * dst_dpitch, acc.data(), sizeof(float) * N);
            }
    });
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// Convolution of binary16 tensors in fp64: what the fp16 convolution (fp32 accumulate) is checked against, as the fp16
// GEMM is against oracle_gemm_f64_rows_f16.  Same index arithmetic as oracle_conv2_chain (k = (ki*kw + kj)*dpitch + c,
// cross-correlation, im2col.cuh:150-163; flag as conv2_mk_im2col.h:63-66, :173-176); all strides in halves.
// out[(y*W_out + x)*N + n] = sum of products, scale[...] = sum of |products| (the denominator of the relative error).
// The reference has no binary16 im2col convolution, so there is no reference arithmetic to restate beyond the indexing.
// ---------------------------------------------------------------------------------------------------------------
static inline float h2f(uint16_t h);      // defined with the conversions below
int oracle_conv2_f64_f16(const uint16_t* src, int H, int W, int dpitch, long src_row_stride, const uint16_t* filt, int N,
                         int kh, int kw, long filt_stride, long filt_row_stride, double* out, double* scale, int flag,
                         int nthreads) {
    if (flag != 0 && flag != 1) return -1;
    int Hout = flag ? H : H - 2 * (kh / 2), Wout = flag ? W : W - 2 * (kw / 2);
    if (Hout <= 0 || Wout <= 0 || N <= 0 || dpitch <= 0) return -1;
    int oy = flag ? kh / 2 : 0, ox = flag ? kw / 2 : 0;
    int K = kh * kw * dpitch;
    std::vector<double> Wt((size_t)K * N);
    for (int n = 0; n < N; ++n)
        for (int ki = 0; ki < kh; ++ki)
            for (int kj = 0; kj < kw; ++kj)
                for (int c = 0; c < dpitch; ++c)
                    Wt[(size_t)((ki * kw + kj) * dpitch + c) * N + n] =
                        (double)h2f(filt[(size_t)n * filt_stride + (size_t)ki * filt_row_stride + (size_t)kj * dpitch + c]);
    parallel_ranges(nthreads, Hout, [&](long lo, long hi) {
        std::vector<double> patch(K);
        for (long y = lo; y < hi; ++y)
            for (int x = 0; x < Wout; ++x) {
                for (int ki = 0; ki < kh; ++ki)
                    for (int kj = 0; kj < kw; ++kj) {
                        long sy = y + ki - oy, sx = x + kj - ox;
                        double* p = patch.data() + (size_t)(ki * kw + kj) * dpitch;
                        const bool inside = sy >= 0 && sy < H && sx >= 0 && sx < W;
                        for (int c = 0; c < dpitch; ++c)
                            p[c] = inside ? (double)h2f(src[(size_t)sy * src_row_stride + (size_t)sx * dpitch + c]) : 0.0;
                    }
                double* o = out + ((size_t)y * Wout + x) * N;
                double* sc = scale + ((size_t)y * Wout + x) * N;
                for (int n = 0; n < N; ++n) o[n] = sc[n] = 0.0;
                for (int k = 0; k < K; ++k) {
                    const double a = patch[k];
                    if (a == 0.0) continue;
                    const double* w = Wt.data() + (size_t)k * N;
                    for (int n = 0; n < N; ++n) { o[n] += a * w[n]; sc[n] += std::fabs(a * w[n]); }
                }
            }
    });
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------
// IEEE binary16 <-> binary32, round-to-nearest-even (what __float2half does, float_half_convert.h:32-43).
// ---------------------------------------------------------------------------------------------------------------
static inline uint16_t f2h(float f) {
    uint32_t x; std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u | ((mag >> 13) & 0x3ffu) : 0));
    if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);            // rounds to >= 65520 -> inf
    if (mag < 0x33000001u) return (uint16_t)sign;                          // <= 2^-25 -> 0 (tie to even = 0)
    int exp = (int)(mag >> 23) - 127;
    uint32_t man = (mag & 0x7fffffu) | 0x800000u;
    int shift = exp >= -14 ? 13 : 13 + (-14 - exp);                        // subnormal halves lose more bits
    uint32_t q = man >> shift, rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) ++q;
    uint32_t h = exp >= -14 ? (uint32_t)((exp + 15 - 1) << 10) + q : q;    // q carries the implicit bit / overflow
    return (uint16_t)(sign | h);
}
static inline float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ffu, x;
    if (e == 0) {
        if (m == 0) x = sign;
        else { int s = 0; while (!(m & 0x400u)) { m <<= 1; ++s; } x = sign | (uint32_t)(127 - 15 - s + 1) << 23 | (m & 0x3ffu) << 13; }
    } else if (e == 31) x = sign | 0x7f800000u | m << 13;
    else x = sign | (e + 112) << 23 | m << 13;
    float f; std::memcpy(&f, &x, 4); return f;
}
void oracle_float_to_half(const float* in, uint16_t* out, long n) { for (long i = 0; i < n; ++i) out[i] = f2h(in[i]); }
void oracle_half_to_float(const uint16_t* in, float* out, long n) { for (long i = 0; i < n; ++i) out[i] = h2f(in[i]); }

// fp64 product of binary16 operands for a list of rows: out[r][j] = sum_k double(A[rows[r]][k]) * double(B[k][j]),
// ascending k, plain double multiply-add (each product of two halves is exact in double).  out is nrows x N dense.
// abs_out (nullable) receives sum_k |a||b|, the scale used for the relative-error metric.
void oracle_gemm_f64_rows_f16(const uint16_t* A, long lda, const uint16_t* B, long ldb, const int* rows, int nrows,
                              double* out, double* abs_out, int N, int K, int nthreads) {
    parallel_ranges(nthreads, nrows, [&](long lo, long hi) {
        std::vector<double> brow(N);
        for (long r = lo; r < hi; ++r) {
            double* acc = out + (size_t)r * N;
            double* aacc = abs_out ? abs_out + (size_t)r * N : nullptr;
            for (int j = 0; j < N; ++j) acc[j] = 0.0;
            if (aacc) for (int j = 0; j < N; ++j) aacc[j] = 0.0;
            const uint16_t* a = A + (size_t)rows[r] * lda;
            for (int k = 0; k < K; ++k) {
                double av = (double)h2f(a[k]);
                const uint16_t* b = B + (size_t)k * ldb;
                for (int j = 0; j < N; ++j) brow[j] = (double)h2f(b[j]);
                for (int j = 0; j < N; ++j) acc[j] += av * brow[j];
                if (aacc) { double aa = std::fabs(av); for (int j = 0; j < N; ++j) aacc[j] += aa * std::fabs(brow[j]); }
            }
        }
    });
}

// fp64 product of fp32 operands for a list of rows (+ sum |a||b|): the error scale for the fp32 tolerance.
void oracle_gemm_f64_rows_f32(const float* A, long lda, const float* B, long ldb, const int* rows, int nrows, double* out,
                              double* abs_out, int N, int K, int nthreads) {
    parallel_ranges(nthreads, nrows, [&](long lo, long hi) {
        for (long r = lo; r < hi; ++r) {
            double* acc = out + (size_t)r * N;
            double* aacc = abs_out ? abs_out + (size_t)r * N : nullptr;
            for (int j = 0; j < N; ++j) acc[j] = 0.0;
            if (aacc) for (int j = 0; j < N; ++j) aacc[j] = 0.0;
            const float* a = A + (size_t)rows[r] * lda;
            for (int k = 0; k < K; ++k) {
                double av = (double)a[k];
                const float* b = B + (size_t)k * ldb;
                for (int j = 0; j < N; ++j) acc[j] += av * (double)b[j];
                if (aacc) { double aa = std::fabs(av); for (int j = 0; j < N; ++j) aacc[j] += aa * std::fabs((double)b[j]); }
            }
        }
    });
}

// nn/operators/ReLU.h:57-82: _sign = ~(bits & 0x80000000) >> 31 (unsigned), dst = float(_sign) * src.
static inline float relu_by_sign(float v, unsigned* kept) {
    uint32_t bits;
    std::memcpy(&bits, &v, 4);
    const unsigned s = (~(bits & 0x80000000u)) >> 31;
    if (kept) *kept = s;
    volatile float f = (float)s;       // keep the multiplication (0 * -inf must give NaN, 0 * -x must give -0)
    return f * v;
}
void oracle_relu_f32(const float* src, float* dst, long n) {
    for (long i = 0; i < n; ++i) dst[i] = relu_by_sign(src[i], nullptr);
}
// ReLU.h:86-127: thread t handles floats 8t..8t+7 as two float4; first quad -> bits 4..7, second quad -> bits 0..3.
void oracle_relu_f32_rec(const float* src, float* dst, unsigned char* rec_map, long n) {
    for (long t = 0; t < n / 8; ++t) {
        unsigned mask = 0;
        for (int e = 0; e < 8; ++e) {
            unsigned s;
            dst[8 * t + e] = relu_by_sign(src[8 * t + e], &s);
            mask |= s << (e < 4 ? 4 + e : e - 4);
        }
        rec_map[t] = (unsigned char)mask;
    }
}
// ReLU.h:131-165
void oracle_relu_f32_backward(const float* src, float* dst, const unsigned char* rec_map, long n) {
    for (long t = 0; t < n / 8; ++t)
        for (int e = 0; e < 8; ++e) {
            volatile float f = (float)((rec_map[t] >> (e < 4 ? 4 + e : e - 4)) & 1u);
            dst[8 * t + e] = f * src[8 * t + e];
        }
}

int oracle_pool_size(int nthreads) { return (int)global_pool(nthreads).size(); }

}  // extern "C"
