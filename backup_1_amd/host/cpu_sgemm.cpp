// de::cpu::sgemm: host SGEMM for de::Matrix<float> (reference: GEMM/CPU/sgemm.h:22-60, which re-packs B into
// 16-column panels and runs 32x16x64 AVX2 blocks on a 3x4 grid of thread-pool tasks, sgemm_callers.h:1227-1249).
//
// Same arithmetic contract as the reference -- every output element is ONE fp32 accumulator updated by a fused
// multiply-add over ascending k -- with a different blocking: B is packed once into 16-column panels, then worker
// threads pull (6-row x 16-column) register tiles from an atomic counter and run the whole K extent with the
// twelve accumulators held in registers (the reference stores and reloads C every 64 k).
// Departures from the reference, all of them defect fixes: dst is constructed (N wide, M high) (sgemm.h:40 passes
// (K, K)); row partitions cannot overlap; K need not be a multiple of 8.
#include <immintrin.h>

#include <atomic>
#include <thread>
#include <vector>

#include "decx_classes.hpp"

namespace {

constexpr int kRowTile = 6, kPanel = 16;

// rows x 16 tile over the full K extent; `rows` <= 6.  Bp: packed panel [K][16].
template <int ROWS>
void tile_kernel(const float* A, size_t lda, const float* Bp, float* C, size_t ldc, int K, int cols) {
    __m256 acc[ROWS][2];
    for (int r = 0; r < ROWS; ++r) acc[r][0] = acc[r][1] = _mm256_setzero_ps();
    for (int k = 0; k < K; ++k) {
        const __m256 b0 = _mm256_loadu_ps(Bp + (size_t)k * kPanel), b1 = _mm256_loadu_ps(Bp + (size_t)k * kPanel + 8);
        for (int r = 0; r < ROWS; ++r) {
            const __m256 a = _mm256_set1_ps(A[r * lda + k]);
            acc[r][0] = _mm256_fmadd_ps(a, b0, acc[r][0]);
            acc[r][1] = _mm256_fmadd_ps(a, b1, acc[r][1]);
        }
    }
    for (int r = 0; r < ROWS; ++r) {
        _mm256_storeu_ps(C + r * ldc, acc[r][0]);
        if (cols > 8) _mm256_storeu_ps(C + r * ldc + 8, acc[r][1]);
    }
}

void run_tile(int rows, const float* A, size_t lda, const float* Bp, float* C, size_t ldc, int K, int cols) {
    switch (rows) {
        case 6: tile_kernel<6>(A, lda, Bp, C, ldc, K, cols); break;
        case 5: tile_kernel<5>(A, lda, Bp, C, ldc, K, cols); break;
        case 4: tile_kernel<4>(A, lda, Bp, C, ldc, K, cols); break;
        case 3: tile_kernel<3>(A, lda, Bp, C, ldc, K, cols); break;
        case 2: tile_kernel<2>(A, lda, Bp, C, ldc, K, cols); break;
        default: tile_kernel<1>(A, lda, Bp, C, ldc, K, cols); break;
    }
}

}  // namespace

namespace de {
namespace cpu {

DH sgemm(Matrix<float>& A_, Matrix<float>& B_, Matrix<float>& dst_) {
    static char ok_msg[] = "No error\n";
    static char dims_msg[] = "Matrix Dims don't match each other";
    static char alloc_msg[] = "Fail to allocate memory\n";
    static char factory_msg[] = "Container was not created by this library's factories\n";
    auto* A = dynamic_cast<decx::_Matrix<float>*>(&A_);
    auto* B = dynamic_cast<decx::_Matrix<float>*>(&B_);
    auto* dst = dynamic_cast<decx::_Matrix<float>*>(&dst_);
    if (!A || !B || !dst) return DH{decx::DECX_FAIL_ErrorParams, factory_msg};
    if (A->width != B->height) return DH{decx::DECX_FAIL_DimsNotMatching, dims_msg};       // sgemm.h:35-38
    const int M = (int)A->height, K = (int)A->width, N = (int)B->width;
    // a dst that is (or shares its payload with) an operand is computed into a fresh matrix whose payload it then takes
    decx::_Matrix<float> fresh;
    decx::_Matrix<float>* user_dst = dst;
    if (dst == A || dst == B || dst->shares_block_with(*A) || dst->shares_block_with(*B)) {
        if (!fresh.construct((uint)N, (uint)M, decx::Page_Default)) return DH{decx::DECX_FAIL_ALLOCATION, alloc_msg};
        dst = &fresh;
    } else if (!dst->re_construct((uint)N, (uint)M, decx::Page_Default)) {
        return DH{decx::DECX_FAIL_ALLOCATION, alloc_msg};
    }
    if (M == 0 || N == 0) {
        if (dst != user_dst) user_dst->share_from(fresh);
        return DH{decx::DECX_SUCCESS, ok_msg};
    }

    const int n8 = (N + 7) / 8 * 8;                      // columns are produced in units of 8, inside the pitch
    const int panels = (n8 + kPanel - 1) / kPanel;
    float* packed = static_cast<float*>(std::aligned_alloc(64, ((size_t)panels * kPanel * (K > 0 ? K : 1) * 4 + 63) / 64 * 64));
    if (!packed) return DH{decx::DECX_FAIL_ALLOCATION, alloc_msg};

    int nthreads = (int)std::thread::hardware_concurrency();
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 16) nthreads = 16;                    // the reference sizes its pool arrays to 16 (thread_pool.h:18)

    auto parallel = [&](auto&& body) {
        std::vector<std::thread> th;
        for (int t = 1; t < nthreads; ++t) th.emplace_back(body);
        body();
        for (auto& x : th) x.join();
    };

    // pack B: panel p holds columns [16p, 16p+16) as [K][16]; a last half panel is zero-extended
    std::atomic<int> next_panel{0};
    parallel([&] {
        for (int p = next_panel++; p < panels; p = next_panel++) {
            const int c0 = p * kPanel, w = n8 - c0 < kPanel ? n8 - c0 : kPanel;
            float* d = packed + (size_t)p * kPanel * K;
            for (int k = 0; k < K; ++k) {
                const float* s = B->Mat.ptr + (size_t)k * B->pitch + c0;
                _mm256_storeu_ps(d + (size_t)k * kPanel, _mm256_loadu_ps(s));
                _mm256_storeu_ps(d + (size_t)k * kPanel + 8, w > 8 ? _mm256_loadu_ps(s + 8) : _mm256_setzero_ps());
            }
        }
    });

    const int row_tiles = (M + kRowTile - 1) / kRowTile;
    const long total = (long)row_tiles * panels;
    std::atomic<long> next_tile{0};
    parallel([&] {
        for (long id = next_tile++; id < total; id = next_tile++) {
            const int p = (int)(id / row_tiles), rt = (int)(id % row_tiles);    // walk one panel's rows before the next panel
            const int r0 = rt * kRowTile, rows = M - r0 < kRowTile ? M - r0 : kRowTile;
            const int c0 = p * kPanel, cols = n8 - c0 < kPanel ? n8 - c0 : kPanel;
            run_tile(rows, A->Mat.ptr + (size_t)r0 * A->pitch, A->pitch, packed + (size_t)p * kPanel * K,
                     dst->Mat.ptr + (size_t)r0 * dst->pitch + c0, dst->pitch, K, cols);
        }
    });
    std::free(packed);
    if (dst != user_dst) user_dst->share_from(fresh);
    return DH{decx::DECX_SUCCESS, ok_msg};
}

}  // namespace cpu
}  // namespace de
