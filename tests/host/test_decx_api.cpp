// Exercises the DECX-named C++ API (backup_1_amd/host/DECX.h) the way the reference's demo programs do
// (test/test/CUDA_GEMM/CUDA_GEMM.cpp, test/test/"generating classes"/*.h), but with assertions, and checks results
// against the CPU oracle (liboracle.so).  Usage: test_decx_api cpu | cpu-small | gpu   (cpu-small: what the sanitizer
// builds of backup_1_amd/host/Makefile run)
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../backup_1_amd/host/DECX.h"

extern "C" {
void oracle_sgemm_chain_fast(const float* A, long lda, const float* B, long ldb, const float* Cin, long ldc, float* D,
                             long ldd, int M, int N, int K, int nthreads);
int oracle_conv2_chain(const float* src, int H, int W, int dpitch, long src_row_stride, const float* filt, int N, int kh,
                       int kw, long filt_stride, long filt_row_stride, float* dst, int dst_dpitch, long dst_row_stride,
                       int flag, int nthreads);
int oracle_conv2_f64_f16(const uint16_t* src, int H, int W, int dpitch, long src_row_stride, const uint16_t* filt, int N,
                         int kh, int kw, long filt_stride, long filt_row_stride, double* out, double* scale, int flag,
                         int nthreads);
int oracle_decx_cpu_sgemm(const float* A, long lda, const float* B, long ldb, float* D, long ldd, int M, int N, int K,
                          int nthreads);
void oracle_gemm_f64_rows_f16(const uint16_t* A, long lda, const uint16_t* B, long ldb, const int* rows, int nrows,
                              double* out, double* abs_out, int N, int K, int nthreads);
}

static int g_fail = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) { std::printf("  CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_fail; } \
    } while (0)
#define RUN(fn)                                   \
    do {                                          \
        int before = g_fail;                      \
        std::printf("RUN  %s\n", #fn); std::fflush(stdout); \
        fn();                                     \
        std::printf("%s %s\n", g_fail == before ? "PASS" : "FAIL", #fn); std::fflush(stdout); \
    } while (0)

static std::mt19937 rng(12345);
static float small_int() { return (float)((int)(rng() % 9) - 4); }
static float unif() { return (float)((rng() >> 8) * (1.0 / 8388608.0) - 1.0); }

template <class F>
static void fill(de::Matrix<float>& m, F f) {
    for (uint i = 0; i < m.Height(); ++i)
        for (uint j = 0; j < m.Width(); ++j) m.index(i, j) = f();
}
static std::vector<float> dense(de::Matrix<float>& m) {
    std::vector<float> v((size_t)m.Height() * m.Width());
    for (uint i = 0; i < m.Height(); ++i)
        for (uint j = 0; j < m.Width(); ++j) v[(size_t)i * m.Width() + j] = m.index(i, j);
    return v;
}
static std::vector<float> chain(de::Matrix<float>& A, de::Matrix<float>& B, de::Matrix<float>* C = nullptr) {
    int M = A.Height(), K = A.Width(), N = B.Width();
    std::vector<float> a = dense(A), b = dense(B), c, d((size_t)M * N);
    if (C) c = dense(*C);
    oracle_sgemm_chain_fast(a.data(), K, b.data(), N, C ? c.data() : nullptr, N, d.data(), N, M, N, K, 0);
    return d;
}

// ------------------------------------------------------------------ CPU-only checks ----------------------------
static void containers_follow_reference_pitch_rules() {
    de::Matrix<float>& m = de::CreateMatrixRef<float>(13, 7, decx::Page_Default);
    CHECK(m.Width() == 13 && m.Height() == 7 && m.TotalBytes() == 13u * 7 * 4);     // width*height*sizeof (Matrix.h:262-263), not the pitched size
    m.index(6, 12) = 3.5f;
    CHECK((&m.index(6, 12)) - (&m.index(0, 0)) == 6 * 16 + 12);
    de::Matrix<de::Half>& h = de::CreateMatrixRef<de::Half>(17, 3, decx::Page_Default);
    CHECK(h.TotalBytes() == 17u * 3 * 2);                                             // Matrix.h:317-318
    CHECK((&h.index(1, 0)) - (&h.index(0, 0)) == 32);                                 // pitch = ceil16(17) = 32
    de::Tensor<float>& t = de::CreateTensorRef<float>(5, 6, 3, decx::Page_Default);  // width 5, height 6, depth 3
    CHECK(t.Width() == 5 && t.Height() == 6 && t.Depth() == 3);
    CHECK((&t.index(1, 0, 0)) - (&t.index(0, 0, 0)) == 8 * 4);                        // wpitch 8, dpitch 4
    CHECK((&t.index(0, 1, 0)) - (&t.index(0, 0, 0)) == 4);
    bool zero = true;
    for (int i = 0; i < 6 * 8 * 4; ++i) zero = zero && (&t.index(0, 0, 0))[i] == 0.0f;
    CHECK(zero);                                                                      // Tensor.h:312 zero-fills
    de::TensorArray<float>& ta = de::CreateTensorArrayRef<float>(3, 3, 64, 5, decx::Page_Default);
    CHECK(ta.TensorNum() == 5 && (&ta.index(0, 0, 0, 1)) - (&ta.index(0, 0, 0, 0)) == 3 * 4 * 64);   // _gap
    CHECK((&ta.index(1, 2, 7, 0)) - (&ta.index(0, 0, 0, 0)) == 1 * 4 * 64 + 2 * 64 + 7);
    m.release(); h.release(); t.release(); ta.release();
}

static void assignment_shares_the_payload() {   // Matrix.h:510-530, Tensor.h:501-526: the block is shared and counted
    de::Matrix<float>& a = de::CreateMatrixRef<float>(13, 7, decx::Page_Default);
    de::Matrix<float>& b = de::CreateMatrixRef<float>();
    fill(a, small_int);
    b = a;
    CHECK(b.Width() == 13 && b.Height() == 7 && b.TotalBytes() == a.TotalBytes());
    CHECK(&b.index(3, 5) == &a.index(3, 5));                       // same memory, not a copy
    a.index(3, 5) = 42.f;
    CHECK(b.index(3, 5) == 42.f);
    a.release();                                                    // the other holder keeps the block alive
    CHECK(b.index(3, 5) == 42.f);
    b.index(6, 12) = 1.f;
    b.release();
    de::Tensor<float>& t = de::CreateTensorRef<float>(5, 6, 3, decx::Page_Default);
    de::Tensor<float>& u = de::CreateTensorRef<float>();
    u = t;
    CHECK(&u.index(2, 1, 1) == &t.index(2, 1, 1) && u.Depth() == 3);
    t.release();
    u.index(5, 4, 2) = 2.f;
    u.release();
    de::MatrixArray<float>& ma = de::CreateMatrixArrayRef<float>(9, 4, 3, decx::Page_Default);
    de::MatrixArray<float>& mb = de::CreateMatrixArrayRef<float>();
    mb = ma;
    CHECK(&mb.index(3, 8, 2) == &ma.index(3, 8, 2) && mb.MatrixNumber() == 3);
    ma.release(); mb.release();
}

static void cpu_sgemm_into_an_operand() {        // dst is A (square): computed aside, then dst takes the new payload
    const int S = 40;
    de::Matrix<float>& A = de::CreateMatrixRef<float>(S, S, decx::Page_Default);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(S, S, decx::Page_Default);
    de::Matrix<float>& A2 = de::CreateMatrixRef<float>();
    fill(A, unif); fill(B, unif);
    std::vector<float> want = chain(A, B);
    A2 = A;                                                          // a second holder of A's payload
    std::vector<float> a_before = dense(A);
    CHECK(de::cpu::sgemm(A, B, A).error_type == decx::DECX_SUCCESS);
    std::vector<float> got = dense(A);
    CHECK(std::memcmp(got.data(), want.data(), got.size() * 4) == 0);
    CHECK(dense(A2) == a_before);                                    // the old payload is untouched
    A.release(); B.release(); A2.release();
}

static void half_conversion() {
    CHECK(de::Float2Half(1.0f).val == 0x3C00 && de::Float2Half(-2.0f).val == 0xC000);
    CHECK(de::Float2Half(65504.0f).val == 0x7BFF && de::Float2Half(65520.0f).val == 0x7C00);
    CHECK(de::Float2Half(1.00048828125f).val == 0x3C00 && de::Float2Half(1.00146484375f).val == 0x3C02);   // ties to even
    CHECK(de::Float2Half(5.9604645e-8f).val == 0x0001 && de::Float2Half(2.9802322e-8f).val == 0x0000);
    for (unsigned v = 0; v < 0x7C00; ++v) {
        de::Half h; h.val = (unsigned short)v;
        CHECK(de::Float2Half(de::Half2Float(h)).val == v);
        if (g_fail) break;
    }
}

static void gemm_refuses_before_init() {
    de::Matrix<float>& A = de::CreateMatrixRef<float>(8, 8, decx::Page_Default);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(8, 8, decx::Page_Default);
    de::Matrix<float>& C = de::CreateMatrixRef<float>();
    de::DH h = de::cuda::GEMM(A, B, C);
    CHECK(h.error_type == decx::DECX_FAIL_not_init && std::strstr(h.error_string, "initialized first"));
    de::Tensor<float>& s = de::CreateTensorRef<float>(8, 8, 4, decx::Page_Default);
    de::TensorArray<float>& k = de::CreateTensorArrayRef<float>(3, 3, 4, 2, decx::Page_Default);
    de::Tensor<float>& d = de::CreateTensorRef<float>();
    CHECK(de::cuda::Conv2_MK_im2col(s, k, d, 1).error_type == decx::DECX_FAIL_not_init);
}

static void cpu_sgemm_case(int M, int K, int N, bool ints) {
    de::Matrix<float>& A = de::CreateMatrixRef<float>(K, M, decx::Page_Default);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(N, K, decx::Page_Default);
    de::Matrix<float>& C = de::CreateMatrixRef<float>();
    if (ints) { fill(A, small_int); fill(B, small_int); } else { fill(A, unif); fill(B, unif); }
    de::DH h = de::cpu::sgemm(A, B, C);
    CHECK(h.error_type == decx::DECX_SUCCESS && C.Width() == (uint)N && C.Height() == (uint)M);
    std::vector<float> got = dense(C), want = chain(A, B);
    CHECK(std::memcmp(got.data(), want.data(), got.size() * 4) == 0);                // bit-identical to the fused chain
    A.release(); B.release(); C.release();
}
// the restated thread-pool SGEMM of the oracle (12 tasks on a pool of workers, packaged tasks and futures) against its own
// scalar chain: the data-race and memory checks of the sanitizer builds run over this
static void oracle_pool_sgemm_case(int M, int K, int N) {
    const int n8 = (N + 7) / 8 * 8;
    std::vector<float> a((size_t)M * K), b((size_t)K * n8, 0.f), d((size_t)M * n8, 0.f), bd((size_t)K * N), want((size_t)M * N);
    for (auto& v : a) v = unif();
    for (int k = 0; k < K; ++k) for (int j = 0; j < N; ++j) bd[(size_t)k * N + j] = b[(size_t)k * n8 + j] = unif();
    CHECK(oracle_decx_cpu_sgemm(a.data(), K, b.data(), n8, d.data(), n8, M, N, K, 0) == 0);
    oracle_sgemm_chain_fast(a.data(), K, bd.data(), N, nullptr, 0, want.data(), N, M, N, K, 0);
    bool same = true;
    for (int i = 0; i < M; ++i) same = same && std::memcmp(&d[(size_t)i * n8], &want[(size_t)i * N], (size_t)N * 4) == 0;
    CHECK(same);
}
static void oracle_thread_pool_sgemm() {
    oracle_pool_sgemm_case(200, 136, 72);
    oracle_pool_sgemm_case(97, 64, 40);
    oracle_pool_sgemm_case(33, 24, 9);
    for (int rep = 0; rep < 3; ++rep) oracle_pool_sgemm_case(64, 128, 128);      // the pool is reused between calls
}

static bool g_small = false;     // "cpu-small": the sanitizer builds skip the one large case
static void cpu_sgemm_matches_chain_bit_for_bit() {
    if (!g_small) cpu_sgemm_case(1024, 1024, 1024, false);      // config 1
    cpu_sgemm_case(100, 136, 72, false);
    cpu_sgemm_case(33, 7, 9, false);
    cpu_sgemm_case(1, 1, 1, false);
    cpu_sgemm_case(301, 150, 455, true);
    de::Matrix<float>& A = de::CreateMatrixRef<float>(10, 4, decx::Page_Default);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(4, 11, decx::Page_Default);
    de::Matrix<float>& C = de::CreateMatrixRef<float>();
    CHECK(de::cpu::sgemm(A, B, C).error_type == decx::DECX_FAIL_DimsNotMatching);    // sgemm.h:35-38
}

// ------------------------------------------------------------------ GPU checks --------------------------------

template <int M, int N, int K>
static void cuda_gemm_mem_exch() {     // CUDA_GEMM.cpp:15-57
    de::Matrix<float>& A = de::CreateMatrixRef<float>(K, M, 0);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(N, K, 0);
    de::Matrix<float>& C = de::CreateMatrixRef<float>(N, M, 0);
    for (uint i = 0; i < A.Height(); ++i) for (uint j = 0; j < A.Width(); ++j) A.index(i, j) = j * 0.1;
    for (uint i = 0; i < B.Height(); ++i) for (uint j = 0; j < B.Width(); ++j) B.index(i, j) = i * 0.1;
    float sum = 0;
    for (int i = 0; i < K; ++i) sum += (0.1 * i * 0.1 * i);
    de::DH h = de::cuda::GEMM(A, B, C);
    CHECK(h.error_type == decx::DECX_SUCCESS);
    bool all = true;
    for (uint i = 0; i < C.Height(); ++i)
        for (uint j = 0; j < C.Width(); ++j) all = all && std::fabs(C.index(i, j) - sum) / sum < 1e-5 * std::sqrt((double)K);
    CHECK(all);
    A.release(); B.release(); C.release();
}
template <int M, int N, int K>
static void cuda_gemm_on_GPU() {       // CUDA_GEMM.cpp:59-109
    de::Matrix<float>& A = de::CreateMatrixRef<float>(K, M, 0);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(N, K, 0);
    de::Matrix<float>& C = de::CreateMatrixRef<float>(N, M, 0);
    de::GPU_Matrix<float>& dA = de::CreateGPUMatrixRef<float>(K, M);
    de::GPU_Matrix<float>& dB = de::CreateGPUMatrixRef<float>(N, K);
    de::GPU_Matrix<float>& dC = de::CreateGPUMatrixRef<float>(N, M);
    for (uint i = 0; i < A.Height(); ++i) for (uint j = 0; j < A.Width(); ++j) A.index(i, j) = j * 0.1;
    for (uint i = 0; i < B.Height(); ++i) for (uint j = 0; j < B.Width(); ++j) B.index(i, j) = i * 0.1;
    float sum = 0;
    for (int i = 0; i < K; ++i) sum += (0.1 * i * 0.1 * i);
    dA.Load_from_host(A); dB.Load_from_host(B);
    de::DH h = de::cuda::GEMM(dA, dB, dC);
    CHECK(h.error_type == decx::DECX_SUCCESS);
    dC.Load_to_host(C);
    bool all = true;
    for (uint i = 0; i < C.Height(); ++i)
        for (uint j = 0; j < C.Width(); ++j) all = all && std::fabs(C.index(i, j) - sum) / sum < 1e-5 * std::sqrt((double)K);
    CHECK(all);
    A.release(); B.release(); C.release(); dA.release(); dB.release(); dC.release();
}
static void reference_demo_known_answer() {
    cuda_gemm_mem_exch<512, 1024, 2048>();
    cuda_gemm_on_GPU<2048, 2048, 2048>();        // what the reference's main() runs (CUDA_GEMM.cpp:112-116)
}

static void gemm_fp32_all_flavours() {
    const int M = 300, K = 150, N = 450;     // ragged everywhere
    de::Matrix<float>& A = de::CreateMatrixRef<float>(K, M, 0);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(N, K, 0);
    de::Matrix<float>& C = de::CreateMatrixRef<float>(N, M, 0);
    de::Matrix<float>& D = de::CreateMatrixRef<float>();
    fill(A, small_int); fill(B, small_int); fill(C, small_int);
    CHECK(de::cuda::GEMM(A, B, D).error_type == 0 && D.Width() == (uint)N && D.Height() == (uint)M);
    CHECK(dense(D) == chain(A, B));                                        // integer data: exact
    CHECK(de::cuda::GEMM(A, B, C, D).error_type == 0);
    CHECK(dense(D) == chain(A, B, &C));
    de::release_all_tmp();            // Memory_pool.h:23-37: the device blocks the host overloads kept go back; calls go on working
    CHECK(de::cuda::GEMM(A, B, C, D).error_type == 0);
    CHECK(dense(D) == chain(A, B, &C));
    std::vector<float> want = chain(A, B, &C);
    CHECK(de::cuda::GEMM(A, B, C, C).error_type == 0);                     // dst aliasing C
    CHECK(dense(C) == want);
    {   // a pageable C used in place keeps its data (re-constructing it as pinned would drop C before the upload)
        de::Matrix<float>& Cp = de::CreateMatrixRef<float>(N, M, decx::Page_Default);
        fill(Cp, small_int);
        std::vector<float> want_p = chain(A, B, &Cp);
        CHECK(de::cuda::GEMM(A, B, Cp, Cp).error_type == 0);
        CHECK(dense(Cp) == want_p);
        Cp.release();
        // dst is A itself (square): computed aside, dst then holds the product
        de::Matrix<float>& S1 = de::CreateMatrixRef<float>(96, 96, decx::Page_Default);
        de::Matrix<float>& S2 = de::CreateMatrixRef<float>(96, 96, decx::Page_Locked);
        fill(S1, small_int); fill(S2, small_int);
        std::vector<float> want_s = chain(S1, S2);
        CHECK(de::cuda::GEMM(S1, S2, S1).error_type == 0);
        CHECK(dense(S1) == want_s);
        std::vector<float> want_t = chain(S1, S2);
        CHECK(de::cuda::GEMM(S1, S2, S2).error_type == 0);
        CHECK(dense(S2) == want_t);
        S1.release(); S2.release();
    }
    // device-resident flavours
    de::GPU_Matrix<float>& dA = de::CreateGPUMatrixRef<float>(K, M);
    de::GPU_Matrix<float>& dB = de::CreateGPUMatrixRef<float>(N, K);
    de::GPU_Matrix<float>& dC = de::CreateGPUMatrixRef<float>(N, M);
    de::GPU_Matrix<float>& dD = de::CreateGPUMatrixRef<float>();          // empty: GEMM sizes it (GEMM.h:414)
    CHECK(dA.TotalBytes() == (size_t)K * M * 4 && dB.TotalBytes() == (size_t)N * K * 4);   // width*height*sizeof (GPU_Matrix.h:218-219)
    {
        de::GPU_Matrix<de::Half>& dh = de::CreateGPUMatrixRef<de::Half>(17, 3);
        CHECK(dh.TotalBytes() == 17u * 3 * 2);                             // GPU_Matrix.h:266-267
        de::GPU_Matrix<de::Half>& dh2 = de::CreateGPUMatrixRef<de::Half>();
        dh2 = dh;                                                          // shares the device block (GPU_Matrix.h:441-451)
        dh.release();
        CHECK(dh2.Width() == 17 && dh2.TotalBytes() == 17u * 3 * 2);
        dh2.release();
    }
    fill(A, unif); fill(B, unif); fill(C, unif);
    dA.Load_from_host(A); dB.Load_from_host(B); dC.Load_from_host(C);
    CHECK(de::cuda::GEMM(dA, dB, dD).error_type == 0 && dD.Width() == (uint)N && dD.Height() == (uint)M);
    de::Matrix<float>& R = de::CreateMatrixRef<float>(N, M, 0);
    dD.Load_to_host(R);
    CHECK(dense(R) == chain(A, B));          // real-valued data: the kernel is the reference's fused chain, bit for bit
    CHECK(de::cuda::GEMM(dA, dB, dC, dD).error_type == 0);
    dD.Load_to_host(R);
    CHECK(dense(R) == chain(A, B, &C));
    // dims mismatch -> 0x03 (GEMM.h:68, :408)
    de::Matrix<float>& Bad = de::CreateMatrixRef<float>(N, K + 1, 0);
    de::DH h = de::cuda::GEMM(A, Bad, D);
    CHECK(h.error_type == decx::DECX_FAIL_DimsNotMatching && std::strstr(h.error_string, "width of matrix A"));
    de::GPU_Matrix<float>& dBad = de::CreateGPUMatrixRef<float>(N, K + 1);
    CHECK(de::cuda::GEMM(dA, dBad, dD).error_type == decx::DECX_FAIL_DimsNotMatching);
}

static void gemm_fp16_flavours() {
    const int M = 130, K = 200, N = 77;
    de::Matrix<de::Half>& A = de::CreateMatrixRef<de::Half>(K, M, 0);
    de::Matrix<de::Half>& B = de::CreateMatrixRef<de::Half>(N, K, 0);
    de::Matrix<de::Half>& D = de::CreateMatrixRef<de::Half>();
    std::vector<uint16_t> a((size_t)M * K), b((size_t)K * N);
    for (int i = 0; i < M; ++i) for (int j = 0; j < K; ++j) { A.index(i, j) = de::Float2Half(unif()); a[(size_t)i * K + j] = A.index(i, j).val; }
    for (int i = 0; i < K; ++i) for (int j = 0; j < N; ++j) { B.index(i, j) = de::Float2Half(unif()); b[(size_t)i * N + j] = B.index(i, j).val; }
    std::vector<int> rows(M);
    for (int i = 0; i < M; ++i) rows[i] = i;
    std::vector<double> ref((size_t)M * N), scale((size_t)M * N);
    oracle_gemm_f64_rows_f16(a.data(), K, b.data(), N, rows.data(), M, ref.data(), scale.data(), N, K, 0);
    auto check = [&](de::Matrix<de::Half>& R) {
        double e = 0;
        for (int i = 0; i < M; ++i)
            for (int j = 0; j < N; ++j)
                e = std::fmax(e, std::fabs(de::Half2Float(R.index(i, j)) - ref[(size_t)i * N + j]) / scale[(size_t)i * N + j]);
        return e;
    };
    CHECK(de::cuda::GEMM(A, B, D).error_type == 0 && D.Width() == (uint)N && D.Height() == (uint)M);
    CHECK(check(D) < 2e-3);
    de::GPU_Matrix<de::Half>& dA = de::CreateGPUMatrixRef<de::Half>(K, M);
    de::GPU_Matrix<de::Half>& dB = de::CreateGPUMatrixRef<de::Half>(N, K);
    de::GPU_Matrix<de::Half>& dD = de::CreateGPUMatrixRef<de::Half>();    // not pre-sized: the fp32 behaviour (GEMM.h:414)
    dA.Load_from_host(A); dB.Load_from_host(B);
    CHECK(de::cuda::GEMM(dA, dB, dD).error_type == 0);
    de::Matrix<de::Half>& R = de::CreateMatrixRef<de::Half>(N, M, 0);
    dD.Load_to_host(R);
    CHECK(check(R) < 2e-3);
}

static void conv_case(int H, int W, int C, int N, int kh, int kw, int flag) {
    de::Tensor<float>& src = de::CreateTensorRef<float>(W, H, C, 0);
    de::TensorArray<float>& ker = de::CreateTensorArrayRef<float>(kw, kh, C, N, 0);
    de::Tensor<float>& dst = de::CreateTensorRef<float>();
    for (int y = 0; y < H; ++y) for (int x = 0; x < W; ++x) for (int c = 0; c < C; ++c) src.index(y, x, c) = small_int();
    for (int n = 0; n < N; ++n) for (int i = 0; i < kh; ++i) for (int j = 0; j < kw; ++j) for (int c = 0; c < C; ++c) ker.index(i, j, c, n) = small_int();
    de::DH h = de::cuda::Conv2_MK_im2col(src, ker, dst, flag);
    CHECK(h.error_type == decx::DECX_SUCCESS);
    const int Ho = flag ? H : H - 2 * (kh / 2), Wo = flag ? W : W - 2 * (kw / 2);
    CHECK(dst.Width() == (uint)Wo && dst.Height() == (uint)Ho && dst.Depth() == (uint)N);
    const long s_row = &src.index(1, 0, 0) - &src.index(0, 0, 0), dp = &src.index(0, 1, 0) - &src.index(0, 0, 0);
    const long k_gap = N > 1 ? &ker.index(0, 0, 0, 1) - &ker.index(0, 0, 0, 0) : (long)kh * ((kw + 3) / 4 * 4) * dp;
    const long k_row = kh > 1 ? &ker.index(1, 0, 0, 0) - &ker.index(0, 0, 0, 0) : (long)((kw + 3) / 4 * 4) * dp;
    std::vector<float> want((size_t)Ho * Wo * N);
    CHECK(oracle_conv2_chain(&src.index(0, 0, 0), H, W, (int)dp, s_row, &ker.index(0, 0, 0, 0), N, kh, kw, k_gap, k_row,
                             want.data(), N, (long)Wo * N, flag, 0) == 0);
    bool same = true;
    for (int y = 0; y < Ho; ++y) for (int x = 0; x < Wo; ++x) for (int n = 0; n < N; ++n)
        same = same && dst.index(y, x, n) == want[((size_t)y * Wo + x) * N + n];
    CHECK(same);
    src.release(); ker.release(); dst.release();
}
static void gemm_long_lr() {
    const int M = 48, K = 16384, N = 200;        // short M, long K (GEMM_long_Lr.h's shape class), ragged N
    de::Matrix<float>& A = de::CreateMatrixRef<float>(K, M, 0);
    de::Matrix<float>& B = de::CreateMatrixRef<float>(N, K, 0);
    de::Matrix<float>& R = de::CreateMatrixRef<float>(N, M, 0);
    fill(A, unif); fill(B, unif);
    de::GPU_Matrix<float>& dA = de::CreateGPUMatrixRef<float>(K, M);
    de::GPU_Matrix<float>& dB = de::CreateGPUMatrixRef<float>(N, K);
    de::GPU_Matrix<float>& dD = de::CreateGPUMatrixRef<float>();
    dA.Load_from_host(A); dB.Load_from_host(B);
    CHECK(de::cuda::GEMM_Long_Lr(dA, dB, dD).error_type == decx::DECX_SUCCESS && dD.Width() == (uint)N && dD.Height() == (uint)M);
    dD.Load_to_host(R);
    CHECK(dense(R) == chain(A, B));               // real-valued data: the reference's fused chain over all of K, bit for bit
    de::GPU_Matrix<float>& dBad = de::CreateGPUMatrixRef<float>(N, K + 8);
    CHECK(de::cuda::GEMM_Long_Lr(dA, dBad, dD).error_type == decx::DECX_FAIL_DimsNotMatching);
}

static uint32_t bits_of(float v) { uint32_t b; std::memcpy(&b, &v, 4); return b; }
static void nn_relu_family() {               // nn/operators/ReLU.h:28-34
    const int W = 37, H = 13;                // pitch 40: the kernels run over the padding too
    de::Matrix<float>& X = de::CreateMatrixRef<float>(W, H, 0);
    de::Matrix<float>& G = de::CreateMatrixRef<float>(W, H, 0);
    de::Matrix<float>& R = de::CreateMatrixRef<float>(W, H, 0);
    fill(X, unif); fill(G, unif);
    X.index(0, 0) = 0.f; X.index(0, 1) = -0.f; X.index(0, 2) = -INFINITY; X.index(0, 3) = INFINITY;
    de::GPU_Matrix<float>& dX = de::CreateGPUMatrixRef<float>(W, H);
    de::GPU_Matrix<float>& dY = de::CreateGPUMatrixRef<float>(W, H);
    de::GPU_Matrix<float>& dG = de::CreateGPUMatrixRef<float>(W, H);
    de::GPU_Matrix<uchar>& dMap = de::CreateGPUMatrixRef<uchar>();
    dX.Load_from_host(X); dG.Load_from_host(G);
    auto expect_forward = [&](de::Matrix<float>& got) {
        int bad = 0;
        for (int i = 0; i < H; ++i)
            for (int j = 0; j < W; ++j) {
                const float x = X.index(i, j), y = got.index(i, j);
                if (std::isinf(x) && x < 0) bad += !std::isnan(y);                       // 0 * -inf
                else if (std::signbit(x)) bad += bits_of(y) != 0x80000000u;             // 0 * negative = -0.0
                else bad += bits_of(y) != bits_of(x);
            }
        return bad;
    };
    CHECK(de::nn::ReLU_f(dX, dY).error_type == decx::DECX_SUCCESS);
    dY.Load_to_host(R);
    CHECK(expect_forward(R) == 0);
    de::GPU_Matrix<float>& dY2 = de::CreateGPUMatrixRef<float>(W, H);
    CHECK(de::nn::ReLU_f_Rec(dX, dY2, dMap).error_type == decx::DECX_SUCCESS);
    CHECK(dMap.TotalBytes() >= (size_t)40 * H / 8);
    dY2.Load_to_host(R);
    CHECK(expect_forward(R) == 0);
    CHECK(de::nn::ReLU_f_Backward(dG, dY, dMap).error_type == decx::DECX_SUCCESS);
    dY.Load_to_host(R);
    int bad = 0;
    for (int i = 0; i < H; ++i)
        for (int j = 0; j < W; ++j) {
            const float g = G.index(i, j);
            const uint32_t want = std::signbit(X.index(i, j)) ? (bits_of(g) & 0x80000000u) : bits_of(g);   // 0 * g keeps g's sign
            bad += bits_of(R.index(i, j)) != want;
        }
    CHECK(bad == 0);
    de::GPU_Matrix<float>& dBad = de::CreateGPUMatrixRef<float>(W + 1, H);
    CHECK(de::nn::ReLU_f(dX, dBad).error_type == decx::DECX_FAIL_DimsNotMatching);
    de::GPU_Matrix<uchar>& dEmpty = de::CreateGPUMatrixRef<uchar>();
    CHECK(de::nn::ReLU_f_Backward(dG, dY, dEmpty).error_type == decx::DECX_FAIL_DimsNotMatching);
}

static void gemm3_matrix_arrays() {
    const int M = 150, K = 90, N = 210, NUM = 5;
    de::MatrixArray<float>& A = de::CreateMatrixArrayRef<float>(K, M, NUM, 0);
    de::MatrixArray<float>& B = de::CreateMatrixArrayRef<float>(N, K, NUM, 0);
    de::MatrixArray<float>& C = de::CreateMatrixArrayRef<float>(N, M, NUM, 0);
    de::MatrixArray<float>& D = de::CreateMatrixArrayRef<float>();
    CHECK(A.MatrixNumber() == (uint)NUM && (&A.index(0, 0, 1)) - (&A.index(0, 0, 0)) == 96 * M);   // pitch = ceil8(90) = 96
    for (int s = 0; s < NUM; ++s) {
        for (int i = 0; i < M; ++i) for (int j = 0; j < K; ++j) A.index(i, j, s) = small_int();
        for (int i = 0; i < K; ++i) for (int j = 0; j < N; ++j) B.index(i, j, s) = small_int();
        for (int i = 0; i < M; ++i) for (int j = 0; j < N; ++j) C.index(i, j, s) = small_int();
    }
    auto check = [&](de::MatrixArray<float>& R, bool with_c) {
        bool same = R.Width() == (uint)N && R.Height() == (uint)M && R.MatrixNumber() == (uint)NUM;
        for (int s = 0; s < NUM && same; ++s) {
            std::vector<float> a((size_t)M * K), b((size_t)K * N), c((size_t)M * N), d((size_t)M * N);
            for (int i = 0; i < M; ++i) for (int j = 0; j < K; ++j) a[(size_t)i * K + j] = A.index(i, j, s);
            for (int i = 0; i < K; ++i) for (int j = 0; j < N; ++j) b[(size_t)i * N + j] = B.index(i, j, s);
            for (int i = 0; i < M; ++i) for (int j = 0; j < N; ++j) c[(size_t)i * N + j] = C.index(i, j, s);
            oracle_sgemm_chain_fast(a.data(), K, b.data(), N, with_c ? c.data() : nullptr, N, d.data(), N, M, N, K, 0);
            for (int i = 0; i < M; ++i) for (int j = 0; j < N; ++j) same = same && R.index(i, j, s) == d[(size_t)i * N + j];
        }
        return same;
    };
    CHECK(de::cuda::GEMM3(A, B, D).error_type == decx::DECX_SUCCESS);
    CHECK(check(D, false));                                          // integer data: exact, every matrix of the array
    CHECK(de::cuda::GEMM3(A, B, C, D).error_type == decx::DECX_SUCCESS);
    CHECK(check(D, true));
    de::MatrixArray<float>& B4 = de::CreateMatrixArrayRef<float>(N, K, NUM - 1, 0);
    CHECK(de::cuda::GEMM3(A, B4, D).error_type == decx::DECX_FAIL_MNumNotMatching);
    // fp16 arrays against the fp64 product
    de::MatrixArray<de::Half>& Ah = de::CreateMatrixArrayRef<de::Half>(K, M, 3, 0);
    de::MatrixArray<de::Half>& Bh = de::CreateMatrixArrayRef<de::Half>(N, K, 3, 0);
    de::MatrixArray<de::Half>& Dh = de::CreateMatrixArrayRef<de::Half>();
    for (int s = 0; s < 3; ++s) {
        for (int i = 0; i < M; ++i) for (int j = 0; j < K; ++j) Ah.index(i, j, s) = de::Float2Half(unif());
        for (int i = 0; i < K; ++i) for (int j = 0; j < N; ++j) Bh.index(i, j, s) = de::Float2Half(unif());
    }
    CHECK(de::cuda::GEMM3(Ah, Bh, Dh).error_type == decx::DECX_SUCCESS);
    double worst = 0;
    for (int s = 0; s < 3; ++s)
        for (int i = 0; i < M; i += 7) for (int j = 0; j < N; ++j) {
            double r = 0, sc = 0;
            for (int k = 0; k < K; ++k) { double x = de::Half2Float(Ah.index(i, k, s)), y = de::Half2Float(Bh.index(k, j, s)); r += x * y; sc += std::fabs(x * y); }
            worst = std::fmax(worst, std::fabs(de::Half2Float(Dh.index(i, j, s)) - r) / sc);
        }
    CHECK(worst < 2e-3);
}

static void conv_device_resident() {
    const int H = 30, W = 26, C = 12, N = 10, kh = 3, kw = 3;        // width not a multiple of 4: padded rows in dst
    de::Tensor<float>& src = de::CreateTensorRef<float>(W, H, C, 0);
    de::TensorArray<float>& ker = de::CreateTensorArrayRef<float>(kw, kh, C, N, 0);
    for (int y = 0; y < H; ++y) for (int x = 0; x < W; ++x) for (int c = 0; c < C; ++c) src.index(y, x, c) = small_int();
    for (int n = 0; n < N; ++n) for (int i = 0; i < kh; ++i) for (int j = 0; j < kw; ++j) for (int c = 0; c < C; ++c) ker.index(i, j, c, n) = small_int();
    de::GPU_Tensor<float>& dsrc = de::CreateGPUTensorRef<float>(W, H, C);
    de::GPU_TensorArray<float>& dker = de::CreateGPUTensorArrayRef<float>(kw, kh, C, N);
    de::GPU_Tensor<float>& ddst = de::CreateGPUTensorRef<float>();
    dsrc.Load_from_host(src); dker.Load_from_host(ker);
    for (int flag = 0; flag < 2; ++flag) {
        de::Tensor<float>& want = de::CreateTensorRef<float>();
        CHECK(de::cuda::Conv2_MK_im2col(src, ker, want, flag).error_type == decx::DECX_SUCCESS);
        CHECK(de::cuda::Conv2_MK_im2col(dsrc, dker, ddst, flag).error_type == decx::DECX_SUCCESS);
        CHECK(ddst.Width() == want.Width() && ddst.Height() == want.Height() && ddst.Depth() == (uint)N);
        de::Tensor<float>& got = de::CreateTensorRef<float>(want.Width(), want.Height(), N, 0);
        ddst.Load_to_host(got);
        bool same = true;
        for (uint y = 0; y < want.Height(); ++y) for (uint x = 0; x < want.Width(); ++x) for (int n = 0; n < N; ++n)
            same = same && got.index(y, x, n) == want.index(y, x, n);
        CHECK(same);
        want.release(); got.release();
    }
    CHECK(de::cuda::Conv2_MK_im2col(dsrc, dker, ddst, 5).error_type == decx::DECX_FAIL_ErrorFlag);
    dsrc.release(); dker.release(); ddst.release(); src.release(); ker.release();
}

static void conv_half_containers() {
    // binary16 containers: channel pitch ceil8 (Tensor.h:214-235), fp32 accumulation, checked against fp64 on the same halves
    const int H = 30, W = 26, C = 12, N = 10, kh = 3, kw = 3;
    de::Tensor<de::Half>& src = de::CreateTensorRef<de::Half>(W, H, C, 0);
    de::TensorArray<de::Half>& ker = de::CreateTensorArrayRef<de::Half>(kw, kh, C, N, 0);
    for (int y = 0; y < H; ++y) for (int x = 0; x < W; ++x) for (int c = 0; c < C; ++c) src.index(y, x, c) = de::Float2Half(unif());
    for (int n = 0; n < N; ++n) for (int i = 0; i < kh; ++i) for (int j = 0; j < kw; ++j) for (int c = 0; c < C; ++c)
        ker.index(i, j, c, n) = de::Float2Half(0.1f * unif());
    const long dp = &src.index(0, 1, 0) - &src.index(0, 0, 0), s_row = &src.index(1, 0, 0) - &src.index(0, 0, 0);
    const long k_gap = &ker.index(0, 0, 0, 1) - &ker.index(0, 0, 0, 0), k_row = &ker.index(1, 0, 0, 0) - &ker.index(0, 0, 0, 0);
    CHECK(dp == 16 && s_row == 16 * 28 && k_row == 16 * 4 && k_gap == 16 * 4 * 3);
    de::GPU_Tensor<de::Half>& dsrc = de::CreateGPUTensorRef<de::Half>(W, H, C);
    de::GPU_TensorArray<de::Half>& dker = de::CreateGPUTensorArrayRef<de::Half>(kw, kh, C, N);
    de::GPU_Tensor<de::Half>& ddst = de::CreateGPUTensorRef<de::Half>();
    dsrc.Load_from_host(src); dker.Load_from_host(ker);
    for (int flag = 0; flag < 2; ++flag) {
        const int Ho = flag ? H : H - 2, Wo = flag ? W : W - 2;
        std::vector<double> ref((size_t)Ho * Wo * N), scale(ref.size());
        CHECK(oracle_conv2_f64_f16(reinterpret_cast<const uint16_t*>(&src.index(0, 0, 0)), H, W, (int)dp, s_row,
                                   reinterpret_cast<const uint16_t*>(&ker.index(0, 0, 0, 0)), N, kh, kw, k_gap, k_row, ref.data(),
                                   scale.data(), flag, 0) == 0);
        de::Tensor<de::Half>& host_out = de::CreateTensorRef<de::Half>();
        CHECK(de::cuda::Conv2_MK_im2col(src, ker, host_out, flag).error_type == decx::DECX_SUCCESS);
        CHECK(de::cuda::Conv2_MK_im2col(dsrc, dker, ddst, flag).error_type == decx::DECX_SUCCESS);
        CHECK(host_out.Width() == (uint)Wo && host_out.Height() == (uint)Ho && host_out.Depth() == (uint)N);
        CHECK(ddst.Width() == (uint)Wo && ddst.Height() == (uint)Ho && ddst.Depth() == (uint)N);
        de::Tensor<de::Half>& dev_out = de::CreateTensorRef<de::Half>(Wo, Ho, N, 0);
        ddst.Load_to_host(dev_out);
        double worst = 0.0;
        bool same = true;
        for (int y = 0; y < Ho; ++y) for (int x = 0; x < Wo; ++x) for (int n = 0; n < N; ++n) {
            const size_t i = ((size_t)y * Wo + x) * N + n;
            const double got = de::Half2Float(host_out.index(y, x, n));
            const double err = (std::fabs(got - ref[i]) - std::fabs(ref[i]) / 2048.0) / (scale[i] + 1e-30);   // minus the final rounding
            if (err > worst) worst = err;
            same = same && host_out.index(y, x, n).val == dev_out.index(y, x, n).val;
        }
        CHECK(worst < 2e-3);
        CHECK(same);                                   // host-tensor and device-resident flavours run the same kernel
        host_out.release(); dev_out.release();
    }
    CHECK(de::cuda::Conv2_MK_im2col(dsrc, dker, ddst, 5).error_type == decx::DECX_FAIL_ErrorFlag);
    dsrc.release(); dker.release(); ddst.release(); src.release(); ker.release();
}

static void conv_flavours_and_flags() {
    conv_case(20, 22, 8, 6, 3, 3, decx::de_conv_zero_compensate);
    conv_case(20, 22, 8, 6, 3, 3, decx::de_conv_no_compensate);
    conv_case(33, 31, 3, 7, 5, 3, decx::de_conv_zero_compensate);
    conv_case(56, 56, 64, 128, 3, 3, decx::de_conv_zero_compensate);
    de::Tensor<float>& s = de::CreateTensorRef<float>(8, 8, 4, 0);
    de::TensorArray<float>& k = de::CreateTensorArrayRef<float>(3, 3, 4, 2, 0);
    de::Tensor<float>& d = de::CreateTensorRef<float>();
    de::DH h = de::cuda::Conv2_MK_im2col(s, k, d, 7);
    CHECK(h.error_type == decx::DECX_FAIL_ErrorFlag);
    de::TensorArray<float>& k2 = de::CreateTensorArrayRef<float>(3, 3, 8, 2, 0);
    CHECK(de::cuda::Conv2_MK_im2col(s, k2, d, 1).error_type == decx::DECX_FAIL_DimsNotMatching);
}


// A result container that is one of the operands, or shares its payload with one (operator= shares: Matrix.h:510-530
// and its twins): every path must deliver the product of the operands as they were before the call.
static void results_that_alias_operands() {
    // device-resident GEMM: D = A (shared payload), square so that re_construct alone would be a no-op
    {
        const int S = 160;
        de::Matrix<float>& A = de::CreateMatrixRef<float>(S, S, 0);
        de::Matrix<float>& B = de::CreateMatrixRef<float>(S, S, 0);
        de::Matrix<float>& R = de::CreateMatrixRef<float>(S, S, 0);
        fill(A, unif); fill(B, unif);
        const std::vector<float> want = chain(A, B);
        de::GPU_Matrix<float>& dA = de::CreateGPUMatrixRef<float>(S, S);
        de::GPU_Matrix<float>& dB = de::CreateGPUMatrixRef<float>(S, S);
        de::GPU_Matrix<float>& dD = de::CreateGPUMatrixRef<float>();
        dA.Load_from_host(A); dB.Load_from_host(B);
        dD = dA;                                                       // shares A's device block
        CHECK(de::cuda::GEMM(dA, dB, dD).error_type == decx::DECX_SUCCESS);
        dD.Load_to_host(R);
        CHECK(dense(R) == want);
        dA.Load_to_host(R);
        CHECK(dense(R) == dense(A));                                   // A itself is untouched
        CHECK(de::cuda::GEMM(dA, dB, dA).error_type == decx::DECX_SUCCESS);      // dst IS A
        dA.Load_to_host(R);
        CHECK(dense(R) == want);
        dA.Load_from_host(A);
        CHECK(de::cuda::GEMM(dA, dB, dB).error_type == decx::DECX_SUCCESS);      // dst IS B
        dB.Load_to_host(R);
        CHECK(dense(R) == want);
    }
    // GEMM3 over arrays: dst shares A's payload, and dst is B
    {
        const int S = 96, NUM = 3;
        de::MatrixArray<float>& A = de::CreateMatrixArrayRef<float>(S, S, NUM, 0);
        de::MatrixArray<float>& B = de::CreateMatrixArrayRef<float>(S, S, NUM, 0);
        de::MatrixArray<float>& D = de::CreateMatrixArrayRef<float>();
        for (int s = 0; s < NUM; ++s)
            for (int i = 0; i < S; ++i) for (int j = 0; j < S; ++j) { A.index(i, j, s) = small_int(); B.index(i, j, s) = small_int(); }
        std::vector<std::vector<float>> want(NUM);
        for (int s = 0; s < NUM; ++s) {
            want[s].resize((size_t)S * S);
            oracle_sgemm_chain_fast(&A.index(0, 0, s), S, &B.index(0, 0, s), S, nullptr, 0, want[s].data(), S, S, S, S, 0);
        }
        auto same_as_want = [&](de::MatrixArray<float>& R) {
            bool same = R.Width() == (uint)S && R.Height() == (uint)S && R.MatrixNumber() == (uint)NUM;
            for (int s = 0; s < NUM && same; ++s)
                for (int i = 0; i < S; ++i) for (int j = 0; j < S; ++j) same = same && R.index(i, j, s) == want[s][(size_t)i * S + j];
            return same;
        };
        D = A;
        const float a00 = A.index(0, 0, 0);
        CHECK(de::cuda::GEMM3(A, B, D).error_type == decx::DECX_SUCCESS);
        CHECK(same_as_want(D));
        CHECK(A.index(0, 0, 0) == a00 && &A.index(0, 0, 0) != &D.index(0, 0, 0));   // A kept its payload, D has a new one
        CHECK(de::cuda::GEMM3(A, B, B).error_type == decx::DECX_SUCCESS);
        CHECK(same_as_want(B));
    }
    // convolution on host tensors with dst == src: as many filters as channels (same shape), and a different count
    for (int N : {8, 5, 12}) {
        const int H = 14, W = 12, C = 8, kh = 3, kw = 3;
        de::Tensor<float>& src = de::CreateTensorRef<float>(W, H, C, 0);
        de::Tensor<float>& copy = de::CreateTensorRef<float>(W, H, C, 0);
        de::TensorArray<float>& ker = de::CreateTensorArrayRef<float>(kw, kh, C, N, 0);
        de::Tensor<float>& want = de::CreateTensorRef<float>();
        for (int y = 0; y < H; ++y) for (int x = 0; x < W; ++x) for (int c = 0; c < C; ++c) copy.index(y, x, c) = src.index(y, x, c) = small_int();
        for (int n = 0; n < N; ++n) for (int i = 0; i < kh; ++i) for (int j = 0; j < kw; ++j) for (int c = 0; c < C; ++c) ker.index(i, j, c, n) = small_int();
        CHECK(de::cuda::Conv2_MK_im2col(copy, ker, want, 1).error_type == decx::DECX_SUCCESS);
        CHECK(de::cuda::Conv2_MK_im2col(src, ker, src, 1).error_type == decx::DECX_SUCCESS);
        bool same = src.Depth() == (uint)N && src.Width() == (uint)W && src.Height() == (uint)H;
        for (int y = 0; y < H && same; ++y) for (int x = 0; x < W; ++x) for (int n = 0; n < N; ++n) same = same && src.index(y, x, n) == want.index(y, x, n);
        CHECK(same);
        // device-resident tensors: dst shares src's block
        de::GPU_Tensor<float>& dsrc = de::CreateGPUTensorRef<float>(W, H, C);
        de::GPU_TensorArray<float>& dker = de::CreateGPUTensorArrayRef<float>(kw, kh, C, N);
        de::GPU_Tensor<float>& ddst = de::CreateGPUTensorRef<float>();
        dsrc.Load_from_host(copy); dker.Load_from_host(ker);
        ddst = dsrc;
        CHECK(de::cuda::Conv2_MK_im2col(dsrc, dker, ddst, 1).error_type == decx::DECX_SUCCESS);
        de::Tensor<float>& got = de::CreateTensorRef<float>(W, H, N, 0);
        ddst.Load_to_host(got);
        same = ddst.Depth() == (uint)N;
        for (int y = 0; y < H && same; ++y) for (int x = 0; x < W; ++x) for (int n = 0; n < N; ++n) same = same && got.index(y, x, n) == want.index(y, x, n);
        CHECK(same);
        CHECK(de::cuda::Conv2_MK_im2col(dsrc, dker, dsrc, 1).error_type == decx::DECX_SUCCESS);   // dst IS src
        de::Tensor<float>& got2 = de::CreateTensorRef<float>(W, H, N, 0);
        dsrc.Load_to_host(got2);
        same = dsrc.Depth() == (uint)N;
        for (int y = 0; y < H && same; ++y) for (int x = 0; x < W; ++x) for (int n = 0; n < N; ++n) same = same && got2.index(y, x, n) == want.index(y, x, n);
        CHECK(same);
        src.release(); copy.release(); ker.release(); want.release(); got.release(); got2.release(); dsrc.release(); dker.release(); ddst.release();
    }
}

// What a caller of the synchronous C++ API sees on kernels of tens of microseconds (mode "timing", not a test): whole
// calls of de::cuda::Conv2_MK_im2col on device-resident tensors at 224x224x64 under 128 filters of 3x3x64, and of
// de::cuda::GEMM on device-resident 1024^3 matrices.
static void blocking_call_timing() {
    auto report = [](const char* what, std::vector<double>& us) {
        std::sort(us.begin(), us.end());
        std::printf("%-56s min %8.2f us  median %8.2f us\n", what, us.front(), us[us.size() / 2]);
    };
    {
        de::GPU_Tensor<float>& s = de::CreateGPUTensorRef<float>(224, 224, 64);
        de::GPU_TensorArray<float>& k = de::CreateGPUTensorArrayRef<float>(3, 3, 64, 128);
        de::GPU_Tensor<float>& d = de::CreateGPUTensorRef<float>(224, 224, 128);
        std::vector<double> us;
        for (int i = 0; i < 700; ++i) {
            const auto t0 = std::chrono::steady_clock::now();
            de::cuda::Conv2_MK_im2col(s, k, d, 1);
            if (i >= 200) us.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
        }
        report("Conv2_MK_im2col(GPU_Tensor) 224x224x64, 128 x 3x3x64", us);
    }
    {   // the reference's own convolution entry: host tensors in, host tensor out (conv2_mk_im2col.h:25)
        de::Tensor<float>& s = de::CreateTensorRef<float>(224, 224, 64, decx::Page_Locked);
        de::TensorArray<float>& k = de::CreateTensorArrayRef<float>(3, 3, 64, 128, decx::Page_Locked);
        de::Tensor<float>& d = de::CreateTensorRef<float>(224, 224, 128, decx::Page_Locked);
        std::vector<double> us;
        for (int i = 0; i < 150; ++i) {
            const auto t0 = std::chrono::steady_clock::now();
            de::cuda::Conv2_MK_im2col(s, k, d, 1);
            if (i >= 30) us.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
        }
        report("Conv2_MK_im2col(Tensor) 224x224x64, 128 x 3x3x64, host tensors", us);
    }
    {   // host matrices in, host matrix out (GEMM.h:56-131)
        de::Matrix<float>& A = de::CreateMatrixRef<float>(4096, 4096, decx::Page_Locked);
        de::Matrix<float>& B = de::CreateMatrixRef<float>(4096, 4096, decx::Page_Locked);
        de::Matrix<float>& D = de::CreateMatrixRef<float>(4096, 4096, decx::Page_Locked);
        std::vector<double> us;
        for (int i = 0; i < 24; ++i) {
            const auto t0 = std::chrono::steady_clock::now();
            de::cuda::GEMM(A, B, D);
            if (i >= 4) us.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
        }
        report("GEMM(Matrix<float>) 4096^3, host matrices", us);
    }
    {
        de::GPU_Matrix<float>& A = de::CreateGPUMatrixRef<float>(1024, 1024);
        de::GPU_Matrix<float>& B = de::CreateGPUMatrixRef<float>(1024, 1024);
        de::GPU_Matrix<float>& D = de::CreateGPUMatrixRef<float>(1024, 1024);
        std::vector<double> us;
        for (int i = 0; i < 1500; ++i) {
            const auto t0 = std::chrono::steady_clock::now();
            de::cuda::GEMM(A, B, D);
            if (i >= 500) us.push_back(std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count());
        }
        report("GEMM(GPU_Matrix<float>) 1024^3", us);
    }
}

int main(int argc, char** argv) {
    std::string mode = argc > 1 ? argv[1] : "cpu";
    if (mode == "cpu" || mode == "cpu-small") {
        g_small = mode == "cpu-small";
        RUN(oracle_thread_pool_sgemm);
        RUN(containers_follow_reference_pitch_rules);
        RUN(assignment_shares_the_payload);
        RUN(cpu_sgemm_into_an_operand);
        RUN(half_conversion);
        RUN(gemm_refuses_before_init);
        RUN(cpu_sgemm_matches_chain_bit_for_bit);
    } else if (mode == "timing") {
        de::InitCuda();
        blocking_call_timing();
    } else {
        de::InitCuda();
        RUN(reference_demo_known_answer);
        RUN(gemm_fp32_all_flavours);
        RUN(gemm_fp16_flavours);
        RUN(conv_flavours_and_flags);
        RUN(conv_device_resident);
        RUN(conv_half_containers);
        RUN(gemm3_matrix_arrays);
        RUN(gemm_long_lr);
        RUN(nn_relu_family);
        RUN(results_that_alias_operands);
    }
    std::printf("%s: %d failure(s)\n", mode.c_str(), g_fail);
    return g_fail ? 1 : 0;
}
