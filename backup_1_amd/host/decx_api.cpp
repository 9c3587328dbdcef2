// DECX-named API functions over the C ABI (include/decx_hip.h).  Reference call stacks mirrored here:
//   host-matrix GEMM      GEMM/CUDA/large_squares/GEMM.h:56-131   (re_construct dst, H2D, kernel, D2H)
//   GPU_Matrix GEMM       GEMM.h:398-454 (fp32), :457-519 (fp16)
//   Conv2_MK_im2col       convolution/CUDA/im2col/conv2_mk_im2col.h:278-306 (+ :57-274 host drivers)
// Differences on purpose: device copies keep the host pitch (no padding to 128/16 multiples, GEMM.h:80-104 pads);
// errors of the GPU runtime come back in the DH instead of exiting the process; Conv2_MK_im2col fills its DH and
// rejects unknown flags (the reference returns an unfilled DH, conv2_mk_im2col.h:301-305).
#include <cmath>
#include <cstring>

#include "decx_classes.hpp"

namespace {

char kSuccess[] = "No error\n";                                              // core/error.h:61
char kGemmDims[] = "The width of matrix A and the height of matrix B are required to be same";   // core/error.h GEMM_DimNMatch
char kMDims[] = "Matrix Dims don't match each other";
char kNotFactory[] = "Container was not created by this library's factories\n";

de::DH ok() { return de::DH{decx::DECX_SUCCESS, kSuccess}; }
de::DH from_status(int rc) {
    if (rc == 0) return ok();
    return de::DH{rc, const_cast<char*>(decx_hip_last_error())};
}
de::DH not_init() {
    static char msg[] = "CUDA should be initialized first\n";               // core/error.h:60
    return de::DH{decx::DECX_FAIL_not_init, msg};
}
de::DH alloc_fail() {
    static char msg[] = "Fail to allocate memory\n";                          // core/error.h:65
    return de::DH{decx::DECX_FAIL_ALLOCATION, msg};
}

struct DeviceTemp {   // a device block from the library's pool of temporaries, given back to it on scope exit
    void* ptr = nullptr;
    int alloc(size_t bytes) { return decx_hip_tmp_malloc(&ptr, bytes); }
    ~DeviceTemp() { if (ptr) decx_hip_tmp_free(ptr); }
};

template <typename T> struct GemmCall;
template <> struct GemmCall<float> {
    static int run(const float* A, int lda, const float* B, int ldb, const float* C, int ldc, float* D, int ldd, int M,
                   int N, int K) { return decx_hip_sgemm(A, lda, B, ldb, C, ldc, D, ldd, M, N, K); }
};
template <> struct GemmCall<de::Half> {
    static int run(const de::Half* A, int lda, const de::Half* B, int ldb, const de::Half* C, int ldc, de::Half* D, int ldd,
                   int M, int N, int K) {
        return decx_hip_hgemm_f32acc(reinterpret_cast<const uint16_t*>(A), lda, reinterpret_cast<const uint16_t*>(B), ldb,
                                     reinterpret_cast<const uint16_t*>(C), ldc, reinterpret_cast<uint16_t*>(D), ldd, M, N, K);
    }
};

template <typename T> struct HostGemmCall;
template <> struct HostGemmCall<float> {
    static int run(const float* A, int lda, const float* B, int ldb, const float* C, int ldc, float* D, int ldd, int M,
                   int N, int K) { return decx_hip_gemm_host_f32(A, lda, B, ldb, C, ldc, D, ldd, M, N, K); }
};
template <> struct HostGemmCall<de::Half> {
    static int run(const de::Half* A, int lda, const de::Half* B, int ldb, const de::Half* C, int ldc, de::Half* D, int ldd,
                   int M, int N, int K) {
        return decx_hip_gemm_host_f16(reinterpret_cast<const uint16_t*>(A), lda, reinterpret_cast<const uint16_t*>(B), ldb,
                                      reinterpret_cast<const uint16_t*>(C), ldc, reinterpret_cast<uint16_t*>(D), ldd, M, N, K);
    }
};

template <typename T>
de::DH gemm_host(de::Matrix<T>& A_, de::Matrix<T>& B_, de::Matrix<T>* C_, de::Matrix<T>& dst_) {
    auto* A = dynamic_cast<decx::_Matrix<T>*>(&A_);
    auto* B = dynamic_cast<decx::_Matrix<T>*>(&B_);
    auto* C = C_ ? dynamic_cast<decx::_Matrix<T>*>(C_) : nullptr;
    auto* dst = dynamic_cast<decx::_Matrix<T>*>(&dst_);
    if (!A || !B || !dst || (C_ && !C)) return de::DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    if (!decx_hip_is_init()) return not_init();                                           // GEMM.h:63
    if (A->width != B->height) return de::DH{decx::DECX_FAIL_DimsNotMatching, kGemmDims}; // GEMM.h:68
    if (C && (C->width != B->width || C->height != A->height))                            // GEMM.h:154-157
        return de::DH{decx::DECX_FAIL_DimsNotMatching, kMDims};
    const int M = (int)A->height, K = (int)A->width, N = (int)B->width;
    // dst takes its size from the operands (GEMM.h:73).  The pipeline below downloads finished regions of dst while
    // later panels of A and B are still being uploaded, so a dst that is (or shares its payload with) A or B is
    // computed into a fresh matrix whose payload dst then takes over; a dst that shares C's payload is used in
    // place whatever its store type (C is read and dst written region by region, in that order), since
    // re_construct with another store type would free C's data before it is uploaded.
    const bool over_operand = dst == A || dst == B || dst->shares_block_with(*A) || dst->shares_block_with(*B);
    const bool over_c = C && (dst == C || dst->shares_block_with(*C));
    decx::_Matrix<T> fresh;
    decx::_Matrix<T>* out = dst;
    if (over_operand) {
        if (!fresh.construct((uint)N, (uint)M, decx::Page_Locked)) return alloc_fail();
        out = &fresh;
    } else if (over_c) {
        if (dst->width != (uint)N || dst->height != (uint)M || !dst->Mat.ptr) return de::DH{decx::DECX_FAIL_DimsNotMatching, kMDims};
    } else if (!dst->re_construct((uint)N, (uint)M, decx::Page_Locked)) {
        return alloc_fail();
    }
    // allocation, uploads, kernel and download, pipelined over row panels, all below the C ABI
    const int rc = HostGemmCall<T>::run(A->Mat.ptr, (int)A->pitch, B->Mat.ptr, (int)B->pitch, C ? C->Mat.ptr : nullptr,
                                        C ? (int)C->pitch : 0, out->Mat.ptr, (int)out->pitch, M, N, K);
    if (rc == 0 && out != dst) dst->share_from(fresh);   // dst now shares the fresh payload; the operand it stood for keeps its own
    return from_status(rc);
}

template <typename T>
de::DH gemm_device(de::GPU_Matrix<T>& A_, de::GPU_Matrix<T>& B_, de::GPU_Matrix<T>* C_, de::GPU_Matrix<T>& dst_) {
    auto* A = dynamic_cast<decx::_GPU_Matrix<T>*>(&A_);
    auto* B = dynamic_cast<decx::_GPU_Matrix<T>*>(&B_);
    auto* C = C_ ? dynamic_cast<decx::_GPU_Matrix<T>*>(C_) : nullptr;
    auto* dst = dynamic_cast<decx::_GPU_Matrix<T>*>(&dst_);
    if (!A || !B || !dst || (C_ && !C)) return de::DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    if (!decx_hip_is_init()) return not_init();                                           // GEMM.h:403
    if (A->width != B->height) return de::DH{decx::DECX_FAIL_DimsNotMatching, kGemmDims}; // GEMM.h:408
    if (C && (C->width != B->width || C->height != A->height)) return de::DH{decx::DECX_FAIL_DimsNotMatching, kMDims};
    // A dst that is A or B, or shares its payload with one of them (operator= shares, GPU_Matrix.h:441-451), would be
    // written by some workgroups while others still read it: such a product goes into a fresh matrix whose payload dst
    // then takes over.  A dst that is C, or shares C's payload, is used in place (each element of C is read by the
    // workgroup that writes it, before it writes it).
    const bool over_operand = dst == A || dst == B || dst->shares_block_with(*A) || dst->shares_block_with(*B);
    const bool over_c = C && (dst == C || dst->shares_block_with(*C));
    decx::_GPU_Matrix<T> fresh;
    decx::_GPU_Matrix<T>* out = dst;
    if (over_operand) {
        if (!fresh.construct(B->width, A->height))
            return fresh.last_status == DECX_HIP_FAIL_ALLOCATION ? alloc_fail() : from_status(fresh.last_status);
        out = &fresh;
    } else if (over_c) {
        if (dst->width != B->width || dst->height != A->height || !dst->Mat.ptr) return de::DH{decx::DECX_FAIL_DimsNotMatching, kMDims};
    } else if (!dst->re_construct(B->width, A->height)) {                                 // GEMM.h:414 (fp16 too: defect D7 not kept)
        return dst->last_status == DECX_HIP_FAIL_ALLOCATION ? alloc_fail() : from_status(dst->last_status);
    }
    const int rc = GemmCall<T>::run(A->Mat.ptr, (int)A->pitch, B->Mat.ptr, (int)B->pitch, C ? C->Mat.ptr : nullptr,
                                    C ? (int)C->pitch : 0, out->Mat.ptr, (int)out->pitch, (int)A->height, (int)B->width,
                                    (int)A->width);
    if (rc == 0 && out != dst) dst->share_from(fresh);
    return from_status(rc);
}

template <typename T> struct Gemm3Call;
template <> struct Gemm3Call<float> {
    static int run(const float* A, int lda, size_t pa, const float* B, int ldb, size_t pb, const float* C, int ldc, size_t pc,
                   float* D, int ldd, size_t pd, int M, int N, int K, int n) {
        return decx_hip_gemm3_host_f32(A, lda, pa, B, ldb, pb, C, ldc, pc, D, ldd, pd, M, N, K, n);
    }
};
template <> struct Gemm3Call<de::Half> {
    static int run(const de::Half* A, int lda, size_t pa, const de::Half* B, int ldb, size_t pb, const de::Half* C, int ldc,
                   size_t pc, de::Half* D, int ldd, size_t pd, int M, int N, int K, int n) {
        return decx_hip_gemm3_host_f16(reinterpret_cast<const uint16_t*>(A), lda, pa, reinterpret_cast<const uint16_t*>(B), ldb, pb,
                                       reinterpret_cast<const uint16_t*>(C), ldc, pc, reinterpret_cast<uint16_t*>(D), ldd, pd, M,
                                       N, K, n);
    }
};

template <typename T>
de::DH gemm3_host(de::MatrixArray<T>& A_, de::MatrixArray<T>& B_, de::MatrixArray<T>* C_, de::MatrixArray<T>& dst_) {
    auto* A = dynamic_cast<decx::_MatrixArray<T>*>(&A_);
    auto* B = dynamic_cast<decx::_MatrixArray<T>*>(&B_);
    auto* C = C_ ? dynamic_cast<decx::_MatrixArray<T>*>(C_) : nullptr;
    auto* dst = dynamic_cast<decx::_MatrixArray<T>*>(&dst_);
    if (!A || !B || !dst || (C_ && !C)) return de::DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    if (!decx_hip_is_init()) return not_init();                                           // GEMM3.h:42-46
    if (A->width != B->height) return de::DH{decx::DECX_FAIL_DimsNotMatching, kGemmDims};
    static char num_msg[] = "The number of matrices don't match each other";             // core/error.h Matrix_number_not_matching
    if (A->ArrayNumber != B->ArrayNumber || (C && C->ArrayNumber != A->ArrayNumber))
        return de::DH{decx::DECX_FAIL_MNumNotMatching, num_msg};
    if (C && (C->width != B->width || C->height != A->height)) return de::DH{decx::DECX_FAIL_DimsNotMatching, kMDims};
    // the pipeline downloads result i-1 while matrix i+1 is uploaded: a dst that is (or shares its payload with) A or B
    // is computed into a fresh array that dst then takes over; one that shares C's is used in place (as gemm_host)
    const bool over_operand = dst == A || dst == B || dst->shares_block_with(*A) || dst->shares_block_with(*B);
    const bool over_c = C && (dst == C || dst->shares_block_with(*C));
    decx::_MatrixArray<T> fresh;
    decx::_MatrixArray<T>* out = dst;
    if (over_operand) {
        if (!fresh.construct(B->width, A->height, (uint)A->ArrayNumber, decx::Page_Locked)) return alloc_fail();
        out = &fresh;
    } else if (over_c) {
        if (dst->width != B->width || dst->height != A->height || dst->ArrayNumber != A->ArrayNumber || !dst->MatArr.ptr)
            return de::DH{decx::DECX_FAIL_DimsNotMatching, kMDims};
    } else if (!dst->re_construct(B->width, A->height, (uint)A->ArrayNumber, decx::Page_Locked)) {
        return alloc_fail();
    }
    const int rc = Gemm3Call<T>::run(A->MatArr.ptr, (int)A->pitch, A->_plane, B->MatArr.ptr, (int)B->pitch, B->_plane,
                                     C ? C->MatArr.ptr : nullptr, C ? (int)C->pitch : 0, C ? C->_plane : 0, out->MatArr.ptr,
                                     (int)out->pitch, out->_plane, (int)A->height, (int)B->width, (int)A->width,
                                     (int)A->ArrayNumber);
    if (rc == 0 && out != dst) dst->share_from(fresh);
    return from_status(rc);
}

}  // namespace

namespace de {

void InitCuda() {
    int dev = -1;
    (void)decx_hip_init(&dev);   // failures surface as DECX_FAIL_not_init on the first compute call
}
// Memory_pool.h:23-37: gives back what the pools hold; here the device blocks the host-matrix pipelines keep
void release_all_tmp() { (void)decx_hip_release_tmp(); }

// IEEE binary32 -> binary16, round to nearest even
Half Float2Half(const float& x) {
    uint32_t u;
    std::memcpy(&u, &x, 4);
    const uint32_t sign = (u >> 16) & 0x8000u, mag = u & 0x7fffffffu;
    Half h;
    if (mag > 0x7f800000u) { h.val = (unsigned short)(sign | 0x7e00u); return h; }           // NaN
    if (mag >= 0x477ff000u) { h.val = (unsigned short)(sign | 0x7c00u); return h; }          // overflow to inf
    if (mag < 0x33000001u) { h.val = (unsigned short)sign; return h; }                       // underflow to zero
    const int e = (int)(mag >> 23) - 127;
    const uint32_t man = (mag & 0x7fffffu) | 0x800000u;
    const int shift = e >= -14 ? 13 : 13 + (-14 - e);
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    h.val = (unsigned short)(sign | (e >= -14 ? ((uint32_t)(e + 14) << 10) + q : q));
    return h;
}
float Half2Float(const Half& x) {
    const uint32_t sign = (uint32_t)(x.val & 0x8000u) << 16, e = (x.val >> 10) & 0x1fu;
    uint32_t m = x.val & 0x3ffu, u;
    if (e == 0) {
        if (m == 0) u = sign;
        else {
            int s = 0;
            while (!(m & 0x400u)) { m <<= 1; ++s; }
            u = sign | (uint32_t)(113 - s) << 23 | (m & 0x3ffu) << 13;
        }
    } else if (e == 31) u = sign | 0x7f800000u | m << 13;
    else u = sign | (e + 112u) << 23 | m << 13;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// ---- factories ----------------------------------------------------------------------------------------------
template <typename T> Matrix<T>& CreateMatrixRef() { return *(new decx::_Matrix<T>()); }
template <typename T> Matrix<T>* CreateMatrixPtr() { return new decx::_Matrix<T>(); }
template <typename T> Matrix<T>& CreateMatrixRef(const uint w, const uint h, const int st) { return *(new decx::_Matrix<T>(w, h, st)); }
template <typename T> Matrix<T>* CreateMatrixPtr(const uint w, const uint h, const int st) { return new decx::_Matrix<T>(w, h, st); }
template <typename T> GPU_Matrix<T>& CreateGPUMatrixRef() { return *(new decx::_GPU_Matrix<T>()); }
template <typename T> GPU_Matrix<T>* CreateGPUMatrixPtr() { return new decx::_GPU_Matrix<T>(); }
template <typename T> GPU_Matrix<T>& CreateGPUMatrixRef(const uint w, const uint h) { return *(new decx::_GPU_Matrix<T>(w, h)); }
template <typename T> GPU_Matrix<T>* CreateGPUMatrixPtr(const uint w, const uint h) { return new decx::_GPU_Matrix<T>(w, h); }
template <typename T> Tensor<T>& CreateTensorRef() { return *(new decx::_Tensor<T>()); }
template <typename T> Tensor<T>* CreateTensorPtr() { return new decx::_Tensor<T>(); }
template <typename T> Tensor<T>& CreateTensorRef(const uint w, const uint h, const uint d, const int f) { return *(new decx::_Tensor<T>(w, h, d, f)); }
template <typename T> Tensor<T>* CreateTensorPtr(const uint w, const uint h, const uint d, const int f) { return new decx::_Tensor<T>(w, h, d, f); }
template <typename T> TensorArray<T>& CreateTensorArrayRef() { return *(new decx::_TensorArray<T>()); }
template <typename T> TensorArray<T>* CreateTensorArrayPtr() { return new decx::_TensorArray<T>(); }
template <typename T> TensorArray<T>& CreateTensorArrayRef(const uint w, const uint h, const uint d, const uint n, const int f) { return *(new decx::_TensorArray<T>(w, h, d, n, f)); }
template <typename T> TensorArray<T>* CreateTensorArrayPtr(const uint w, const uint h, const uint d, const uint n, const int f) { return new decx::_TensorArray<T>(w, h, d, n, f); }

template <typename T> GPU_Tensor<T>& CreateGPUTensorRef() { return *(new decx::_GPU_Tensor<T>()); }
template <typename T> GPU_Tensor<T>* CreateGPUTensorPtr() { return new decx::_GPU_Tensor<T>(); }
template <typename T> GPU_Tensor<T>& CreateGPUTensorRef(const uint w, const uint h, const uint d) { return *(new decx::_GPU_Tensor<T>(w, h, d)); }
template <typename T> GPU_Tensor<T>* CreateGPUTensorPtr(const uint w, const uint h, const uint d) { return new decx::_GPU_Tensor<T>(w, h, d); }
template <typename T> GPU_TensorArray<T>& CreateGPUTensorArrayRef() { return *(new decx::_GPU_TensorArray<T>()); }
template <typename T> GPU_TensorArray<T>* CreateGPUTensorArrayPtr() { return new decx::_GPU_TensorArray<T>(); }
template <typename T> GPU_TensorArray<T>& CreateGPUTensorArrayRef(const uint w, const uint h, const uint d, const uint n) { return *(new decx::_GPU_TensorArray<T>(w, h, d, n)); }
template <typename T> GPU_TensorArray<T>* CreateGPUTensorArrayPtr(const uint w, const uint h, const uint d, const uint n) { return new decx::_GPU_TensorArray<T>(w, h, d, n); }
template <typename T> MatrixArray<T>& CreateMatrixArrayRef() { return *(new decx::_MatrixArray<T>()); }
template <typename T> MatrixArray<T>* CreateMatrixArrayPtr() { return new decx::_MatrixArray<T>(); }
template <typename T> MatrixArray<T>& CreateMatrixArrayRef(uint w, uint h, uint n, const int f) { return *(new decx::_MatrixArray<T>(w, h, n, f)); }
template <typename T> MatrixArray<T>* CreateMatrixArrayPtr(uint w, uint h, uint n, const int f) { return new decx::_MatrixArray<T>(w, h, n, f); }
template MatrixArray<float>& CreateMatrixArrayRef<float>();
template MatrixArray<float>* CreateMatrixArrayPtr<float>();
template MatrixArray<float>& CreateMatrixArrayRef<float>(uint, uint, uint, const int);
template MatrixArray<float>* CreateMatrixArrayPtr<float>(uint, uint, uint, const int);
template MatrixArray<Half>& CreateMatrixArrayRef<Half>();
template MatrixArray<Half>* CreateMatrixArrayPtr<Half>();
template MatrixArray<Half>& CreateMatrixArrayRef<Half>(uint, uint, uint, const int);
template MatrixArray<Half>* CreateMatrixArrayPtr<Half>(uint, uint, uint, const int);
template GPU_Tensor<float>& CreateGPUTensorRef<float>();
template GPU_Tensor<Half>& CreateGPUTensorRef<Half>();
template GPU_Tensor<float>* CreateGPUTensorPtr<float>();
template GPU_Tensor<Half>* CreateGPUTensorPtr<Half>();
template GPU_Tensor<float>& CreateGPUTensorRef<float>(const uint, const uint, const uint);
template GPU_Tensor<Half>& CreateGPUTensorRef<Half>(const uint, const uint, const uint);
template GPU_Tensor<float>* CreateGPUTensorPtr<float>(const uint, const uint, const uint);
template GPU_Tensor<Half>* CreateGPUTensorPtr<Half>(const uint, const uint, const uint);
template GPU_TensorArray<float>& CreateGPUTensorArrayRef<float>();
template GPU_TensorArray<Half>& CreateGPUTensorArrayRef<Half>();
template GPU_TensorArray<float>* CreateGPUTensorArrayPtr<float>();
template GPU_TensorArray<Half>* CreateGPUTensorArrayPtr<Half>();
template GPU_TensorArray<float>& CreateGPUTensorArrayRef<float>(const uint, const uint, const uint, const uint);
template GPU_TensorArray<Half>& CreateGPUTensorArrayRef<Half>(const uint, const uint, const uint, const uint);
template GPU_TensorArray<float>* CreateGPUTensorArrayPtr<float>(const uint, const uint, const uint, const uint);
template GPU_TensorArray<Half>* CreateGPUTensorArrayPtr<Half>(const uint, const uint, const uint, const uint);

#define DECX_INSTANTIATE_MATRIX(T)                                                     \
    template Matrix<T>& CreateMatrixRef<T>();                                          \
    template Matrix<T>* CreateMatrixPtr<T>();                                          \
    template Matrix<T>& CreateMatrixRef<T>(const uint, const uint, const int);         \
    template Matrix<T>* CreateMatrixPtr<T>(const uint, const uint, const int);         \
    template GPU_Matrix<T>& CreateGPUMatrixRef<T>();                                   \
    template GPU_Matrix<T>* CreateGPUMatrixPtr<T>();                                   \
    template GPU_Matrix<T>& CreateGPUMatrixRef<T>(const uint, const uint);             \
    template GPU_Matrix<T>* CreateGPUMatrixPtr<T>(const uint, const uint);
DECX_INSTANTIATE_MATRIX(float)
DECX_INSTANTIATE_MATRIX(Half)
DECX_INSTANTIATE_MATRIX(uchar)
template Tensor<float>& CreateTensorRef<float>();
template Tensor<Half>& CreateTensorRef<Half>();
template Tensor<float>* CreateTensorPtr<float>();
template Tensor<Half>* CreateTensorPtr<Half>();
template Tensor<float>& CreateTensorRef<float>(const uint, const uint, const uint, const int);
template Tensor<Half>& CreateTensorRef<Half>(const uint, const uint, const uint, const int);
template Tensor<float>* CreateTensorPtr<float>(const uint, const uint, const uint, const int);
template Tensor<Half>* CreateTensorPtr<Half>(const uint, const uint, const uint, const int);
template TensorArray<float>& CreateTensorArrayRef<float>();
template TensorArray<Half>& CreateTensorArrayRef<Half>();
template TensorArray<float>* CreateTensorArrayPtr<float>();
template TensorArray<Half>* CreateTensorArrayPtr<Half>();
template TensorArray<float>& CreateTensorArrayRef<float>(const uint, const uint, const uint, const uint, const int);
template TensorArray<Half>& CreateTensorArrayRef<Half>(const uint, const uint, const uint, const uint, const int);
template TensorArray<float>* CreateTensorArrayPtr<float>(const uint, const uint, const uint, const uint, const int);
template TensorArray<Half>* CreateTensorArrayPtr<Half>(const uint, const uint, const uint, const uint, const int);

// ---- GEMM ---------------------------------------------------------------------------------------------------
namespace cuda {
DH GEMM(Matrix<float>& A, Matrix<float>& B, Matrix<float>& dst) { return gemm_host<float>(A, B, nullptr, dst); }
DH GEMM(Matrix<float>& A, Matrix<float>& B, Matrix<float>& C, Matrix<float>& dst) { return gemm_host<float>(A, B, &C, dst); }
DH GEMM(Matrix<Half>& A, Matrix<Half>& B, Matrix<Half>& dst) { return gemm_host<Half>(A, B, nullptr, dst); }
DH GEMM(Matrix<Half>& A, Matrix<Half>& B, Matrix<Half>& C, Matrix<Half>& dst) { return gemm_host<Half>(A, B, &C, dst); }
DH GEMM(GPU_Matrix<float>& A, GPU_Matrix<float>& B, GPU_Matrix<float>& dst) { return gemm_device<float>(A, B, nullptr, dst); }
DH GEMM(GPU_Matrix<float>& A, GPU_Matrix<float>& B, GPU_Matrix<float>& C, GPU_Matrix<float>& dst) { return gemm_device<float>(A, B, &C, dst); }
DH GEMM(GPU_Matrix<Half>& A, GPU_Matrix<Half>& B, GPU_Matrix<Half>& dst) { return gemm_device<Half>(A, B, nullptr, dst); }
DH GEMM(GPU_Matrix<Half>& A, GPU_Matrix<Half>& B, GPU_Matrix<Half>& C, GPU_Matrix<Half>& dst) { return gemm_device<Half>(A, B, &C, dst); }

DH GEMM_Long_Lr(GPU_Matrix<float>& A_, GPU_Matrix<float>& B_, GPU_Matrix<float>& dst_) {
    auto* A = dynamic_cast<decx::_GPU_Matrix<float>*>(&A_);
    auto* B = dynamic_cast<decx::_GPU_Matrix<float>*>(&B_);
    auto* dst = dynamic_cast<decx::_GPU_Matrix<float>*>(&dst_);
    if (!A || !B || !dst) return DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    if (!decx_hip_is_init()) return not_init();
    if (A->width != B->height) return DH{decx::DECX_FAIL_DimsNotMatching, kGemmDims};
    if (!dst->re_construct(B->width, A->height))
        return dst->last_status == DECX_HIP_FAIL_ALLOCATION ? alloc_fail() : from_status(dst->last_status);
    // the reference's long-K kernel is one fused chain per output like every other (GEMM_long_linear_region.cuh:35-55):
    // decx_hip_sgemm follows it bit for bit and sends results this small to its one-wave-per-block kernel
    return from_status(decx_hip_sgemm(A->Mat.ptr, (int)A->pitch, B->Mat.ptr, (int)B->pitch, nullptr, 0, dst->Mat.ptr,
                                      (int)dst->pitch, (int)A->height, (int)B->width, (int)A->width));
}

DH GEMM3(MatrixArray<float>& A, MatrixArray<float>& B, MatrixArray<float>& dst) { return gemm3_host<float>(A, B, nullptr, dst); }
DH GEMM3(MatrixArray<Half>& A, MatrixArray<Half>& B, MatrixArray<Half>& dst) { return gemm3_host<Half>(A, B, nullptr, dst); }
DH GEMM3(MatrixArray<float>& A, MatrixArray<float>& B, MatrixArray<float>& C, MatrixArray<float>& dst) { return gemm3_host<float>(A, B, &C, dst); }
DH GEMM3(MatrixArray<Half>& A, MatrixArray<Half>& B, MatrixArray<Half>& C, MatrixArray<Half>& dst) { return gemm3_host<Half>(A, B, &C, dst); }

// ---- convolution ----------------------------------------------------------------------------------------------
namespace {
template <typename T> struct ConvCall;
template <> struct ConvCall<float> {
    static int run(const float* src, int H, int W, int dpitch, size_t src_row, const float* filt, int N, int kh, int kw,
                   size_t filt_stride, size_t filt_row, float* dst, int dst_dpitch, size_t dst_row, int flag) {
        return decx_hip_conv2_im2col_f32(src, H, W, dpitch, src_row, filt, N, kh, kw, filt_stride, filt_row, dst, dst_dpitch,
                                         dst_row, flag);
    }
};
template <> struct ConvCall<Half> {
    static int run(const Half* src, int H, int W, int dpitch, size_t src_row, const Half* filt, int N, int kh, int kw,
                   size_t filt_stride, size_t filt_row, Half* dst, int dst_dpitch, size_t dst_row, int flag) {
        return decx_hip_conv2_im2col_f16(reinterpret_cast<const uint16_t*>(src), H, W, dpitch, src_row,
                                         reinterpret_cast<const uint16_t*>(filt), N, kh, kw, filt_stride, filt_row,
                                         reinterpret_cast<uint16_t*>(dst), dst_dpitch, dst_row, flag, nullptr, 0);
    }
};

// what both container flavours check before anything is allocated (conv2_mk_im2col.h:285-289, :63-66, :173-176)
DH conv_precheck(uint src_depth, uint ker_depth, int H, int W, int kh, int kw, int flag, int& Hout, int& Wout) {
    if (!decx_hip_is_init()) return not_init();
    if (flag != decx::de_conv_no_compensate && flag != decx::de_conv_zero_compensate) {
        static char msg[] = "This flag is meaningless in current context\n";              // core/error.h:67
        return DH{decx::DECX_FAIL_ErrorFlag, msg};
    }
    static char dims_msg[] = "Tensor Dims don't match each other";
    if (src_depth != ker_depth) return DH{decx::DECX_FAIL_DimsNotMatching, dims_msg};
    Hout = flag ? H : H - 2 * (kh / 2);
    Wout = flag ? W : W - 2 * (kw / 2);
    if (Hout <= 0 || Wout <= 0) return DH{decx::DECX_FAIL_DimsNotMatching, dims_msg};
    return ok();
}

template <typename T>
DH conv_host(Tensor<T>& src_, TensorArray<T>& kernel_, Tensor<T>& dst_, const int flag) {
    auto* src = dynamic_cast<decx::_Tensor<T>*>(&src_);
    auto* ker = dynamic_cast<decx::_TensorArray<T>*>(&kernel_);
    auto* dst = dynamic_cast<decx::_Tensor<T>*>(&dst_);
    if (!src || !ker || !dst) return DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    const int H = (int)src->height, W = (int)src->width, kh = (int)ker->height, kw = (int)ker->width;
    int Hout = 0, Wout = 0;
    DH pre = conv_precheck(src->depth, ker->depth, H, W, kh, kw, flag, Hout, Wout);
    if (pre.error_type != decx::DECX_SUCCESS) return pre;
    decx::_Tensor<T> out_shape;
    out_shape.attribute_assign((uint)Wout, (uint)Hout, ker->tensor_num, decx::Page_Locked);
    DeviceTemp dS, dK, dD;
    if (dS.alloc(src->total_bytes) || dK.alloc(ker->total_bytes) || dD.alloc(out_shape.total_bytes)) return alloc_fail();
    int rc = decx_hip_memcpy(dS.ptr, src->Tens.ptr, src->total_bytes, DECX_HIP_H2D);
    if (rc) return from_status(rc);
    rc = decx_hip_memcpy(dK.ptr, ker->TensArr.ptr, ker->total_bytes, DECX_HIP_H2D);
    if (rc) return from_status(rc);
    // dst may be src (or share its payload): it is sized (and zero-filled) only now that the operands are on the device,
    // and what the kernel needs of src's layout is taken down before that, since re_construct may rewrite those fields
    const int src_dpitch = (int)src->dpitch;
    const size_t src_row = src->dp_x_wp;
    // (:178; every byte of dst, padding included, then comes down from the device block, which is zero where the
    // kernel does not write: the zero fill of re_construct would be written over)
    if (!dst->re_construct_for_overwrite((uint)Wout, (uint)Hout, ker->tensor_num, decx::Page_Locked)) return alloc_fail();
    rc = decx_hip_memset(dD.ptr, 0, dst->total_bytes);   // the width / channel padding of dst stays zero
    if (rc) return from_status(rc);
    rc = ConvCall<T>::run(static_cast<const T*>(dS.ptr), H, W, src_dpitch, src_row, static_cast<const T*>(dK.ptr),
                          (int)ker->tensor_num, kh, kw, ker->_gap, ker->dp_x_wp, static_cast<T*>(dD.ptr), (int)dst->dpitch,
                          dst->dp_x_wp, flag);
    if (rc) return from_status(rc);
    return from_status(decx_hip_memcpy(dst->Tens.ptr, dD.ptr, dst->total_bytes, DECX_HIP_D2H));   // :266
}

template <typename T>
DH conv_device(GPU_Tensor<T>& src_, GPU_TensorArray<T>& kernel_, GPU_Tensor<T>& dst_, const int flag) {
    auto* src = dynamic_cast<decx::_GPU_Tensor<T>*>(&src_);
    auto* ker = dynamic_cast<decx::_GPU_TensorArray<T>*>(&kernel_);
    auto* dst = dynamic_cast<decx::_GPU_Tensor<T>*>(&dst_);
    if (!src || !ker || !dst) return DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    const int H = (int)src->height, W = (int)src->width, kh = (int)ker->height, kw = (int)ker->width;
    int Hout = 0, Wout = 0;
    DH pre = conv_precheck(src->depth, ker->depth, H, W, kh, kw, flag, Hout, Wout);
    if (pre.error_type != decx::DECX_SUCCESS) return pre;
    // a dst that is src or shares its payload would be overwritten while neighbouring outputs still read it (or be
    // freed by re_construct before the kernel runs): such a result goes into a fresh tensor that dst then takes over
    decx::_GPU_Tensor<T> fresh;
    decx::_GPU_Tensor<T>* out = dst;
    if (dst == src || dst->shares_block_with(*src)) {
        if (!fresh.construct((uint)Wout, (uint)Hout, ker->tensor_num))
            return fresh.last_status == DECX_HIP_FAIL_ALLOCATION ? alloc_fail() : from_status(fresh.last_status);
        out = &fresh;
    } else if (!dst->re_construct((uint)Wout, (uint)Hout, ker->tensor_num)) {
        return dst->last_status == DECX_HIP_FAIL_ALLOCATION ? alloc_fail() : from_status(dst->last_status);
    }
    const int rc = ConvCall<T>::run(src->Tens.ptr, H, W, (int)src->dpitch, src->dp_x_wp, ker->TensArr.ptr,
                                    (int)ker->tensor_num, kh, kw, ker->_gap, ker->dp_x_wp, out->Tens.ptr, (int)out->dpitch,
                                    out->dp_x_wp, flag);
    if (rc == 0 && out != dst) dst->share_from(fresh);
    return from_status(rc);
}
}  // namespace

DH Conv2_MK_im2col(Tensor<float>& src, TensorArray<float>& kernel, Tensor<float>& dst, const int flag) {
    return conv_host<float>(src, kernel, dst, flag);
}
DH Conv2_MK_im2col(GPU_Tensor<float>& src, GPU_TensorArray<float>& kernel, GPU_Tensor<float>& dst, const int flag) {
    return conv_device<float>(src, kernel, dst, flag);
}
DH Conv2_MK_im2col(Tensor<Half>& src, TensorArray<Half>& kernel, Tensor<Half>& dst, const int flag) {
    return conv_host<Half>(src, kernel, dst, flag);
}
DH Conv2_MK_im2col(GPU_Tensor<Half>& src, GPU_TensorArray<Half>& kernel, GPU_Tensor<Half>& dst, const int flag) {
    return conv_device<Half>(src, kernel, dst, flag);
}
}  // namespace cuda

// ---- nn::ReLU (nn/operators/ReLU.h:169-210) ----------------------------------------------------------------------
namespace nn {
namespace {
struct ReluArgs {
    decx::_GPU_Matrix<float>* src;
    decx::_GPU_Matrix<float>* dst;
    size_t len;         // floats the kernels run over: pitch * height (ReLU.h:175)
    DH status;
    bool ok;
};
ReluArgs relu_args(GPU_Matrix<float>& src_, GPU_Matrix<float>& dst_) {
    ReluArgs r{dynamic_cast<decx::_GPU_Matrix<float>*>(&src_), dynamic_cast<decx::_GPU_Matrix<float>*>(&dst_), 0, DH{}, false};
    static char dims_msg[] = "Matrix Dims don't match each other";
    if (!r.src || !r.dst) r.status = DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    else if (!decx_hip_is_init()) r.status = not_init();
    else if (r.src->width != r.dst->width || r.src->height != r.dst->height || !r.src->Mat.ptr || !r.dst->Mat.ptr)
        r.status = DH{decx::DECX_FAIL_DimsNotMatching, dims_msg};
    else {
        r.len = (size_t)r.src->pitch * r.src->height;
        r.ok = true;
    }
    return r;
}
}  // namespace

DH ReLU_f(GPU_Matrix<float>& src, GPU_Matrix<float>& dst) {
    ReluArgs a = relu_args(src, dst);
    if (!a.ok) return a.status;
    return from_status(decx_hip_relu_f32(a.src->Mat.ptr, a.dst->Mat.ptr, a.len));
}

DH ReLU_f_Rec(GPU_Matrix<float>& src, GPU_Matrix<float>& dst, GPU_Matrix<uchar>& rec_map) {
    ReluArgs a = relu_args(src, dst);
    if (!a.ok) return a.status;
    auto* map = dynamic_cast<decx::_GPU_Matrix<uchar>*>(&rec_map);
    if (!map) return DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    if ((!map->Mat.ptr || map->_total_bytes < a.len / 8) && !map->re_construct(a.src->pitch / 8, a.src->height))
        return map->last_status == DECX_HIP_FAIL_ALLOCATION ? alloc_fail() : from_status(map->last_status);
    return from_status(decx_hip_relu_f32_rec(a.src->Mat.ptr, a.dst->Mat.ptr, map->Mat.ptr, a.len));
}

DH ReLU_f_Backward(GPU_Matrix<float>& src, GPU_Matrix<float>& dst, GPU_Matrix<uchar>& rec_map) {
    ReluArgs a = relu_args(src, dst);
    if (!a.ok) return a.status;
    auto* map = dynamic_cast<decx::_GPU_Matrix<uchar>*>(&rec_map);
    if (!map) return DH{decx::DECX_FAIL_ErrorParams, kNotFactory};
    static char dims_msg[] = "Matrix Dims don't match each other";
    if (!map->Mat.ptr || map->_total_bytes < a.len / 8) return DH{decx::DECX_FAIL_DimsNotMatching, dims_msg};
    return from_status(decx_hip_relu_f32_backward(a.src->Mat.ptr, a.dst->Mat.ptr, map->Mat.ptr, a.len));
}
}  // namespace nn
}  // namespace de
