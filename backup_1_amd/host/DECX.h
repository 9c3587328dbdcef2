// Public C++ API of the dense-contraction path, with DECX's own names and call signatures, so that code written
// against the reference (e.g. test/test/CUDA_GEMM/CUDA_GEMM.cpp) compiles against this header unchanged and links
// libdecx.so.  Everything below is implemented on top of the C ABI in include/decx_hip.h; no CUDA headers, no
// CUDA-named runtime calls.  The reference interface each declaration mirrors is cited next to it (paths relative
// to the reference tree's srcs/ directory).
//
// Conventions kept from the reference: containers are created (width, height[, depth]) by the factories below and
// returned as references to heap objects whose payload is freed by release(); API functions take the abstract
// classes by reference, return a de::DH by value and require containers made by this library's factories; calls
// are synchronous and not thread-safe.
#pragma once
#include <cstddef>
#include <cstdint>

typedef unsigned int uint;
typedef unsigned char uchar;

namespace decx {
// handles/decx_handles.h:6-38
enum DECX_error_types {
    DECX_SUCCESS = 0x00,
    DECX_FAIL_not_init = 0x01,
    DECX_FAIL_FFT_error_length = 0x02,
    DECX_FAIL_DimsNotMatching = 0x03,
    DECX_FAIL_Complex_comparing = 0x04,
    DECX_FAIL_ConvBadKernel = 0x05,
    DECX_FAIL_StepError = 0x06,
    DECX_FAIL_ChannelError = 0x07,
    DECX_FAIL_CVNLM_BadArea = 0x08,
    DECX_FAIL_FileNotExist = 0x09,
    DECX_GEMM_DimsError = 0x0a,
    DECX_FAIL_ErrorFlag = 0x0b,
    DECX_FAIL_DimError = 0x0c,
    DECX_FAIL_ErrorParams = 0x0d,
    DECX_FAIL_StoreError = 0x0e,
    DECX_FAIL_MNumNotMatching = 0x0f,
    DECX_FAIL_ALLOCATION = 0x10
};
// classes/store_types.h:24-28
enum DATA_STORE_TYPE { Page_Locked = 0x00, Page_Default = 0x01 };
// convolution/CUDA/conv_flags.h:16-20
enum conv_property { de_conv_no_compensate = 0, de_conv_zero_compensate = 1 };
}  // namespace decx

namespace de {

// handles/decx_handles.h:42-49.  error_string points at storage owned by the library; never free it.
// Values >= 1000 in error_type are 1000 + a HIP runtime error (the reference exits the process instead,
// core/error.h:32-45).
typedef struct DECX_Handle {
    int error_type;
    char* error_string;
} DH;

// classes/classes_util.h:58-63: IEEE binary16 bit pattern
struct alignas(2) Half {
    unsigned short val;
};

// basic_process/float_half_convert.h:20-43 (round to nearest even, as __float2half)
Half Float2Half(const float& x);
float Half2Float(const Half& x);

// classes/Matrix.h:34-64.  TotalBytes() is width * height * sizeof(T) (Matrix.h:104, :262-263), not the pitched size.
// operator= of every container shares src's payload instead of copying it, as in the reference (Matrix.h:510-530):
// both objects then address the same memory, and it is freed when the last holder releases it.
template <typename T>
class Matrix {
public:
    Matrix() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual size_t TotalBytes() = 0;
    virtual T& index(const int row, const int col) = 0;
    virtual void release() = 0;
    virtual Matrix<T>& operator=(Matrix<T>& src) = 0;
    virtual ~Matrix() {}
};

// classes/GPU_Matrix.h:19-47
template <typename T>
class GPU_Matrix {
public:
    GPU_Matrix() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual size_t TotalBytes() = 0;
    virtual void Load_from_host(Matrix<T>& src) = 0;
    virtual void Load_to_host(Matrix<T>& dst) = 0;
    virtual void release() = 0;
    virtual GPU_Matrix<T>& operator=(GPU_Matrix<T>& src) = 0;
    virtual ~GPU_Matrix() {}
};

// classes/Tensor.h:31-52.  index(x = row, y = column, z = channel)  (Tensor.h:389-394)
template <typename T>
class Tensor {
public:
    Tensor() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual uint Depth() = 0;
    virtual T& index(const int x, const int y, const int z) = 0;
    virtual Tensor<T>& operator=(Tensor<T>& src) = 0;
    virtual void release() = 0;
    virtual ~Tensor() {}
};

// classes/TensorArray.h:26-50.  index(x = row, y = column, z = channel, tensor_id)  (TensorArray.h:521-525)
template <typename T>
class TensorArray {
public:
    TensorArray() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual uint Depth() = 0;
    virtual uint TensorNum() = 0;
    virtual T& index(const int x, const int y, const int z, const int tensor_id) = 0;
    virtual TensorArray<T>& operator=(TensorArray<T>& src) = 0;
    virtual void release() = 0;
    virtual ~TensorArray() {}
};

// classes/MatrixArray.h:28-52.  MatrixNum equally sized host matrices back to back (pitch*height elements apart).
template <typename T>
class MatrixArray {
public:
    MatrixArray() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual uint MatrixNumber() = 0;
    virtual T& index(uint row, uint col, size_t seq) = 0;
    virtual MatrixArray<T>& operator=(MatrixArray<T>& src) = 0;
    virtual void release() = 0;
    virtual ~MatrixArray() {}
};

// classes/GPU_Tensor.h:19-47.  Device-resident tensor with the host Tensor's layout (dpitch = ceil4(depth) for 4-byte and ceil8(depth) for 2-byte elements,
// wpitch = ceil4(width)).
template <typename T>
class GPU_Tensor {
public:
    GPU_Tensor() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual uint Depth() = 0;
    virtual GPU_Tensor<T>& operator=(GPU_Tensor<T>& src) = 0;
    virtual void Load_from_host(Tensor<T>& src) = 0;
    virtual void Load_to_host(Tensor<T>& dst) = 0;
    virtual void release() = 0;
    virtual ~GPU_Tensor() {}
};

// classes/GPU_TensorArray.h:24-52
template <typename T>
class GPU_TensorArray {
public:
    GPU_TensorArray() {}
    virtual uint Width() = 0;
    virtual uint Height() = 0;
    virtual uint Depth() = 0;
    virtual uint TensorNum() = 0;
    virtual void Load_from_host(TensorArray<T>& src) = 0;
    virtual void Load_to_host(TensorArray<T>& dst) = 0;
    virtual GPU_TensorArray<T>& operator=(GPU_TensorArray<T>& src) = 0;
    virtual void release() = 0;
    virtual ~GPU_TensorArray() {}
};

// factories: classes/Matrix.h:430-476, GPU_Matrix.h:361-435, Tensor.h:401-463, TensorArray.h:440-474.
// Instantiated for float and de::Half.
template <typename T> Matrix<T>& CreateMatrixRef();
template <typename T> Matrix<T>* CreateMatrixPtr();
template <typename T> Matrix<T>& CreateMatrixRef(const uint width, const uint height, const int store_type);
template <typename T> Matrix<T>* CreateMatrixPtr(const uint width, const uint height, const int store_type);
template <typename T> GPU_Matrix<T>& CreateGPUMatrixRef();
template <typename T> GPU_Matrix<T>* CreateGPUMatrixPtr();
template <typename T> GPU_Matrix<T>& CreateGPUMatrixRef(const uint width, const uint height);
template <typename T> GPU_Matrix<T>* CreateGPUMatrixPtr(const uint width, const uint height);
template <typename T> Tensor<T>& CreateTensorRef();
template <typename T> Tensor<T>* CreateTensorPtr();
template <typename T> Tensor<T>& CreateTensorRef(const uint width, const uint height, const uint depth, const int flag);
template <typename T> Tensor<T>* CreateTensorPtr(const uint width, const uint height, const uint depth, const int flag);
template <typename T> TensorArray<T>& CreateTensorArrayRef();
template <typename T> TensorArray<T>* CreateTensorArrayPtr();
template <typename T> TensorArray<T>& CreateTensorArrayRef(const uint width, const uint height, const uint depth, const uint tensor_num, const int flag);
template <typename T> TensorArray<T>* CreateTensorArrayPtr(const uint width, const uint height, const uint depth, const uint tensor_num, const int flag);

// classes/MatrixArray.h:377-389; instantiated for float and de::Half
template <typename T> MatrixArray<T>& CreateMatrixArrayRef();
template <typename T> MatrixArray<T>* CreateMatrixArrayPtr();
template <typename T> MatrixArray<T>& CreateMatrixArrayRef(uint width, uint height, uint MatrixNum, const int flag);
template <typename T> MatrixArray<T>* CreateMatrixArrayPtr(uint width, uint height, uint MatrixNum, const int flag);

// classes/GPU_Tensor.h:385-397, GPU_TensorArray.h (same pattern); instantiated for float and de::Half
template <typename T> GPU_Tensor<T>& CreateGPUTensorRef();
template <typename T> GPU_Tensor<T>* CreateGPUTensorPtr();
template <typename T> GPU_Tensor<T>& CreateGPUTensorRef(const uint width, const uint height, const uint depth);
template <typename T> GPU_Tensor<T>* CreateGPUTensorPtr(const uint width, const uint height, const uint depth);
template <typename T> GPU_TensorArray<T>& CreateGPUTensorArrayRef();
template <typename T> GPU_TensorArray<T>* CreateGPUTensorArrayPtr();
template <typename T> GPU_TensorArray<T>& CreateGPUTensorArrayRef(const uint width, const uint height, const uint depth, const uint tensor_num);
template <typename T> GPU_TensorArray<T>* CreateGPUTensorArrayPtr(const uint width, const uint height, const uint depth, const uint tensor_num);

// core/configs/config.h:62, :73-78.  The name is kept for drop-in use; it initialises the HIP device.
void InitCuda();
// core/memory_management/Memory_pool.h:23-37.  There are no pools here; kept as a no-op.
void release_all_tmp();

namespace cuda {
// GEMM/CUDA/large_squares/GEMM.h:27-49.  A is (K wide, M high), B (N wide, K high); dst becomes (N wide, M high).
DH GEMM(Matrix<float>& A, Matrix<float>& B, Matrix<float>& dst);
DH GEMM(Matrix<float>& A, Matrix<float>& B, Matrix<float>& C, Matrix<float>& dst);
DH GEMM(Matrix<Half>& A, Matrix<Half>& B, Matrix<Half>& dst);
DH GEMM(Matrix<Half>& A, Matrix<Half>& B, Matrix<Half>& C, Matrix<Half>& dst);
DH GEMM(GPU_Matrix<float>& A, GPU_Matrix<float>& B, GPU_Matrix<float>& dst);
DH GEMM(GPU_Matrix<float>& A, GPU_Matrix<float>& B, GPU_Matrix<float>& C, GPU_Matrix<float>& dst);
DH GEMM(GPU_Matrix<Half>& A, GPU_Matrix<Half>& B, GPU_Matrix<Half>& dst);
DH GEMM(GPU_Matrix<Half>& A, GPU_Matrix<Half>& B, GPU_Matrix<Half>& C, GPU_Matrix<Half>& dst);
// GEMM/CUDA/extreme_shapes/GEMM_long_Lr.h:22.  dst = A * B for short-M / long-K shapes: one fused chain per output over
// ascending k like the reference's kernel (no split over K), so the result is bit-identical to GEMM's.  Unlike the
// reference it checks initialisation and dimensions, sizes dst, handles any shape and reports its status.
DH GEMM_Long_Lr(GPU_Matrix<float>& A, GPU_Matrix<float>& B, GPU_Matrix<float>& dst);
// GEMM/CUDA/large_squares/GEMM3.h:27-36.  dst[i] = A[i] * B[i] (+ C[i]) for every matrix of the arrays, uploads and
// downloads overlapped with the kernels.
DH GEMM3(MatrixArray<float>& A, MatrixArray<float>& B, MatrixArray<float>& dst);
DH GEMM3(MatrixArray<Half>& A, MatrixArray<Half>& B, MatrixArray<Half>& dst);
DH GEMM3(MatrixArray<float>& A, MatrixArray<float>& B, MatrixArray<float>& C, MatrixArray<float>& dst);
DH GEMM3(MatrixArray<Half>& A, MatrixArray<Half>& B, MatrixArray<Half>& C, MatrixArray<Half>& dst);
// convolution/CUDA/im2col/conv2_mk_im2col.h:25.  flag: decx::conv_property.
DH Conv2_MK_im2col(Tensor<float>& src, TensorArray<float>& kernel, Tensor<float>& dst, const int flag);
// Device-resident flavour of the same convolution (the reference only has the host one; its GPU_Tensor /
// GPU_TensorArray containers, classes/GPU_Tensor.h and GPU_TensorArray.h, are what it would take).  dst is
// (re)constructed to the output size; no host copies are made.
DH Conv2_MK_im2col(GPU_Tensor<float>& src, GPU_TensorArray<float>& kernel, GPU_Tensor<float>& dst, const int flag);
// The same convolution on binary16 containers (de::Tensor<de::Half> etc., channel pitch a multiple of 8: classes/Tensor.h:214-235,
// TensorArray.h:232-256, GPU_Tensor.h:201-222, GPU_TensorArray.h:234-257), accumulated in fp32.  The reference declares
// the containers but no binary16 im2col convolution; these overloads are what it would look like.
DH Conv2_MK_im2col(Tensor<Half>& src, TensorArray<Half>& kernel, Tensor<Half>& dst, const int flag);
DH Conv2_MK_im2col(GPU_Tensor<Half>& src, GPU_TensorArray<Half>& kernel, GPU_Tensor<Half>& dst, const int flag);
}  // namespace cuda

namespace nn {
// nn/operators/ReLU.h:28-34.  Element-wise over the whole pitched buffer of src (padding included), with the
// reference's arithmetic: value * float(sign bit clear).  dst must have src's dimensions (the reference prints a
// message and still reports success; here the DH carries DECX_FAIL_DimsNotMatching).  rec_map takes one byte per 8
// floats, filled linearly; ReLU_f_Rec sizes it to (pitch/8, height) if it is too small.
DH ReLU_f(GPU_Matrix<float>& src, GPU_Matrix<float>& dst);
DH ReLU_f_Rec(GPU_Matrix<float>& src, GPU_Matrix<float>& dst, GPU_Matrix<uchar>& rec_map);
DH ReLU_f_Backward(GPU_Matrix<float>& src, GPU_Matrix<float>& dst, GPU_Matrix<uchar>& rec_map);
}  // namespace nn

namespace cpu {
// GEMM/CPU/sgemm.h:22.  Host thread-pool SGEMM.
DH sgemm(Matrix<float>& A, Matrix<float>& B, Matrix<float>& dst);
}  // namespace cpu

}  // namespace de
