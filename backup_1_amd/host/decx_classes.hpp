// Concrete containers behind the abstract classes of DECX.h, with the reference's layout rules:
//   Matrix / GPU_Matrix : row pitch = width rounded up to 8 (4-byte), 16 (2-byte), 4 (8-byte), 32 (1-byte) elements
//                         (classes/Matrix.h:24-27, :253-322; GPU_Matrix.h:211-271)
//   Tensor              : channel-innermost, dpitch = ceil4(depth), wpitch = ceil4(width), row stride dp_x_wp,
//                         zero-filled on allocation (classes/Tensor.h:162-184, :312, :389-394)
//   TensorArray         : tensor_num tensors back to back, stride _gap = dp_x_wp * height
//                         (classes/TensorArray.h:174-198, :349-352, :521-525)
// Field names and their meaning follow the reference, so that code reading them ports directly:
//   Matrix / GPU_Matrix : element_num = width*height, total_bytes = element_num*sizeof(T)          (the true extent)
//                         _element_num = pitch*height, _total_bytes = _element_num*sizeof(T)        (the allocation)
//                         (Matrix.h:253-267, :308-322; GPU_Matrix.h:211-223, :259-271); TotalBytes() = total_bytes
//   Tensor(Array), MatrixArray : element_num = true count, _element_num = padded count, total_bytes = padded bytes
//                         (Tensor.h:162-184, TensorArray.h:174-198, MatrixArray.h:222-239)
// operator= shares the payload like the reference (Matrix.h:510-530, GPU_Matrix.h:441-451, Tensor.h:501-526,
// MatrixArray.h:473-498: the block pointer is copied and its reference count raised): both objects then read and write
// the same memory, release() of one leaves the other valid, the last release frees it.
#pragma once
#include <cstdlib>
#include <cstring>
#include <memory>

#include "../../include/decx_hip.h"
#include "DECX.h"

namespace decx {

inline uint ceil_to(uint v, uint a) { return (v + a - 1) / a * a; }

template <typename T>
constexpr uint matrix_align() {
    return sizeof(T) == 4 ? 8 : sizeof(T) == 2 ? 16 : sizeof(T) == 8 ? 4 : 32;
}

// Host storage: pinned (Page_Locked) through the C ABI when a device is initialised, else 64-byte aligned pageable.
struct HostBlock {
    void* ptr = nullptr;
    bool pinned = false;
    bool alloc(size_t bytes, int store_type) {
        free();
        if (bytes == 0) bytes = 64;
        if (store_type == Page_Locked && decx_hip_is_init()) {
            if (decx_hip_host_malloc(&ptr, bytes) == 0) {
                pinned = true;
                return true;
            }
            ptr = nullptr;
        }
        pinned = false;
        ptr = std::aligned_alloc(64, (bytes + 63) / 64 * 64);
        return ptr != nullptr;
    }
    void free() {
        if (!ptr) return;
        if (pinned) decx_hip_host_free(ptr);
        else std::free(ptr);
        ptr = nullptr;
    }
    HostBlock() = default;
    HostBlock(const HostBlock&) = delete;
    HostBlock& operator=(const HostBlock&) = delete;
    ~HostBlock() { free(); }
};

// Device storage through the C ABI; zero-filled over its whole (padded) size.
struct DeviceBlock {
    void* ptr = nullptr;
    int alloc(size_t bytes) {
        free();
        int rc = decx_hip_malloc(&ptr, bytes ? bytes : 64);
        if (rc != 0) { ptr = nullptr; return rc; }
        return decx_hip_memset(ptr, 0, bytes);
    }
    void free() {
        if (ptr) decx_hip_free(ptr);
        ptr = nullptr;
    }
    DeviceBlock() = default;
    DeviceBlock(const DeviceBlock&) = delete;
    DeviceBlock& operator=(const DeviceBlock&) = delete;
    ~DeviceBlock() { free(); }
};

template <typename T>
struct PtrInfo {   // the reference's decx::PtrInfo<T> exposes .ptr (core/memory_management/MemBlock.h:45-133)
    T* ptr = nullptr;
};

template <typename T>
class _Matrix : public de::Matrix<T> {
    std::shared_ptr<HostBlock> block_;

public:
    uint width = 0, height = 0;
    unsigned short Store_Type = Page_Default;
    size_t element_num = 0, total_bytes = 0;     // true extent: width * height            (Matrix.h:262-263)
    uint pitch = 0;
    PtrInfo<T> Mat;
    size_t _element_num = 0, _total_bytes = 0;   // the allocation: pitch * height         (Matrix.h:265-266)

    _Matrix() {}
    _Matrix(uint w, uint h, int store_type) { construct(w, h, store_type); }
    void attribute_assign(uint w, uint h, int store_type) {
        width = w;
        height = h;
        Store_Type = (unsigned short)store_type;
        pitch = ceil_to(w, matrix_align<T>());
        element_num = (size_t)w * h;
        total_bytes = element_num * sizeof(T);
        _element_num = (size_t)pitch * h;
        _total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h, int store_type) {
        attribute_assign(w, h, store_type);
        block_ = std::make_shared<HostBlock>();
        bool ok = block_->alloc(_total_bytes, store_type);
        Mat.ptr = static_cast<T*>(block_->ptr);
        return ok;
    }
    bool re_construct(uint w, uint h, int store_type) {   // Matrix.h:238-248: a no-op only when nothing changes
        if (Mat.ptr && w == width && h == height && store_type == Store_Type) return true;
        return construct(w, h, store_type);
    }
    bool shares_block_with(const _Matrix<T>& o) const { return block_ && block_ == o.block_; }
    uint Width() override { return width; }
    uint Height() override { return height; }
    size_t TotalBytes() override { return total_bytes; }
    T& index(const int row, const int col) override { return Mat.ptr[(size_t)pitch * row + col]; }
    void release() override {
        block_.reset();
        Mat.ptr = nullptr;
    }
    void share_from(_Matrix<T>& s) {
        if (&s == this) return;
        block_ = s.block_;
        attribute_assign(s.width, s.height, s.Store_Type);
        Mat.ptr = s.Mat.ptr;
    }
    de::Matrix<T>& operator=(de::Matrix<T>& src) override {   // shares src's block (Matrix.h:510-530)
        share_from(dynamic_cast<_Matrix<T>&>(src));
        return *this;
    }
    _Matrix(const _Matrix&) = delete;
    _Matrix& operator=(const _Matrix&) = delete;
    ~_Matrix() override { release(); }
};

template <typename T>
class _GPU_Matrix : public de::GPU_Matrix<T> {
    std::shared_ptr<DeviceBlock> block_;

public:
    uint width = 0, height = 0;
    size_t element_num = 0, total_bytes = 0;     // true extent: width * height            (GPU_Matrix.h:218-219)
    uint pitch = 0;
    PtrInfo<T> Mat;                              // DEVICE pointer
    size_t _element_num = 0, _total_bytes = 0;   // the allocation: pitch * height         (GPU_Matrix.h:221-222)
    int last_status = 0;                         // status of the most recent allocation / copy

    _GPU_Matrix() {}
    _GPU_Matrix(uint w, uint h) { construct(w, h); }
    void attribute_assign(uint w, uint h) {
        width = w;
        height = h;
        pitch = ceil_to(w, matrix_align<T>());
        element_num = (size_t)w * h;
        total_bytes = element_num * sizeof(T);
        _element_num = (size_t)pitch * h;
        _total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h) {
        release();
        attribute_assign(w, h);
        block_ = std::make_shared<DeviceBlock>();
        // zero the whole pitched buffer (the reference clears only total_bytes of it, GPU_Matrix.h:152, :167)
        last_status = block_->alloc(_total_bytes);
        Mat.ptr = static_cast<T*>(block_->ptr);
        return last_status == 0;
    }
    bool re_construct(uint w, uint h) {
        if (Mat.ptr && w == width && h == height) return true;
        return construct(w, h);
    }
    uint Width() override { return width; }
    uint Height() override { return height; }
    size_t TotalBytes() override { return total_bytes; }
    void Load_from_host(de::Matrix<T>& src) override {
        _Matrix<T>& s = dynamic_cast<_Matrix<T>&>(src);
        if (s.width != width || s.height != height) { last_status = DECX_HIP_FAIL_DIMS; return; }
        last_status = decx_hip_memcpy2d(Mat.ptr, (size_t)pitch * sizeof(T), s.Mat.ptr, (size_t)s.pitch * sizeof(T),
                                        (size_t)width * sizeof(T), height, DECX_HIP_H2D);
    }
    void Load_to_host(de::Matrix<T>& dst) override {
        _Matrix<T>& d = dynamic_cast<_Matrix<T>&>(dst);
        if (d.width != width || d.height != height) { last_status = DECX_HIP_FAIL_DIMS; return; }
        last_status = decx_hip_memcpy2d(d.Mat.ptr, (size_t)d.pitch * sizeof(T), Mat.ptr, (size_t)pitch * sizeof(T),
                                        (size_t)width * sizeof(T), height, DECX_HIP_D2H);
    }
    void release() override {
        block_.reset();
        Mat.ptr = nullptr;
    }
    bool shares_block_with(const _GPU_Matrix<T>& o) const { return block_ && block_ == o.block_; }
    void share_from(_GPU_Matrix<T>& s) {
        if (&s == this) return;
        block_ = s.block_;
        attribute_assign(s.width, s.height);
        Mat.ptr = s.Mat.ptr;
    }
    de::GPU_Matrix<T>& operator=(de::GPU_Matrix<T>& src) override {   // shares src's block (GPU_Matrix.h:441-451)
        share_from(dynamic_cast<_GPU_Matrix<T>&>(src));
        return *this;
    }
    ~_GPU_Matrix() override { release(); }
};

template <typename T>
class _Tensor : public de::Tensor<T> {
    std::shared_ptr<HostBlock> block_;

public:
    uint width = 0, height = 0, depth = 0;
    int _store_type = Page_Default;
    uint dpitch = 0, wpitch = 0;
    size_t dp_x_wp = 0;
    PtrInfo<T> Tens;
    size_t element_num = 0, _element_num = 0, total_bytes = 0;

    _Tensor() {}
    _Tensor(uint w, uint h, uint d, int store_type) { construct(w, h, d, store_type); }
    void attribute_assign(uint w, uint h, uint d, int store_type) {
        width = w;
        height = h;
        depth = d;
        _store_type = store_type;
        wpitch = ceil_to(w, 4);
        dpitch = ceil_to(d, sizeof(T) == 2 ? 8 : 4);     // _TENSOR_ALIGN_4B_ = 4, _TENSOR_ALIGN_2B_ = 8 (classes/Tensor.h:21-23)
        dp_x_wp = (size_t)dpitch * wpitch;
        element_num = (size_t)d * w * h;
        _element_num = (size_t)h * dp_x_wp;
        total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h, uint d, int store_type) {
        attribute_assign(w, h, d, store_type);
        block_ = std::make_shared<HostBlock>();
        bool ok = block_->alloc(total_bytes, store_type);
        Tens.ptr = static_cast<T*>(block_->ptr);
        if (ok) std::memset(Tens.ptr, 0, total_bytes);
        return ok;
    }
    bool re_construct(uint w, uint h, uint d, int store_type) {
        if (Tens.ptr && w == width && h == height && d == depth && store_type == _store_type) {
            std::memset(Tens.ptr, 0, total_bytes);
            return true;
        }
        return construct(w, h, d, store_type);
    }
    // re_construct for a caller that writes all total_bytes itself right away (padding included): a tensor that
    // already has the shape is left as it is instead of zero-filled (Tensor.h:350-355 fills; 25.7 MB take 0.3 ms)
    bool re_construct_for_overwrite(uint w, uint h, uint d, int store_type) {
        if (Tens.ptr && w == width && h == height && d == depth && store_type == _store_type) return true;
        return construct(w, h, d, store_type);
    }
    uint Width() override { return width; }
    uint Height() override { return height; }
    uint Depth() override { return depth; }
    T& index(const int x, const int y, const int z) override { return Tens.ptr[(size_t)x * dp_x_wp + (size_t)y * dpitch + z]; }
    de::Tensor<T>& operator=(de::Tensor<T>& src) override {   // shares src's block (Tensor.h:501-526)
        _Tensor<T>& s = dynamic_cast<_Tensor<T>&>(src);
        if (&s != this) {
            block_ = s.block_;
            attribute_assign(s.width, s.height, s.depth, s._store_type);
            Tens.ptr = s.Tens.ptr;
        }
        return *this;
    }
    void release() override {
        block_.reset();
        Tens.ptr = nullptr;
    }
    ~_Tensor() override { release(); }
};

template <typename T>
class _TensorArray : public de::TensorArray<T> {
    std::shared_ptr<HostBlock> block_;

public:
    uint width = 0, height = 0, depth = 0, tensor_num = 0;
    int _store_type = Page_Default;
    uint dpitch = 0, wpitch = 0;
    size_t dp_x_wp = 0, _gap = 0;
    PtrInfo<T> TensArr;
    size_t element_num = 0, _element_num = 0, total_bytes = 0;

    _TensorArray() {}
    _TensorArray(uint w, uint h, uint d, uint n, int store_type) { construct(w, h, d, n, store_type); }
    void attribute_assign(uint w, uint h, uint d, uint n, int store_type) {
        width = w;
        height = h;
        depth = d;
        tensor_num = n;
        _store_type = store_type;
        wpitch = ceil_to(w, 4);
        dpitch = ceil_to(d, sizeof(T) == 2 ? 8 : 4);     // _TENSOR_ALIGN_4B_ = 4, _TENSOR_ALIGN_2B_ = 8 (classes/Tensor.h:21-23)
        dp_x_wp = (size_t)dpitch * wpitch;
        _gap = dp_x_wp * h;
        element_num = (size_t)d * w * h * n;
        _element_num = (size_t)n * _gap;
        total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h, uint d, uint n, int store_type) {
        attribute_assign(w, h, d, n, store_type);
        block_ = std::make_shared<HostBlock>();
        bool ok = block_->alloc(total_bytes, store_type);
        TensArr.ptr = static_cast<T*>(block_->ptr);
        if (ok) std::memset(TensArr.ptr, 0, total_bytes);
        return ok;
    }
    uint Width() override { return width; }
    uint Height() override { return height; }
    uint Depth() override { return depth; }
    uint TensorNum() override { return tensor_num; }
    T& index(const int x, const int y, const int z, const int tensor_id) override {
        return TensArr.ptr[(size_t)tensor_id * _gap + (size_t)x * dp_x_wp + (size_t)y * dpitch + z];
    }
    de::TensorArray<T>& operator=(de::TensorArray<T>& src) override {   // shares src's block (TensorArray.h:529-554)
        _TensorArray<T>& s = dynamic_cast<_TensorArray<T>&>(src);
        if (&s != this) {
            block_ = s.block_;
            attribute_assign(s.width, s.height, s.depth, s.tensor_num, s._store_type);
            TensArr.ptr = s.TensArr.ptr;
        }
        return *this;
    }
    void release() override {
        block_.reset();
        TensArr.ptr = nullptr;
    }
    ~_TensorArray() override { release(); }
};

// classes/MatrixArray.h:222-239 (attributes), :367-370 (index)
template <typename T>
class _MatrixArray : public de::MatrixArray<T> {
    std::shared_ptr<HostBlock> block_;

public:
    int _store_type = Page_Default;
    PtrInfo<T> MatArr;
    uint width = 0, height = 0, pitch = 0;
    size_t element_num = 0, _element_num = 0, total_bytes = 0, ArrayNumber = 0;
    size_t plane = 0, _plane = 0;                // true / padded elements per matrix

    _MatrixArray() {}
    _MatrixArray(uint w, uint h, uint n, int flag) { construct(w, h, n, flag); }
    void attribute_assign(uint w, uint h, uint n, int flag) {
        width = w;
        height = h;
        ArrayNumber = n;
        _store_type = flag;
        pitch = ceil_to(w, matrix_align<T>());
        plane = (size_t)w * h;
        _plane = (size_t)pitch * h;
        element_num = plane * n;
        _element_num = _plane * n;
        total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h, uint n, int flag) {
        attribute_assign(w, h, n, flag);
        block_ = std::make_shared<HostBlock>();
        bool ok = block_->alloc(total_bytes, flag);
        MatArr.ptr = static_cast<T*>(block_->ptr);
        return ok;
    }
    bool re_construct(uint w, uint h, uint n, int flag) {
        if (MatArr.ptr && w == width && h == height && n == ArrayNumber && flag == _store_type) return true;
        return construct(w, h, n, flag);
    }
    uint Width() override { return width; }
    uint Height() override { return height; }
    uint MatrixNumber() override { return (uint)ArrayNumber; }
    bool shares_block_with(const _MatrixArray<T>& o) const { return block_ && block_ == o.block_; }
    T& index(uint row, uint col, size_t seq) override { return MatArr.ptr[seq * _plane + (size_t)row * pitch + col]; }
    void share_from(_MatrixArray<T>& s) {
        if (&s == this) return;
        block_ = s.block_;
        attribute_assign(s.width, s.height, (uint)s.ArrayNumber, s._store_type);
        MatArr.ptr = s.MatArr.ptr;
    }
    de::MatrixArray<T>& operator=(de::MatrixArray<T>& src) override {   // shares src's block (MatrixArray.h:473-498)
        share_from(dynamic_cast<_MatrixArray<T>&>(src));
        return *this;
    }
    void release() override {
        block_.reset();
        MatArr.ptr = nullptr;
    }
    ~_MatrixArray() override { release(); }
};

template <typename T>
class _GPU_Tensor : public de::GPU_Tensor<T> {
    std::shared_ptr<DeviceBlock> block_;

public:
    uint width = 0, height = 0, depth = 0;
    uint dpitch = 0, wpitch = 0;
    size_t dp_x_wp = 0;
    PtrInfo<T> Tens;                             // DEVICE pointer
    size_t element_num = 0, _element_num = 0, total_bytes = 0;
    int last_status = 0;

    _GPU_Tensor() {}
    _GPU_Tensor(uint w, uint h, uint d) { construct(w, h, d); }
    void attribute_assign(uint w, uint h, uint d) {
        width = w;
        height = h;
        depth = d;
        wpitch = ceil_to(w, 4);
        dpitch = ceil_to(d, sizeof(T) == 2 ? 8 : 4);     // _TENSOR_ALIGN_4B_ = 4, _TENSOR_ALIGN_2B_ = 8 (classes/Tensor.h:21-23)
        dp_x_wp = (size_t)dpitch * wpitch;
        element_num = (size_t)d * w * h;
        _element_num = (size_t)h * dp_x_wp;
        total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h, uint d) {
        release();
        attribute_assign(w, h, d);
        block_ = std::make_shared<DeviceBlock>();
        last_status = block_->alloc(total_bytes);
        Tens.ptr = static_cast<T*>(block_->ptr);
        return last_status == 0;
    }
    bool re_construct(uint w, uint h, uint d) {
        if (Tens.ptr && w == width && h == height && d == depth) return true;
        return construct(w, h, d);
    }
    uint Width() override { return width; }
    uint Height() override { return height; }
    uint Depth() override { return depth; }
    bool shares_block_with(const _GPU_Tensor<T>& o) const { return block_ && block_ == o.block_; }
    void share_from(_GPU_Tensor<T>& s) {
        if (&s == this) return;
        block_ = s.block_;
        attribute_assign(s.width, s.height, s.depth);
        Tens.ptr = s.Tens.ptr;
    }
    de::GPU_Tensor<T>& operator=(de::GPU_Tensor<T>& src) override {   // shares src's block (GPU_Tensor.h)
        share_from(dynamic_cast<_GPU_Tensor<T>&>(src));
        return *this;
    }
    void Load_from_host(de::Tensor<T>& src) override {
        _Tensor<T>& s = dynamic_cast<_Tensor<T>&>(src);
        if (s.width != width || s.height != height || s.depth != depth) { last_status = DECX_HIP_FAIL_DIMS; return; }
        last_status = decx_hip_memcpy(Tens.ptr, s.Tens.ptr, total_bytes, DECX_HIP_H2D);     // identical layouts
    }
    void Load_to_host(de::Tensor<T>& dst) override {
        _Tensor<T>& d = dynamic_cast<_Tensor<T>&>(dst);
        if (d.width != width || d.height != height || d.depth != depth) { last_status = DECX_HIP_FAIL_DIMS; return; }
        last_status = decx_hip_memcpy(d.Tens.ptr, Tens.ptr, total_bytes, DECX_HIP_D2H);
    }
    void release() override {
        block_.reset();
        Tens.ptr = nullptr;
    }
    ~_GPU_Tensor() override { release(); }
};

template <typename T>
class _GPU_TensorArray : public de::GPU_TensorArray<T> {
    std::shared_ptr<DeviceBlock> block_;

public:
    uint width = 0, height = 0, depth = 0, tensor_num = 0;
    uint dpitch = 0, wpitch = 0;
    size_t dp_x_wp = 0, _gap = 0;
    PtrInfo<T> TensArr;                          // DEVICE pointer
    size_t element_num = 0, _element_num = 0, total_bytes = 0;
    int last_status = 0;

    _GPU_TensorArray() {}
    _GPU_TensorArray(uint w, uint h, uint d, uint n) { construct(w, h, d, n); }
    void attribute_assign(uint w, uint h, uint d, uint n) {
        width = w;
        height = h;
        depth = d;
        tensor_num = n;
        wpitch = ceil_to(w, 4);
        dpitch = ceil_to(d, sizeof(T) == 2 ? 8 : 4);     // _TENSOR_ALIGN_4B_ = 4, _TENSOR_ALIGN_2B_ = 8 (classes/Tensor.h:21-23)
        dp_x_wp = (size_t)dpitch * wpitch;
        _gap = dp_x_wp * h;
        element_num = (size_t)d * w * h * n;
        _element_num = (size_t)n * _gap;
        total_bytes = _element_num * sizeof(T);
    }
    bool construct(uint w, uint h, uint d, uint n) {
        release();
        attribute_assign(w, h, d, n);
        block_ = std::make_shared<DeviceBlock>();
        last_status = block_->alloc(total_bytes);
        TensArr.ptr = static_cast<T*>(block_->ptr);
        return last_status == 0;
    }
    uint Width() override { return width; }
    uint Height() override { return height; }
    uint Depth() override { return depth; }
    uint TensorNum() override { return tensor_num; }
    void Load_from_host(de::TensorArray<T>& src) override {
        _TensorArray<T>& s = dynamic_cast<_TensorArray<T>&>(src);
        if (s.width != width || s.height != height || s.depth != depth || s.tensor_num != tensor_num) { last_status = DECX_HIP_FAIL_DIMS; return; }
        last_status = decx_hip_memcpy(TensArr.ptr, s.TensArr.ptr, total_bytes, DECX_HIP_H2D);
    }
    void Load_to_host(de::TensorArray<T>& dst) override {
        _TensorArray<T>& d = dynamic_cast<_TensorArray<T>&>(dst);
        if (d.width != width || d.height != height || d.depth != depth || d.tensor_num != tensor_num) { last_status = DECX_HIP_FAIL_DIMS; return; }
        last_status = decx_hip_memcpy(d.TensArr.ptr, TensArr.ptr, total_bytes, DECX_HIP_D2H);
    }
    de::GPU_TensorArray<T>& operator=(de::GPU_TensorArray<T>& src) override {   // shares src's block
        _GPU_TensorArray<T>& s = dynamic_cast<_GPU_TensorArray<T>&>(src);
        if (&s != this) {
            block_ = s.block_;
            attribute_assign(s.width, s.height, s.depth, s.tensor_num);
            TensArr.ptr = s.TensArr.ptr;
        }
        return *this;
    }
    void release() override {
        block_.reset();
        TensArr.ptr = nullptr;
    }
    ~_GPU_TensorArray() override { release(); }
};

}  // namespace decx
