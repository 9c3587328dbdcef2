/*
 * C ABI of the MI355X (gfx950) dense-contraction library, libdecx_hip.so.
 *
 * This is the boundary the DECX C++ API (de::cuda::GEMM, de::cuda::Conv2_MK_im2col and the Matrix / GPU_Matrix /
 * Tensor / TensorArray containers) binds to.  DECX itself has no FFI layer: its API functions call CUDA directly.
 * Each entry point below names the piece of the reference it stands in for (paths relative to the reference tree).
 *
 * Conventions
 *   - plain pointers and sizes only; every matrix / tensor pointer is a DEVICE pointer unless the name says host;
 *   - dimensions are the true (unpadded) ones, leading dimensions ("ld", "stride", "pitch") are in ELEMENTS;
 *   - return value 0 = success, 1..0x10 = the matching decx::DECX_error_types value (handles/decx_handles.h:6-38),
 *     >= 1000 = 1000 + hipError_t.  Nothing here calls exit(); the reference does on CUDA errors (core/error.h:32-45);
 *   - calls without the _async suffix block until the result is complete, like the reference's API functions
 *     (cudaDeviceSynchronize at GEMM.h:122, :450; conv2_mk_im2col.h:268);
 *   - one process drives one GPU; the library is not thread-safe (neither is the reference: global pools, no locks).
 */
#ifndef DECX_HIP_H_
#define DECX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* decx::DECX_error_types values used on this path (handles/decx_handles.h:6-38) */
#define DECX_HIP_SUCCESS              0x00
#define DECX_HIP_FAIL_NOT_INIT        0x01
#define DECX_HIP_FAIL_DIMS            0x03
#define DECX_HIP_FAIL_ERROR_FLAG      0x0b
#define DECX_HIP_FAIL_ERROR_PARAMS    0x0d
#define DECX_HIP_FAIL_ALLOCATION      0x10
#define DECX_HIP_FAIL_HIP_BASE        1000

/* decx::conv_property (convolution/CUDA/conv_flags.h:16-20) */
#define DECX_HIP_CONV_NO_COMPENSATE   0
#define DECX_HIP_CONV_ZERO_COMPENSATE 1

/* copy directions for decx_hip_memcpy / decx_hip_memcpy2d */
#define DECX_HIP_H2D 1
#define DECX_HIP_D2H 2
#define DECX_HIP_D2D 3

/* de::InitCuda() (core/configs/config.h:73-78): selects the current device, checks it is gfx950, creates the
 * library's stream.  *device (nullable) receives the device ordinal.  Every compute entry point returns
 * DECX_HIP_FAIL_NOT_INIT before this has succeeded (the decx::cuP.is_init gate, GEMM.h:63). */
int decx_hip_init(int* device);
int decx_hip_is_init(void);

/* Number of compute units and the shader clock in kHz of the initialised device (decx::cuP.prop, config.h:75). */
int decx_hip_device_info(int* compute_units, int* clock_khz, size_t* hbm_bytes);

/* decx::alloc::_device_malloc / _device_dealloc (core/allocators.h:119-247), without the pool behind them. */
int decx_hip_malloc(void** dptr, size_t bytes);
int decx_hip_free(void* dptr);
/* cudaMemset in _GPU_Matrix::alloc_data_space (classes/GPU_Matrix.h:142-168) */
int decx_hip_memset(void* dptr, int value, size_t bytes);
/* decx::alloc::_host_fixed_page_malloc (cudaHostAlloc, store type Page_Locked, classes/store_types.h:24-28) */
int decx_hip_host_malloc(void** hptr, size_t bytes);
int decx_hip_host_free(void* hptr);
/* cudaMemcpy2D in _GPU_Matrix::Load_from_host / Load_to_host (classes/GPU_Matrix.h:334-354) and the
 * cudaMemcpy2DAsync calls of the host-matrix GEMM (GEMM.h:109-120).  Pitches and width in BYTES. */
int decx_hip_memcpy2d(void* dst, size_t dst_pitch_bytes, const void* src, size_t src_pitch_bytes, size_t width_bytes,
                      size_t rows, int direction);
int decx_hip_memcpy(void* dst, const void* src, size_t bytes, int direction);
/* cudaDeviceSynchronize */
int decx_hip_sync(void);

/* de::cuda::GEMM(GPU_Matrix<float>& A, B, dst)            GEMM.h:398-454  (Cin == NULL)
 * de::cuda::GEMM(GPU_Matrix<float>& A, B, C, dst)         GEMM.h:46       (Cin != NULL, dst = A*B + C)
 * and, between the H2D / D2H copies, the kernel step of the host-matrix overloads (decx::sGEMM_part,
 * GEMM3_macros.h:65-78).  Replaces cu_GEMM_fp32_spec / _ABC_spec (GEMM.cuh:31, :206) and the ragged variants
 * (GEMM_nonuniform.cuh:32-693).
 *   D[i*ldd + j] = Cin[i*ldc + j] + sum_k A[i*lda + k] * B[k*ldb + j],  0<=i<M, 0<=j<N, 0<=k<K, fp32 throughout,
 * evaluated exactly as the reference's kernels do: one accumulator per element, started at Cin (or 0) and updated by
 * a fused multiply-add for k = 0, 1, ..., K-1 (GEMM_kernel_def.cuh:33-55, GEMM.cuh:83-92, :223).  The result is
 * therefore bit-identical to the reference's and does not depend on the kernel or tile shape chosen (results too small
 * to fill the chip with tiles, whatever their K, go to a one-wave-per-16x16-block kernel: the shapes of
 * de::cuda::GEMM_Long_Lr, GEMM/CUDA/extreme_shapes/GEMM_long_Lr.h:22-50, are served here).
 * M, N, K are arbitrary positive sizes: ragged edges are handled inside the kernel, no padded copies are made.
 * Cin may alias D.  Fast path needs A, B 16-byte aligned with lda, ldb multiples of 4 (always true for DECX
 * containers, whose pitch is a multiple of 8 floats, Matrix.h:24-27); otherwise a slower element-wise loader runs. */
int decx_hip_sgemm(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                   int N, int K);
int decx_hip_sgemm_async(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd,
                         int M, int N, int K);

/* de::cuda::GEMM(GPU_Matrix<de::Half>& ...)               GEMM.h:457-519 (+ the A*B+C overload, GEMM.h:49)
 * Replaces cu_GEMM_fp16_spec and its variants (GEMM.cuh:119, :297; GEMM_nonuniform.cuh:712-1334).
 * Operands and result are IEEE binary16 bit patterns (de::Half{unsigned short val}, classes/classes_util.h:58-63).
 * Products are accumulated in fp32 and rounded to binary16 (nearest even) once, on store; the reference accumulates
 * in binary16 (GEMM_kernel_def.cuh:100-121), which this library deliberately does not reproduce.
 * Fast path needs A, B 16-byte aligned with lda, ldb multiples of 8 (DECX pitch is a multiple of 16 halves).
 * Results with very few 128x128 tiles and a long K (say 64 x 65536 x 1024) are computed by K ranges in parallel: each
 * range writes its fp32 partial sums into a plane of its own in a workspace of the library (M*N floats per range;
 * decx_hip_init reserves 2 x CUs x 128 x 128 floats, 32 MiB on an MI355X, which covers every split the library chooses
 * by itself; only a larger forced split grows it, which synchronises the device), the planes are added in range order
 * and the sum is rounded to binary16 once.  Like every reference path the result is therefore the same on every run; decx_hip_set_splitk_mode selects
 * the older scheme in which all ranges add into one plane with atomics, in no fixed order. */
int decx_hip_hgemm_f32acc(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc, uint16_t* D,
                          int ldd, int M, int N, int K);
int decx_hip_hgemm_f32acc_async(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                uint16_t* D, int ldd, int M, int N, int K);

/* How the fp16 entry points (decx_hip_hgemm_f32acc*, decx_hip_conv2_im2col_f16*) combine the K ranges of a product they
 * split over K: 0 (default) = one workspace plane per range, added in range order -- run-to-run reproducible, as every
 * path of the reference is (its long-K kernel is a single chain, GEMM_long_linear_region.cuh:35-55); 1 = atomic adds
 * into one plane, whose order is not fixed (last-bit differences between runs on real-valued data; needs M*N floats
 * of workspace instead of M*N per range).  Returns the previous mode. */
int decx_hip_set_splitk_mode(int mode);

/* decx_hip_hgemm_f32acc for callers that cannot allocate device memory.  It has no counterpart in the reference: it is
 * for tight serving loops and harnesses that forbid hipMalloc (it launches on the library's own stream and waits for the
 * result, so it is not for a stream under graph capture).  Same arguments, arithmetic
 * and result as decx_hip_hgemm_f32acc on its K-range route (`splits` ranges of K; <= 0: the count decx_hip_hgemm_f32acc
 * would choose, 1 if it would not split), but the fp32 planes of the ranges live in a fixed array inside the library's
 * code object, DECX_HIP_STATIC_WORKSPACE_BYTES per GPU, held until the process ends.  It calls no allocating routine.
 * Needs A, B 16-byte aligned with lda, ldb multiples of 8, and M*N*4 bytes times the number of ranges within the
 * workspace: larger problems are refused with DECX_HIP_FAIL_ERROR_PARAMS and a message that says so (they fill the
 * chip without splitting K: decx_hip_hgemm_f32acc does not allocate for them either).  Every call on a GPU uses that
 * GPU's one array: calls that overlap on one GPU (two host threads, two processes' worth of streams) race; nothing in
 * the array has to be zero beforehand, each range overwrites the plane it owns.  Blocks until complete. */
#define DECX_HIP_STATIC_WORKSPACE_BYTES ((size_t)32 << 20)
int decx_hip_hgemm_f32acc_noalloc(const uint16_t* A, int lda, const uint16_t* B, int ldb, const uint16_t* Cin, int ldc,
                                  uint16_t* D, int ldd, int M, int N, int K, int splits);

/* A faster, NOT bit-exact alternative for the shape class of de::cuda::GEMM_Long_Lr(GPU_Matrix<float>& A, B, dst)
 * (GEMM/CUDA/extreme_shapes/GEMM_long_Lr.h:22-50; kernel GEMM_long_linear_region.cuh:73-131): short M, long K, whose
 * M x N tiles alone leave most of the chip idle.  The reference's kernel there is one fused chain per output like all
 * the others, and decx_hip_sgemm follows it bit for bit on these shapes too (with a kernel that gives every 16x16
 * block of the result a wave of its own); that is what the drop-in for GEMM_Long_Lr should call.  This entry point
 * instead cuts K into `splits` ranges (<= 0: chosen from the CU count) that run as separate workgroups and add their
 * partial products to D with fp32 atomics; the order in which ranges are added is not fixed, so results can differ
 * in the last bits from the reference and between runs (integer-valued data stays exact).  About 1.8x faster than the
 * exact path at 64 x 65536 x 1024.  Same arguments and any-shape handling as decx_hip_sgemm (the reference kernel
 * requires M % 16 == 0 and N, K % 64 == 0).  Cin may be NULL or alias D. */
int decx_hip_sgemm_splitk(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                          int N, int K, int splits);

/* Batched GEMM on device-resident data: `batch` independent problems of one shape in ONE launch; problem b uses
 * A + b*stride_a, B + b*stride_b, Cin + b*stride_c (Cin nullable), D + b*stride_d (strides in elements).  This is the
 * kernel step of de::cuda::GEMM3 over a MatrixArray (GEMM/CUDA/large_squares/GEMM3.h:27-36), whose matrices lie
 * `_plane` = pitch*height elements apart (classes/MatrixArray.h:222-239), without its one-launch-per-matrix loop. */
int decx_hip_sgemm_batched(const float* A, int lda, size_t stride_a, const float* B, int ldb, size_t stride_b,
                           const float* Cin, int ldc, size_t stride_c, float* D, int ldd, size_t stride_d, int M, int N, int K,
                           int batch);
int decx_hip_hgemm_f32acc_batched(const uint16_t* A, int lda, size_t stride_a, const uint16_t* B, int ldb, size_t stride_b,
                                  const uint16_t* Cin, int ldc, size_t stride_c, uint16_t* D, int ldd, size_t stride_d, int M,
                                  int N, int K, int batch);

/* de::cuda::GEMM(Matrix<T>& A, B, [C,] dst) on HOST-resident matrices (GEMM.h:56-131, :139-228; decx::sGEMM_part /
 * hGEMM_part, GEMM3_macros.h:65-134): everything between the caller's host buffers -- device allocation, uploads, the
 * kernel, the download -- without the reference's padded device copies (GEMM.h:80-104).  The rows of the result are
 * processed in panels so that the upload of the next panel of A, the kernel and the download of the previous result
 * panel overlap (the reference runs them back to back on one stream).  hA, hB, hC (nullable, may equal hD), hD are
 * HOST pointers; pinned memory (decx_hip_host_malloc) is needed for the overlap, pageable memory works serially.
 * The device blocks stay with the library for the next call (decx_hip_release_tmp gives them back). */
int decx_hip_gemm_host_f32(const float* hA, int lda, const float* hB, int ldb, const float* hC, int ldc, float* hD, int ldd,
                           int M, int N, int K);
int decx_hip_gemm_host_f16(const uint16_t* hA, int lda, const uint16_t* hB, int ldb, const uint16_t* hC, int ldc, uint16_t* hD,
                           int ldd, int M, int N, int K);

/* de::cuda::GEMM3(MatrixArray<T>& A, B, [C,] dst) on HOST-resident arrays (GEMM3.h:40-300): the reference's pipeline of
 * GEMM3_macros.h:140-374 -- upload of matrix i+1, kernel on matrix i and download of result i-1 overlap on three
 * streams with two device buffer sets.  hA, hB, hC (nullable), hD are HOST pointers (pinned memory overlaps best);
 * matrix i of an array starts plane_x elements after matrix i-1.  Device copies keep the host pitches (the reference
 * pads them to 128/16 multiples, GEMM3.h:58-60). */
int decx_hip_gemm3_host_f32(const float* hA, int lda, size_t plane_a, const float* hB, int ldb, size_t plane_b,
                            const float* hC, int ldc, size_t plane_c, float* hD, int ldd, size_t plane_d, int M, int N, int K,
                            int count);
int decx_hip_gemm3_host_f16(const uint16_t* hA, int lda, size_t plane_a, const uint16_t* hB, int ldb, size_t plane_b,
                            const uint16_t* hC, int ldc, size_t plane_c, uint16_t* hD, int ldd, size_t plane_d, int M, int N,
                            int K, int count);

/* de::cuda::Conv2_MK_im2col(Tensor<float>& src, TensorArray<float>& kernel, Tensor<float>& dst, int flag)
 * (convolution/CUDA/im2col/conv2_mk_im2col.h:25, :278-306): the device part, i.e. what cu_sIm2Col_r8_within
 * (im2col.cuh:86-178) followed by cu_conv_eq_mm (eq_GEMM.cuh:109-209) produce.  The patch matrix is never built:
 * the GEMM's A-tile loader reads the tensor directly.
 *   src  : H x W pixels, dpitch channels each (dpitch % 4 == 0), pixel (y,x) at src + y*src_row_stride + x*dpitch
 *          (Tensor.h:389-394);
 *   filt : N filters kh x kw x dpitch, tap (ki,kj) of filter n at filt + n*filt_stride + ki*filt_row_stride + kj*dpitch
 *          (TensorArray.h:521-525);
 *   dst  : dst(y,x,n) at dst + y*dst_row_stride + x*dst_dpitch + n;
 *   flag : DECX_HIP_CONV_ZERO_COMPENSATE -> H x W outputs, input taken as 0 outside the image;
 *          DECX_HIP_CONV_NO_COMPENSATE   -> (H-2*(kh/2)) x (W-2*(kw/2)) outputs;  anything else -> DECX_HIP_FAIL_ERROR_FLAG.
 *   dst(y,x,n) = sum over k = (ki*kw + kj)*dpitch + c, ascending, one fused accumulator (eq_GEMM.cuh:65-74, :172-193),
 *                of src(y+ki-oy, x+kj-ox, c) * filt(n,ki,kj,c),
 *   (oy,ox) = (kh/2, kw/2) for ZERO_COMPENSATE, (0,0) otherwise: cross-correlation, stride 1 (im2col.cuh:150-163).
 * Channels c in [C, dpitch) are read like any other, so the containers' zero padding must be zero.
 * Columns x >= W_out of a dst row (the wpitch padding) are not written.
 * Small images (few 32x32 tiles of the lowered H_out*W_out x N result) run on a one-wave-per-16x16-block kernel instead
 * of the big tiles; the result is the same bit for bit. */
int decx_hip_conv2_im2col_f32(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt, int N,
                              int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst, int dst_dpitch,
                              size_t dst_row_stride, int flag);
int decx_hip_conv2_im2col_f32_async(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag);

/* The convolution above with the layer's element-wise tail applied to each result before it is stored, instead of in
 * passes of their own over dst: an optional per-filter bias (N floats on the device, NULL for none) and, if relu != 0,
 * the activation of de::nn::ReLU_f (nn/operators/ReLU.h:57-82) with its exact arithmetic (see decx_hip_relu_f32).
 *   dst(y,x,n) = relu( conv(y,x,n) + bias[n] ). */
int decx_hip_conv2_im2col_f32_fused(const float* src, int H, int W, int dpitch, size_t src_row_stride, const float* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, float* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag, const float* bias, int relu);

/* The same convolution on binary16 tensors with fp32 accumulation: the fp16 twin of the entry points above, named as a
 * next step beside them; the reference itself has no binary16 im2col convolution (convolution/CUDA/im2col/ holds fp32
 * only), its binary16 containers fix the layout: de::Tensor<de::Half> / de::TensorArray<de::Half> pad the channel
 * pitch to a multiple of 8 halves and the width pitch to a multiple of 4 (classes/Tensor.h:214-235,
 * classes/TensorArray.h:232-256; device twins classes/GPU_Tensor.h:201-222, classes/GPU_TensorArray.h:234-257).
 * All strides and pitches in halves; dpitch % 8 == 0; src and filt 16-byte aligned.  Same index arithmetic, flags and
 * error codes as decx_hip_conv2_im2col_f32.  Products are accumulated in fp32 (in the matrix instruction's order),
 * then   dst(y,x,n) = half( relu( sum + float(bias[n]) ) )   with bias (N halves on the device) and relu optional (NULL / 0),
 * rounded to binary16, nearest even, once.  Checked against fp64 arithmetic on the binary16 inputs to 2e-3 relative.
 * Small images with long filters (few 128x128 tiles of the lowered result, many K steps) are computed as ranges of K
 * that meet in the library's fp32 workspace (the one decx_hip_hgemm uses; grown on demand, kept until the process
 * ends): calls that take this route must not overlap on one GPU, which the library's single stream guarantees. */
int decx_hip_conv2_im2col_f16(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt, int N,
                              int kh, int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst, int dst_dpitch,
                              size_t dst_row_stride, int flag, const uint16_t* bias, int relu);
int decx_hip_conv2_im2col_f16_async(const uint16_t* src, int H, int W, int dpitch, size_t src_row_stride, const uint16_t* filt,
                                    int N, int kh, int kw, size_t filt_stride, size_t filt_row_stride, uint16_t* dst,
                                    int dst_dpitch, size_t dst_row_stride, int flag, const uint16_t* bias, int relu);
/* decx_hip_sgemm followed by de::nn::ReLU_f on the result, in one kernel: D = relu(A*B + Cin). */
int decx_hip_sgemm_relu(const float* A, int lda, const float* B, int ldb, const float* Cin, int ldc, float* D, int ldd, int M,
                        int N, int K);

/* de::nn::ReLU_f(GPU_Matrix<float>& src, dst)                    nn/operators/ReLU.h:28, :57-82, :169-180
 * de::nn::ReLU_f_Rec(src, dst, GPU_Matrix<uchar>& rec_map)       ReLU.h:31, :98-127, :184-195
 * de::nn::ReLU_f_Backward(src, dst, rec_map)                     ReLU.h:34, :131-165, :199-210
 * over n consecutive floats (the reference passes pitch*height, padding included).  Arithmetic as in the reference:
 *   forward : dst[i] = float(sign bit of src[i] clear) * src[i]  -- so negative inputs give -0.0f, -inf gives NaN;
 *   rec     : forward, and byte j of rec_map records floats 8j..8j+7: bit 4+e = float 8j+e kept, bit e = float 8j+4+e
 *             kept (e = 0..3);
 *   backward: dst[i] = float(recorded bit of i) * src[i].
 * src and dst 16-byte aligned (may be the same buffer); rec and backward need n % 8 == 0, rec_map holds n/8 bytes. */
int decx_hip_relu_f32(const float* src, float* dst, size_t n);
int decx_hip_relu_f32_async(const float* src, float* dst, size_t n);
int decx_hip_relu_f32_rec(const float* src, float* dst, unsigned char* rec_map, size_t n);
int decx_hip_relu_f32_backward(const float* src, float* dst, const unsigned char* rec_map, size_t n);

/* de::release_all_tmp (core/memory_management/Memory_pool.h:23-37: releases the blocks its memory pools hold).  The
 * host-matrix entry points (decx_hip_gemm_host_*, decx_hip_gemm3_host_*) keep their device blocks for the next call, as
 * the reference's device pool does (MemoryPool_D.h); this waits for the device and frees them. */
int decx_hip_release_tmp(void);

/* Temporary device blocks from that pool: what decx::alloc::_device_malloc / _device_dealloc are to the reference's host
 * overloads, whose device temporaries come from and go back to decx::mem_pool_D (core/allocators.h:184-189, :137-140;
 * conv2_mk_im2col.h:167-274 takes ker_buf, src_buf, I2C_buf and dst_buf that way).  tmp_free keeps the block for the next
 * tmp_malloc of a similar size; the work that used it must be complete.  Not for blocks a caller keeps: decx_hip_malloc. */
int decx_hip_tmp_malloc(void** dptr, size_t bytes);
int decx_hip_tmp_free(void* dptr);

/* The HIP stream (a hipStream_t) on which every _async entry point enqueues and on which the blocking ones wait: for
 * callers that order work of their own behind the library's (the reference keeps its streams to itself; no
 * counterpart).  NULL before decx_hip_init.  The stream has default priority and does not synchronise with the NULL
 * stream. */
void* decx_hip_stream(void);

/* Timing on the library's own stream (the reference's demos time with clock(), CUDA_GEMM.cpp:43-46, :93-96).
 * start records an event, stop records another, waits for it and returns the elapsed milliseconds. */
int decx_hip_timer_start(void);
int decx_hip_timer_stop(float* milliseconds);

/* Message of the most recent failure on this thread of control ("No error\n" if none), a static string the caller
 * must not free -- the char* error_string of de::DH (handles/decx_handles.h:42-49). */
const char* decx_hip_last_error(void);

/* Tile-shape override for experiments: 0 = automatic choice by problem shape; other values select a fixed
 * kernel variant (tables in backup_1_amd/csrc/sgemm_launch.hpp and hgemm.hip).  Returns the previous value.  fp32 results
 * never depend on it (every shape walks k in the same order); fp16 results can differ in the last bit of the fp32 sum. */
int decx_hip_set_sgemm_variant(int variant);
int decx_hip_set_hgemm_variant(int variant);

/* Host-only (no device call, no counterpart in the reference; usable before decx_hip_init, when 256 compute units are
 * assumed): which kernel decx_hip_sgemm / decx_hip_hgemm_f32acc take for `batch` products of M x N x K with these pitches
 * (elements), computed by the very functions the entry points use -- the number decx_hip_set_*_variant would force that
 * kernel with (tables in backup_1_amd/csrc/sgemm_launch.hpp and hgemm.hip), 0 for operands the vector loaders cannot take
 * (`aligned` = 0: a pointer off the 16-byte grid; or a pitch not in fours / eights), -1 on bad sizes.  The fp16 variant
 * stores the number of K ranges to *splits (nullable) when the answer is 11 (split over K), else 0.  Tests walk these
 * over grids of shapes; nothing in the compute path depends on them. */
int decx_hip_sgemm_plan(int M, int N, int K, int batch, long lda, long ldb, int aligned);
int decx_hip_hgemm_plan(int M, int N, int K, int batch, long lda, long ldb, int aligned, int* splits);

/* Host-only, like the two above: whether decx_hip_sgemm runs the product as two launches -- the rows (columns, when
 * *by_columns is set to 1) that fill whole rounds of a 256-row tile, one tile per compute unit and round, on that tile
 * (*shape = 26, 27 or 28), the rest on a kernel of its own choice (which may be split again) -- and how many rows
 * (columns) the first launch takes; 0 = one launch (*shape = 0), -1 on bad sizes.  Either way every element is the same
 * chain of products (GEMM.h:46 computes it in one launch).  decx_hip_set_sgemm_variant(34) keeps every product in
 * one launch. */
int decx_hip_sgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, int aligned, int* shape, int* by_columns);
/* The same for decx_hip_hgemm_f32acc (GEMM.h:457-519 likewise): the first launch is on the 256x256 tile (variant 15);
 * decx_hip_set_hgemm_variant(20) keeps every product in one launch. */
int decx_hip_hgemm_plan_split(int M, int N, int K, int batch, long lda, long ldb, int aligned, int* by_columns);
/* The same for decx_hip_conv2_im2col_f32 and its fused form (conv2_mk_im2col.h:167-274 runs one launch) where the
 * convolution reaches the register-staged tiles (large images; the small-image, patch and block-chain kernels run in one
 * launch): the output rows of the first launch, on tile *shape (7: 256x256), or 0.  The second
 * launch computes the rows below with the same source tensor, so both sides of the seam see their real neighbours.
 * decx_hip_set_sgemm_variant(34) keeps every convolution in one launch. */
int decx_hip_conv_plan_split(int H, int W, int dpitch, int N, int kh, int kw, int flag, int* shape);

/* Host-only: 1 if the convolution kernels that work on patch-shaped tiles may run on a source tensor of these dimensions
 * (their 32-bit byte offsets, the apron's negative ones and the patches' reach past the output included, stay on the
 * right side of 2^31: see conv_patch_offsets_fit in backup_1_amd/csrc/runtime.hpp), 0 if the library takes its other
 * kernels for it, -1 on bad arguments.  elem_bytes 4 (fp32) or 2 (binary16); strides in elements. */
int decx_hip_conv_patch_offsets_fit(int H, int W, int dpitch, size_t src_row_stride, int kh, int kw, int flag, int elem_bytes);

/* Host-only arithmetic check (no device call, no counterpart in the reference): the largest column index, relative to
 * the B pointer passed to a GEMM entry point, that the vector loaders of a kernel with tile_n-wide tiles fetch when B
 * has N valid columns and is read in groups of `unit` columns (4 for fp32, 8 for fp16) -- computed with the very
 * function the kernels use to place those fetches.  It is N rounded up to `unit`, minus 1, whatever the tile width:
 * B may therefore be a column range of a wider matrix (B = parent + c0, ldb = the parent's pitch, c0 a multiple of
 * `unit`) without any row being read beyond the parent's pitch.  Returns -1 on bad arguments. */
int decx_hip_b_read_extent(int N, int tile_n, int unit);

#ifdef __cplusplus
}
#endif
#endif /* DECX_HIP_H_ */
