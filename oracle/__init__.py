"""CPU oracle for DECX's dense-contraction path -- TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this package.
The product package never does.  The arithmetic and the reference citations live in ``decx_oracle.cpp``; this
module is the numpy/ctypes face of it.  All matrices are row-major numpy arrays; a 2-D array's row stride is its
pitch, so pitched DECX containers can be modelled by slicing a wider array.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        P, I, L_ = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
        L.oracle_sgemm_chain.argtypes = [P, L_, P, L_, P, L_, P, L_, I, I, I]
        L.oracle_sgemm_chain.restype = None
        L.oracle_sgemm_chain_fast.argtypes = [P, L_, P, L_, P, L_, P, L_, I, I, I, I]
        L.oracle_sgemm_chain_fast.restype = None
        L.oracle_sgemm_chain_rows.argtypes = [P, L_, P, L_, P, I, P, I, I, I]
        L.oracle_sgemm_chain_rows.restype = None
        L.oracle_decx_cpu_sgemm.argtypes = [P, L_, P, L_, P, L_, I, I, I, I]
        L.oracle_decx_cpu_sgemm.restype = I
        L.oracle_conv2_chain.argtypes = [P, I, I, I, L_, P, I, I, I, L_, L_, P, I, L_, I, I]
        L.oracle_conv2_chain.restype = I
        L.oracle_conv2_f64_f16.argtypes = [P, I, I, I, L_, P, I, I, I, L_, L_, P, P, I, I]
        L.oracle_conv2_f64_f16.restype = I
        L.oracle_float_to_half.argtypes = [P, P, L_]
        L.oracle_float_to_half.restype = None
        L.oracle_half_to_float.argtypes = [P, P, L_]
        L.oracle_half_to_float.restype = None
        L.oracle_gemm_f64_rows_f16.argtypes = [P, L_, P, L_, P, I, P, P, I, I, I]
        L.oracle_gemm_f64_rows_f16.restype = None
        L.oracle_gemm_f64_rows_f32.argtypes = [P, L_, P, L_, P, I, P, P, I, I, I]
        L.oracle_gemm_f64_rows_f32.restype = None
        L.oracle_relu_f32.argtypes = [P, P, L_]
        L.oracle_relu_f32.restype = None
        L.oracle_relu_f32_rec.argtypes = [P, P, P, L_]
        L.oracle_relu_f32_rec.restype = None
        L.oracle_relu_f32_backward.argtypes = [P, P, P, L_]
        L.oracle_relu_f32_backward.restype = None
        L.oracle_pool_size.argtypes = [I]
        L.oracle_pool_size.restype = I
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _ld(a):
    assert a.ndim == 2 and a.strides[1] == a.itemsize, "row-major rows required"
    assert a.strides[0] % a.itemsize == 0
    return a.strides[0] // a.itemsize


def _f32(a):
    assert a.dtype == np.float32
    return a


def sgemm_chain(A, B, C=None, fast=True, nthreads=0):
    """D = A @ B (+ C) as the reference computes it: one fp32 accumulator per element, fused multiply-add,
    k ascending.  ``fast=False`` runs the scalar definitional loop."""
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    D = np.empty((M, N), dtype=np.float32)
    cp, ldc = (None, 0) if C is None else (_p(_f32(C)), _ld(C))
    if fast:
        lib().oracle_sgemm_chain_fast(_p(A), _ld(A), _p(B), _ld(B), cp, ldc, _p(D), N, M, N, K, nthreads)
    else:
        lib().oracle_sgemm_chain(_p(A), _ld(A), _p(B), _ld(B), cp, ldc, _p(D), N, M, N, K)
    return D


def sgemm_chain_rows(A, B, rows, nthreads=0):
    A, B = _f32(A), _f32(B)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    K, N = B.shape
    out = np.empty((len(rows), N), dtype=np.float32)
    lib().oracle_sgemm_chain_rows(_p(A), _ld(A), _p(B), _ld(B), _p(rows), len(rows), _p(out), N, K, nthreads)
    return out


def decx_cpu_sgemm(A, B, nthreads=0, out=None):
    """The restated DECX_cpu thread-pool SGEMM.  B and the output need a pitch >= ceil8(N); pass arrays sliced
    from pitched storage, or let this function pad them."""
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    _, N = B.shape
    n8 = (N + 7) // 8 * 8
    if _ld(B) < n8:
        Bp = np.zeros((K, n8), dtype=np.float32)
        Bp[:, :N] = B
        B = Bp[:, :N]
    if out is None:
        out = np.zeros((M, n8), dtype=np.float32)[:, :N]
    assert _ld(out) >= n8
    rc = lib().oracle_decx_cpu_sgemm(_p(A), _ld(A), _p(B), _ld(B), _p(out), _ld(out), M, N, K, nthreads)
    if rc != 0:
        raise ValueError("oracle_decx_cpu_sgemm rejected its arguments")
    return out


def pool_size(nthreads=0):
    return lib().oracle_pool_size(nthreads)


def conv2_chain(src, filt, flag, nthreads=0):
    """src: (H, W, dpitch) float32, row stride may be padded (src.strides[0]); filt: (N, kh, kw, dpitch) with
    arbitrary filter / filter-row strides; returns dst (H_out, W_out, N) float32 dense.
    flag 1 = same size with zero border, flag 0 = valid region."""
    src, filt = _f32(src), _f32(filt)
    H, W, dp = src.shape
    N, kh, kw, dp2 = filt.shape
    assert dp == dp2
    assert src.strides[2] == 4 and src.strides[1] == 4 * dp
    assert filt.strides[3] == 4 and filt.strides[2] == 4 * dp
    Hout, Wout = (H, W) if flag == 1 else (H - 2 * (kh // 2), W - 2 * (kw // 2))
    dst = np.zeros((max(Hout, 0), max(Wout, 0), N), dtype=np.float32)
    rc = lib().oracle_conv2_chain(_p(src), H, W, dp, src.strides[0] // 4, _p(filt), N, kh, kw, filt.strides[0] // 4,
                                  filt.strides[1] // 4, _p(dst), N, Wout * N if Wout > 0 else 0, flag, nthreads)
    if rc != 0:
        raise ValueError("oracle_conv2_chain rejected its arguments (flag %r)" % (flag,))
    return dst


def float_to_half(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().oracle_float_to_half(_p(x), _p(out), x.size)
    return out


def half_to_float(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().oracle_half_to_float(_p(h), _p(out), h.size)
    return out


def gemm_f64_rows_f16(A_bits, B_bits, rows, nthreads=0):
    """fp64 reference rows for binary16 operands given as uint16 bit patterns.  Returns (ref, abs_scale)."""
    assert A_bits.dtype == np.uint16 and B_bits.dtype == np.uint16
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    K, N = B_bits.shape
    out = np.empty((len(rows), N), dtype=np.float64)
    ab = np.empty((len(rows), N), dtype=np.float64)
    lib().oracle_gemm_f64_rows_f16(_p(A_bits), _ld(A_bits), _p(B_bits), _ld(B_bits), _p(rows), len(rows), _p(out),
                                   _p(ab), N, K, nthreads)
    return out, ab


def gemm_f64_rows_f32(A, B, rows, nthreads=0):
    A, B = _f32(A), _f32(B)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    K, N = B.shape
    out = np.empty((len(rows), N), dtype=np.float64)
    ab = np.empty((len(rows), N), dtype=np.float64)
    lib().oracle_gemm_f64_rows_f32(_p(A), _ld(A), _p(B), _ld(B), _p(rows), len(rows), _p(out), _p(ab), N, K, nthreads)
    return out, ab


def conv2_f64_f16(src_bits, filt_bits, flag, nthreads=0):
    """fp64 convolution of binary16 tensors given as uint16 bit patterns: src (H, W, dpitch), filt (N, kh, kw, dpitch),
    strides as in conv2_chain.  Returns (out, scale), both (H_out, W_out, N) float64: the sums of products and of their
    absolute values.  flag 1 = same size with zero border, flag 0 = valid region."""
    src = np.asarray(src_bits)
    filt = np.asarray(filt_bits)
    assert src.dtype == np.uint16 and filt.dtype == np.uint16
    H, W, dp = src.shape
    N, kh, kw, dp2 = filt.shape
    assert dp == dp2
    assert src.strides[2] == 2 and src.strides[1] == 2 * dp
    assert filt.strides[3] == 2 and filt.strides[2] == 2 * dp
    Hout, Wout = (H, W) if flag == 1 else (H - 2 * (kh // 2), W - 2 * (kw // 2))
    out = np.zeros((max(Hout, 0), max(Wout, 0), N), dtype=np.float64)
    scale = np.zeros_like(out)
    rc = lib().oracle_conv2_f64_f16(_p(src), H, W, dp, src.strides[0] // 2, _p(filt), N, kh, kw, filt.strides[0] // 2,
                                    filt.strides[1] // 2, _p(out), _p(scale), flag, nthreads)
    if rc != 0:
        raise ValueError("oracle_conv2_f64_f16 rejected its arguments (flag %r)" % (flag,))
    return out, scale


def relu(x):
    """de::nn::ReLU_f arithmetic (nn/operators/ReLU.h:57-82) on a float32 array of any shape."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    lib().oracle_relu_f32(_p(x), _p(out), x.size)
    return out


def relu_rec(x):
    """ReLU_f_Rec (ReLU.h:98-127): (dst, rec_map) with one map byte per 8 floats; x.size must be a multiple of 8."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size % 8 == 0
    out = np.empty_like(x)
    rec = np.empty(x.size // 8, dtype=np.uint8)
    lib().oracle_relu_f32_rec(_p(x), _p(out), _p(rec), x.size)
    return out, rec


def relu_backward(x, rec):
    """ReLU_f_Backward (ReLU.h:131-165)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rec = np.ascontiguousarray(rec, dtype=np.uint8)
    assert x.size % 8 == 0 and rec.size == x.size // 8
    out = np.empty_like(x)
    lib().oracle_relu_f32_backward(_p(x), _p(out), _p(rec), x.size)
    return out
