"""Host-side helpers for the GPU parity tests: move numpy data through the C ABI and call the kernels.

Pitched containers are modelled the way DECX lays them out (pitch = width rounded up to 8 floats / 16 halves,
Matrix.h:24-27, :260, :315) with NaN in the padding, so a kernel that lets padding leak into a result fails.
"""
import numpy as np

from backup_1_amd import capi


def pitched(arr, align, fill=np.nan):
    """Copy a 2-D array into storage whose row pitch is a multiple of `align` elements; returns (storage, pitch)."""
    rows, cols = arr.shape
    pitch = (cols + align - 1) // align * align
    buf = np.empty((rows, pitch), dtype=arr.dtype)
    if arr.dtype == np.uint16:
        buf[:] = 0x7E00 if fill is np.nan else fill           # a binary16 NaN
    else:
        buf[:] = fill
    buf[:, :cols] = arr
    return buf, pitch


def gpu_sgemm(A, B, C=None, align=8, variant=0, inplace=False, relu=False):
    M, K = A.shape
    _, N = B.shape
    Ab, lda = pitched(A, align)
    Bb, ldb = pitched(B, align)
    ldd = (N + align - 1) // align * align
    dA, dB = capi.DeviceBuffer.from_numpy(Ab), capi.DeviceBuffer.from_numpy(Bb)
    sentinel = np.full((M, ldd), -12345.0, dtype=np.float32)
    dD = capi.DeviceBuffer.from_numpy(sentinel)
    dC, ldc = None, 0
    if C is not None:
        Cb, ldc = pitched(C, align)
        if inplace:
            dD.upload(Cb)
            dC = dD
        else:
            dC = capi.DeviceBuffer.from_numpy(Cb)
    prev = capi.lib().decx_hip_set_sgemm_variant(variant)
    try:
        if relu:
            capi.check(capi.lib().decx_hip_sgemm_relu(dA.ptr, lda, dB.ptr, ldb, dC.ptr if dC else None, ldc, dD.ptr, ldd,
                                                      M, N, K))
        else:
            capi.sgemm(dA.ptr, lda, dB.ptr, ldb, dD.ptr, ldd, M, N, K, dC.ptr if dC else None, ldc)
    finally:
        capi.lib().decx_hip_set_sgemm_variant(prev)
    out = dD.download((M, ldd), np.float32)
    if not inplace:
        assert np.all(out[:, N:] == -12345.0), "kernel wrote into the pitch padding of dst"
    return out[:, :N].copy()


def gpu_hgemm(Abits, Bbits, Cbits=None, align=16, variant=0):
    M, K = Abits.shape
    _, N = Bbits.shape
    Ab, lda = pitched(Abits, align)
    Bb, ldb = pitched(Bbits, align)
    ldd = (N + align - 1) // align * align
    dA, dB = capi.DeviceBuffer.from_numpy(Ab), capi.DeviceBuffer.from_numpy(Bb)
    dD = capi.DeviceBuffer.from_numpy(np.full((M, ldd), 0x5555, dtype=np.uint16))
    dC, ldc = None, 0
    if Cbits is not None:
        Cb, ldc = pitched(Cbits, align)
        dC = capi.DeviceBuffer.from_numpy(Cb)
    prev = capi.lib().decx_hip_set_hgemm_variant(variant)
    try:
        capi.hgemm(dA.ptr, lda, dB.ptr, ldb, dD.ptr, ldd, M, N, K, dC.ptr if dC else None, ldc)
    finally:
        capi.lib().decx_hip_set_hgemm_variant(prev)
    out = dD.download((M, ldd), np.uint16)
    assert np.all(out[:, N:] == 0x5555), "kernel wrote into the pitch padding of dst"
    return out[:, :N].copy()


def tensor_storage(t, wpitch_align=4, dpitch_align=4, pad_value=np.nan):
    """(H, W, C) -> DECX Tensor storage [H][wpitch][dpitch]: channel padding zero (Tensor.h:312 zero-fills), the
    width padding filled with pad_value.  Returns (storage, wpitch, dpitch)."""
    H, W, C = t.shape
    wp = (W + wpitch_align - 1) // wpitch_align * wpitch_align
    dp = (C + dpitch_align - 1) // dpitch_align * dpitch_align
    buf = np.full((H, wp, dp), pad_value, dtype=np.float32)
    buf[:, :W, :] = 0.0
    buf[:, :W, :C] = t
    return buf, wp, dp


def gpu_conv(src, filt, flag, variant=0, bias=None, relu=False):
    """src (H, W, C), filt (N, kh, kw, C) dense numpy -> dst (H_out, W_out, N), via DECX-style pitched storage.
    bias (N,) and/or relu select the fused entry point."""
    H, W, C = src.shape
    N, kh, kw, _ = filt.shape
    sbuf, swp, dp = tensor_storage(src)
    fb = np.full((N, kh, (kw + 3) // 4 * 4, dp), np.nan, dtype=np.float32)     # TensorArray: wpitch = ceil4(kw)
    fb[:, :, :kw, :] = 0.0
    fb[:, :, :kw, :C] = filt
    fwp = fb.shape[2]
    Hout, Wout = (H, W) if flag == 1 else (H - 2 * (kh // 2), W - 2 * (kw // 2))
    Ho, Wo = max(Hout, 1), max(Wout, 1)
    dwp, ddp = (Wo + 3) // 4 * 4, (N + 3) // 4 * 4
    sentinel = np.full((Ho, dwp, ddp), -777.0, dtype=np.float32)
    dS, dF, dD = (capi.DeviceBuffer.from_numpy(sbuf), capi.DeviceBuffer.from_numpy(fb),
                  capi.DeviceBuffer.from_numpy(sentinel))
    prev = capi.lib().decx_hip_set_sgemm_variant(variant)
    try:
        if bias is None and not relu:
            capi.conv2_im2col(dS.ptr, H, W, dp, swp * dp, dF.ptr, N, kh, kw, kh * fwp * dp, fwp * dp, dD.ptr, ddp,
                              dwp * ddp, flag)
        else:
            dB = capi.DeviceBuffer.from_numpy(np.asarray(bias, dtype=np.float32)) if bias is not None else None
            capi.check(capi.lib().decx_hip_conv2_im2col_f32_fused(
                dS.ptr, H, W, dp, swp * dp, dF.ptr, N, kh, kw, kh * fwp * dp, fwp * dp, dD.ptr, ddp, dwp * ddp, flag,
                dB.ptr if dB else None, 1 if relu else 0))
    finally:
        capi.lib().decx_hip_set_sgemm_variant(prev)
    out = dD.download((Ho, dwp, ddp), np.float32)
    assert np.all(out[:, Wout:, :] == -777.0) and np.all(out[:, :, N:] == -777.0), "kernel wrote into dst padding"
    return out[:Hout, :Wout, :N].copy()


def half_tensor_storage(t16, pad_bits=0x7e00):
    """(H, W, C) float16 -> the reference's binary16 Tensor storage [H][ceil4(W)][ceil8(C)] (Tensor.h:214-235) as uint16
    bit patterns: channel padding zero, width padding filled with pad_bits (a NaN by default)."""
    H, W, C = t16.shape
    wp, dp = (W + 3) // 4 * 4, (C + 7) // 8 * 8
    buf = np.full((H, wp, dp), pad_bits, dtype=np.uint16)
    buf[:, :W, :] = 0
    buf[:, :W, :C] = t16.view(np.uint16)
    return buf, wp, dp


def gpu_hconv(src16, filt16, flag, bias16=None, relu=False, variant=0):
    """fp16 convolution through the C ABI: src16 (H, W, C), filt16 (N, kh, kw, C), bias16 (N,) float16 arrays.
    Returns (dst float16 (H_out, W_out, N), the image storage, the filter storage) -- the storages, as uint16 views
    without their width padding, are what the oracle is fed."""
    H, W, C = src16.shape
    N, kh, kw, _ = filt16.shape
    sbuf, swp, dp = half_tensor_storage(src16)
    fwp = (kw + 3) // 4 * 4
    fb = np.full((N, kh, fwp, dp), 0x7e00, dtype=np.uint16)
    fb[:, :, :kw, :] = 0
    fb[:, :, :kw, :C] = filt16.view(np.uint16)
    Hout, Wout = (H, W) if flag == 1 else (H - 2 * (kh // 2), W - 2 * (kw // 2))
    Ho, Wo = max(Hout, 1), max(Wout, 1)
    dwp, ddp = (Wo + 3) // 4 * 4, (N + 7) // 8 * 8
    sentinel = np.full((Ho, dwp, ddp), 0xd610, dtype=np.uint16)          # -97.0
    dS, dF, dD = (capi.DeviceBuffer.from_numpy(sbuf), capi.DeviceBuffer.from_numpy(fb),
                  capi.DeviceBuffer.from_numpy(sentinel))
    dB = capi.DeviceBuffer.from_numpy(np.asarray(bias16, dtype=np.float16).view(np.uint16)) if bias16 is not None else None
    prev = capi.lib().decx_hip_set_hgemm_variant(variant)      # 12 / 13: the register-staged / the LDS-DMA kernel
    try:
        capi.check(capi.lib().decx_hip_conv2_im2col_f16(dS.ptr, H, W, dp, swp * dp, dF.ptr, N, kh, kw, kh * fwp * dp, fwp * dp,
                                                        dD.ptr, ddp, dwp * ddp, flag, dB.ptr if dB else None, 1 if relu else 0))
    finally:
        capi.lib().decx_hip_set_hgemm_variant(prev)
    out = dD.download((Ho, dwp, ddp), np.uint16)
    assert np.all(out[:, Wout:, :] == 0xd610) and np.all(out[:, :, N:] == 0xd610), "kernel wrote into dst padding"
    return out[:Hout, :Wout, :N].copy().view(np.float16), sbuf[:, :W], fb[:, :, :kw]


def rel_err_vs_abs_scale(got, ref, scale):
    """max |got - ref| / sum_k |a||b|: the relative-error definition used for the fp32 / fp16 tolerances (a bound
    any correct summation order satisfies, and well-defined where the reference value itself is near zero)."""
    return float(np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64)) / np.maximum(scale, 1e-300)))
