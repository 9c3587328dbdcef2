"""Convolutions on tensors just below 2 GiB: the kernels address both tensors with 32-bit byte offsets through buffer
resources, the patch-shaped LDS-DMA kernels in addition throw lanes out of range by adding 2^31, so the last rows of the
largest tensor the library accepts -- and of the largest one its patch kernels accept -- are where an offset would wrap.
Bands of output rows at the top, around the byte offset 2^30 and at the bottom are compared with the oracle on a crop of
the image (bit-equal in fp32; the 2e-3 rule against fp64 in binary16).  A tensor of 2 GiB is refused."""
import ctypes

import numpy as np
import pytest

from backup_1_amd import capi

pytestmark = pytest.mark.gpu

W, C, N, KH, KW = 1024, 64, 8, 3, 3
D2H = 2


def image(H, dtype, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    img = rng.standard_normal((H, W, C), dtype=np.float32)
    return img if dtype == np.float32 else img.astype(np.float16)


def filters(dtype, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    f = (0.1 * rng.standard_normal((N, KH, KW, C), dtype=np.float32))
    fb = np.zeros((N, KH, 4, C), dtype=np.float32)             # TensorArray storage: width pitch ceil4(kw)
    fb[:, :, :KW, :] = f
    return (f, fb) if dtype == np.float32 else (f.astype(np.float16), fb.astype(np.float16))


def rows_of(dD, r0, r1, dst_dpitch, dtype):
    """output rows r0 .. r1-1 of the result on the device"""
    out = np.empty((r1 - r0, W, dst_dpitch), dtype=dtype)
    capi.check(capi.lib().decx_hip_memcpy(out.ctypes.data, dD.ptr + r0 * W * dst_dpitch * out.itemsize, out.nbytes, D2H))
    return out[:, :, :N]


def bands(H):
    mid = (1 << 30) // (W * C * 4)            # the row whose first byte lies 2^30 bytes into an fp32 tensor (2^29 halves likewise)
    return [(0, 6), (mid - 5, mid + 5), (H - 8, H)]


def crop_for(img, r0, r1, H):
    c0, c1 = max(r0 - 1, 0), min(r1 + 1, H)
    return np.ascontiguousarray(img[c0:c1]), r0 - c0


def test_fp32_tensor_just_below_two_gib(gpu, oracle):
    L = capi.lib()
    row_bytes = W * C * 4
    H = (1 << 31) // row_bytes - 1                               # 8191 rows: 2 GiB - 256 KB
    img = image(H, np.float32, 11)
    f, fb = filters(np.float32, 12)
    dS, dF = capi.DeviceBuffer.from_numpy(img), capi.DeviceBuffer.from_numpy(fb)
    dD = capi.DeviceBuffer(H * W * N * 4)
    # the patch kernels (shape 29) stop earlier: the largest H their guard lets through
    H29 = max(h for h in range(H - 64, H + 1) if L.decx_hip_conv_patch_offsets_fit(h, W, C, W * C, KH, KW, 1, 4) == 1)
    assert H29 < H
    for variant, rows in ((0, H), (7, H), (15, H), (29, H29), (30, H29), (29, H)):   # (29, H): the guard sends it elsewhere
        dD.fill(0xff)
        prev = L.decx_hip_set_sgemm_variant(variant)
        try:
            capi.check(L.decx_hip_conv2_im2col_f32(dS.ptr, rows, W, C, W * C, dF.ptr, N, KH, KW, KH * 4 * C, 4 * C, dD.ptr, N, W * N, 1))
        finally:
            L.decx_hip_set_sgemm_variant(prev)
        for r0, r1 in bands(rows):
            crop, skip = crop_for(img[:rows], r0, r1, rows)
            want = oracle.conv2_chain(crop, f, 1)[skip:skip + (r1 - r0)]
            got = rows_of(dD, r0, r1, N, np.float32)
            assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(want).view(np.uint32)), (variant, rows, r0, r1)
    # one more row and the tensor reaches 2 GiB: refused, nothing launched
    rc = L.decx_hip_conv2_im2col_f32(dS.ptr, H + 1, W, C, W * C, dF.ptr, N, KH, KW, KH * 4 * C, 4 * C, dD.ptr, N, W * N, 1)
    assert rc == 0x0d and "2 GiB" in capi.last_error()


def test_fp16_tensor_just_below_two_gib(gpu, oracle):
    L = capi.lib()
    C16 = 2 * C                                                  # 128 halves per pixel: the same 256 KB per image row
    row_bytes = W * C16 * 2
    H = (1 << 31) // row_bytes - 1
    rng = np.random.Generator(np.random.PCG64(21))
    img = rng.standard_normal((H, W, C16), dtype=np.float32).astype(np.float16)
    f = (0.1 * rng.standard_normal((N, KH, KW, C16), dtype=np.float32)).astype(np.float16)
    fb = np.zeros((N, KH, 4, C16), dtype=np.float16)
    fb[:, :, :KW, :] = f
    dS, dF = capi.DeviceBuffer.from_numpy(img.view(np.uint16)), capi.DeviceBuffer.from_numpy(fb.view(np.uint16))
    dD = capi.DeviceBuffer(H * W * N * 2)
    H18 = max(h for h in range(H - 64, H + 1) if L.decx_hip_conv_patch_offsets_fit(h, W, C16, W * C16, KH, KW, 1, 2) == 1)
    assert H18 < H
    for variant, rows in ((0, H), (12, H), (13, H), (14, H), (18, H18), (18, H)):    # (18, H): the guard sends it elsewhere
        dD.fill(0xff)
        prev = L.decx_hip_set_hgemm_variant(variant)
        try:
            capi.check(L.decx_hip_conv2_im2col_f16(dS.ptr, rows, W, C16, W * C16, dF.ptr, N, KH, KW, KH * 4 * C16, 4 * C16, dD.ptr, N, W * N,
                                                   1, None, 0))
        finally:
            L.decx_hip_set_hgemm_variant(prev)
        for r0, r1 in bands(rows):
            crop, skip = crop_for(img[:rows], r0, r1, rows)
            ref, scale = oracle.conv2_f64_f16(crop.view(np.uint16), fb[:, :, :KW].view(np.uint16), 1)
            ref, scale = ref[skip:skip + (r1 - r0)], scale[skip:skip + (r1 - r0)]
            got = rows_of(dD, r0, r1, N, np.float16).astype(np.float64)
            err = np.max((np.abs(got - ref) - np.abs(ref) / 2048.0) / np.maximum(scale, 1e-30))
            assert err < 2e-3, (variant, rows, r0, r1, err)
    rc = L.decx_hip_conv2_im2col_f16(dS.ptr, H + 1, W, C16, W * C16, dF.ptr, N, KH, KW, KH * 4 * C16, 4 * C16, dD.ptr, N, W * N, 1, None, 0)
    assert rc == 0x0d and "2 GiB" in capi.last_error()
