"""Products that decx_hip_sgemm runs as two launches (whole rounds of a 256-row tile, then the rest on a kernel of its
own choice; decx_hip_sgemm_plan_split says which): every element is the same chain of products whatever tile computes
it, so the result has to be the one-launch result (decx_hip_set_sgemm_variant(34)) bit for bit -- on real-valued data,
with and without "+ C", in place, with the ReLU epilogue -- and exact on small integers, at the seam above all.
decx_hip_hgemm_f32acc does the same on its 256x256 tile (decx_hip_hgemm_plan_split; variant 20 = one launch): exact on
small integers, and within the path's 2e-3 rule of the fp64 product on real-valued data on both sides of the seam."""
import ctypes

import numpy as np
import pytest

from backup_1_amd import capi, workloads
from gpu_helpers import gpu_sgemm, gpu_hgemm

pytestmark = pytest.mark.gpu

# (M, K, N): split by rows on the 256x256 tile, by columns on 256x224 and on 256x192, by rows on 256x192 with ragged edges
SHAPES = [(4352, 512, 4352), (4096, 512, 4608), (2048, 512, 6212), (6324, 520, 5986)]


def planned_split(M, K, N):
    shape, by_columns = ctypes.c_int(0), ctypes.c_int(0)
    first = capi.lib().decx_hip_sgemm_plan_split(M, N, K, 1, (K + 7) // 8 * 8, (N + 7) // 8 * 8, 1, ctypes.byref(shape), ctypes.byref(by_columns))
    return first, shape.value, by_columns.value


@pytest.mark.parametrize("shape", SHAPES)
def test_two_launches_give_the_bits_of_one(gpu, shape):
    M, K, N = shape
    first, tile, by_columns = planned_split(M, K, N)
    assert first > 0 and tile in (26, 27, 28), "the shape is meant to be one the library splits"
    A, B, C = workloads.normal((M, K), 61), workloads.normal((K, N), 62), workloads.normal((M, N), 63)
    for kwargs in ({}, {"C": C}, {"C": C, "inplace": True}, {"relu": True}):
        two = gpu_sgemm(A, B, **kwargs)
        one = gpu_sgemm(A, B, variant=34, **kwargs)
        assert np.array_equal(two.view(np.uint32), one.view(np.uint32)), (shape, sorted(kwargs))


@pytest.mark.parametrize("shape", SHAPES[:3])
def test_two_launches_exact_on_small_integers(gpu, shape):
    M, K, N = shape
    assert planned_split(M, K, N)[0] > 0
    A, B = workloads.small_ints((M, K), 64, -2, 2), workloads.small_ints((K, N), 65, -2, 2)
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    got = gpu_sgemm(A, B)
    assert np.array_equal(got, want), shape


def test_rows_at_the_seam_match_the_oracle_chain(gpu, oracle):
    M, K, N = SHAPES[0]
    first, _, by_columns = planned_split(M, K, N)
    assert first > 0 and not by_columns
    A, B = workloads.normal((M, K), 66), workloads.normal((K, N), 67)
    got = gpu_sgemm(A, B)
    rows = [0, first - 1, first, first + 1, M - 1]
    want = oracle.sgemm_chain(np.ascontiguousarray(A[rows]), B)
    assert np.array_equal(got[rows].view(np.uint32), want.view(np.uint32))


H_SHAPES = [(4352, 1024, 4352), (2048, 1024, 8448), (4013, 1032, 4775)]


def planned_hsplit(M, K, N):
    by_columns = ctypes.c_int(0)
    first = capi.lib().decx_hip_hgemm_plan_split(M, N, K, 1, (K + 15) // 16 * 16, (N + 15) // 16 * 16, 1, ctypes.byref(by_columns))
    return first, by_columns.value


@pytest.mark.parametrize("shape", H_SHAPES)
def test_fp16_two_launches_exact_on_small_integers(gpu, shape):
    M, K, N = shape
    assert planned_hsplit(M, K, N)[0] > 0, "the shape is meant to be one the library splits"
    A, B = workloads.small_ints((M, K), 71, -1, 1), workloads.small_ints((K, N), 72, -1, 1)
    C = workloads.small_ints((M, N), 73, -30, 30)
    want = A.astype(np.float64) @ B.astype(np.float64)
    h = lambda x: x.astype(np.float16).view(np.uint16)
    for with_c in (False, True):
        two = gpu_hgemm(h(A), h(B), h(C) if with_c else None)
        one = gpu_hgemm(h(A), h(B), h(C) if with_c else None, variant=20)
        assert np.array_equal(two, one), (shape, with_c)
        assert np.array_equal(two.view(np.float16).astype(np.float64), want + (C if with_c else 0.0)), (shape, with_c)


def test_fp16_rows_around_the_seam_within_the_rule(gpu):
    M, K, N = H_SHAPES[0]
    first, by_columns = planned_hsplit(M, K, N)
    assert first > 0 and not by_columns
    A, B = workloads.normal((M, K), 74).astype(np.float16), workloads.normal((K, N), 75).astype(np.float16)
    got = gpu_hgemm(A.view(np.uint16), B.view(np.uint16)).view(np.float16).astype(np.float64)
    rows = [0, 1, first - 2, first - 1, first, first + 1, M - 2, M - 1]
    ref = A[rows].astype(np.float64) @ B.astype(np.float64)
    scale = np.abs(A[rows].astype(np.float64)) @ np.abs(B.astype(np.float64))
    err = np.max((np.abs(got[rows] - ref) - np.abs(ref) / 2048.0) / np.maximum(scale, 1e-30))     # beyond the rounding of the result to binary16
    assert err < 2e-3, err


# (H, W, C, N, flag): convolutions that reach the register-staged tiles and split by output rows (decx_hip_conv_plan_split)
CONV_SHAPES = [(274, 274, 64, 512, 1), (300, 300, 128, 256, 1), (350, 350, 96, 512, 0)]


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_convolution_in_two_launches(gpu, oracle, shape):
    from gpu_helpers import gpu_conv
    H, W, C, N, flag = shape
    tile = ctypes.c_int(0)
    rows = capi.lib().decx_hip_conv_plan_split(H, W, C, N, 3, 3, flag, ctypes.byref(tile))
    assert rows > 0 and tile.value == 7, "the shape is meant to be one the library splits"
    src, filt = workloads.normal((H, W, C), 81), 0.1 * workloads.normal((N, 3, 3, C), 82)
    bias = workloads.normal((N,), 83)
    two, one = gpu_conv(src, filt, flag), gpu_conv(src, filt, flag, variant=34)
    assert np.array_equal(two.view(np.uint32), one.view(np.uint32)), shape
    two, one = gpu_conv(src, filt, flag, bias=bias, relu=True), gpu_conv(src, filt, flag, variant=34, bias=bias, relu=True)
    assert np.array_equal(two.view(np.uint32), one.view(np.uint32)), shape
    # the output rows on both sides of the seam against the oracle's chain, computed on a crop of the image that gives
    # every one of them its real neighbours
    a, b = rows - 2, rows + 2
    if flag:
        crop = np.ascontiguousarray(src[a - 2:b + 2])
        want = oracle.conv2_chain(crop, filt, 1)[2:2 + (b - a)]
    else:
        crop = np.ascontiguousarray(src[a:b + 2])                 # valid region: output row r reads image rows r .. r + 2
        want = oracle.conv2_chain(crop, filt, 0)
    got = gpu_conv(src, filt, flag)[a:b]
    assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(want).view(np.uint32)), shape


@pytest.mark.parametrize("shape", [(260, 264, 128, 256, 1), (358, 362, 64, 512, 0)])
def test_fp16_convolution_in_two_launches(gpu, oracle, shape):
    """289 (1058) tiles of 256 pixels x 256 filters on 256 compute units: whole rounds of them, then the rows below on tiles of
    their own.  The same bits as one launch (hgemm variant 20), with bias and ReLU too, and the rows around the seam --
    image row 240 (352) -- within the path's 2e-3 rule of the fp64 convolution of the same binary16 tensors."""
    from gpu_helpers import gpu_hconv
    H, W, C, N, flag = shape
    src = workloads.normal((H, W, C), 91).astype(np.float16)
    filt = (0.1 * workloads.normal((N, 3, 3, C), 92)).astype(np.float16)
    bias = workloads.normal((N,), 93).astype(np.float16)
    two, sbuf, fbuf = gpu_hconv(src, filt, flag)
    one, _, _ = gpu_hconv(src, filt, flag, variant=20)
    assert np.array_equal(two.view(np.uint16), one.view(np.uint16)), shape
    two_b, _, _ = gpu_hconv(src, filt, flag, bias16=bias, relu=True)
    one_b, _, _ = gpu_hconv(src, filt, flag, bias16=bias, relu=True, variant=20)
    assert np.array_equal(two_b.view(np.uint16), one_b.view(np.uint16)), shape
    Hout = H if flag else H - 2
    tiles_per_patch_row = -(-(W if flag else W - 2) // 16) * -(-N // 256)
    seam = (-(-Hout // 16) * tiles_per_patch_row // 256) * 256 // tiles_per_patch_row * 16
    assert 0 < seam < Hout
    a, b = seam - 3, seam + 3
    if flag:
        crop = np.ascontiguousarray(sbuf[a - 2:b + 2])
        ref, scale = oracle.conv2_f64_f16(crop, fbuf, 1)
        ref, scale = ref[2:2 + (b - a)], scale[2:2 + (b - a)]
    else:
        crop = np.ascontiguousarray(sbuf[a:b + 2])
        ref, scale = oracle.conv2_f64_f16(crop, fbuf, 0)
    got = two[a:b].astype(np.float64)
    err = np.max((np.abs(got - ref) - np.abs(ref) / 2048.0) / np.maximum(scale, 1e-30))
    assert err < 2e-3, (shape, err)
