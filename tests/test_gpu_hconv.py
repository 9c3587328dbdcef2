"""fp16 convolution (decx_hip_conv2_im2col_f16, backup_1_amd/csrc/hconv_tile.hpp) through the C ABI.

The reference has no binary16 im2col convolution to compare bits with; the bar is the fp16 rule of this build: fp32
accumulation, at most 2e-3 relative to fp64 arithmetic on the same binary16 inputs (relative to sum |a||b|, plus the
half-ulp of the final rounding to binary16), and exact results wherever binary16 can hold them (small integers)."""
import numpy as np
import pytest

from backup_1_amd import capi, workloads
from gpu_helpers import gpu_hconv

pytestmark = pytest.mark.gpu

TOL = 2e-3


def check_against_f64(oracle, got16, sbuf, fb, flag, bias16=None, relu=False):
    ref, scale = oracle.conv2_f64_f16(sbuf, fb, flag)
    if bias16 is not None:
        b = np.asarray(bias16, np.float16).astype(np.float64)
        ref = ref + b[None, None, :]
        scale = scale + np.abs(b)[None, None, :]
    if relu:
        ref = np.maximum(ref, 0.0)
    got = got16.astype(np.float64)
    # fp32 accumulation error relative to sum |a||b|, and the one rounding to binary16 relative to the value itself
    bound = TOL * scale + 2.0 ** -11 * np.abs(ref) + 2.0 ** -24
    assert np.all(np.isfinite(got))
    worst = np.max(np.abs(got - ref) / np.maximum(bound, 1e-300))
    assert worst <= 1.0, worst
    acc_err = np.max((np.abs(got - ref) - 2.0 ** -11 * np.abs(ref) - 2.0 ** -24) / np.maximum(scale, 1e-300))
    return max(acc_err, 0.0)


CASES = [(20, 22, 8, 6, 3, 3), (9, 13, 3, 2, 3, 3), (16, 16, 64, 128, 3, 3), (33, 17, 24, 130, 1, 1), (12, 40, 16, 5, 5, 3),
         (40, 12, 40, 7, 3, 5), (7, 7, 8, 1, 7, 7), (64, 48, 32, 200, 3, 3), (10, 12, 128, 20, 3, 3), (9, 70, 64, 3, 1, 5)]


@pytest.mark.parametrize("flag", [1, 0])
@pytest.mark.parametrize("case", CASES)
def test_small_integers_are_exact(gpu, oracle, case, flag):
    # |values| <= 2, at most 8 taps... products summed stay below 2048, where binary16 holds every integer
    H, W, C, N, kh, kw = case
    if flag == 0 and (H <= 2 * (kh // 2) or W <= 2 * (kw // 2)):
        pytest.skip("no valid region")
    src = workloads.small_ints((H, W, C), 801, -1, 1).astype(np.float16)
    filt = workloads.small_ints((N, kh, kw, C), 802, -1, 1).astype(np.float16)
    got, sbuf, fb = gpu_hconv(src, filt, flag)
    ref, scale = oracle.conv2_f64_f16(sbuf, fb, flag)
    assert scale.max() < 2048
    assert np.array_equal(got.astype(np.float64), ref)


@pytest.mark.parametrize("flag", [1, 0])
@pytest.mark.parametrize("case", CASES)
def test_real_values_within_tolerance(gpu, oracle, case, flag):
    H, W, C, N, kh, kw = case
    if flag == 0 and (H <= 2 * (kh // 2) or W <= 2 * (kw // 2)):
        pytest.skip("no valid region")
    src = workloads.uniform_01((H, W, C), 811).astype(np.float16)
    filt = workloads.normal((N, kh, kw, C), 812, sigma=0.05).astype(np.float16)
    got, sbuf, fb = gpu_hconv(src, filt, flag)
    assert check_against_f64(oracle, got, sbuf, fb, flag) < TOL


def test_all_ones_counts_taps_and_impulse_returns_the_reversed_filter(gpu):
    H, W, C, N = 11, 14, 16, 4
    got, _, _ = gpu_hconv(np.ones((H, W, C), np.float16), np.ones((N, 3, 3, C), np.float16), 1)
    assert np.all(got[1:-1, 1:-1] == 9 * C) and np.all(got[0, 1:-1] == 6 * C) and np.all(got[-1, -1] == 4 * C)
    filt = workloads.normal((N, 3, 5, C), 821).astype(np.float16)
    src = np.zeros((H, W, C), np.float16)
    src[5, 6, 3] = 1.0
    got, _, _ = gpu_hconv(src, filt, 1)
    for di in (-1, 0, 1):
        for dj in (-2, -1, 0, 1, 2):
            assert np.array_equal(got[5 - di, 6 - dj, :].view(np.uint16), filt[:, 1 + di, 2 + dj, 3].view(np.uint16))
    got[4:7, 4:9] = 0
    assert not got.any()


def test_bias_and_relu_in_the_epilogue(gpu, oracle):
    H, W, C, N = 30, 26, 24, 70
    src = workloads.normal((H, W, C), 831).astype(np.float16)
    filt = workloads.normal((N, 3, 3, C), 832, sigma=0.1).astype(np.float16)
    bias = workloads.normal((N,), 833).astype(np.float16)
    for b, r in ((bias, False), (None, True), (bias, True)):
        got, sbuf, fb = gpu_hconv(src, filt, 1, bias16=b, relu=r)
        check_against_f64(oracle, got, sbuf, fb, 1, bias16=b, relu=r)
        if r:
            assert not np.any(got.astype(np.float64) < 0)
    # ReLU by sign as in nn/operators/ReLU.h:57-82: a negative sum becomes -0.0
    got, _, _ = gpu_hconv(-np.ones((4, 4, 8), np.float16), np.ones((1, 1, 1, 8), np.float16), 1, relu=True)
    assert np.all(got.view(np.uint16) == 0x8000)


def test_headline_shape_sampled(gpu, oracle):
    # 224x224x64 image, 128 filters 3x3x64, same size: the fp32 conv config in binary16
    src = workloads.uniform_01((224, 224, 64), 841).astype(np.float16)
    filt = workloads.normal((128, 3, 3, 64), 842, sigma=0.05).astype(np.float16)
    got, sbuf, fb = gpu_hconv(src, filt, 1)
    assert check_against_f64(oracle, got, sbuf, fb, 1) < TOL
    # the library's choice is the tap-row kernel; the LDS-DMA and the register-staged kernels must agree with it to the
    # rounding of the result (they add the same fp32 products in another order)
    for variant in (12, 13, 14, 18, 19):
        other, _, _ = gpu_hconv(src, filt, 1, variant=variant)
        diff = np.abs(other.astype(np.float64) - got.astype(np.float64))
        assert np.all(diff <= 2.0 ** -9 * np.maximum(np.abs(got.astype(np.float64)), 1.0)), variant


def test_many_pixels_take_the_tall_tile(gpu, oracle):
    # enough 256-pixel tiles to cover most CUs: the 256x128 tile shape of hconv_enqueue
    H, W, C, N = 384, 400, 8, 9
    src = workloads.normal((H, W, C), 851).astype(np.float16)
    filt = workloads.normal((N, 3, 3, C), 852, sigma=0.2).astype(np.float16)
    got, sbuf, fb = gpu_hconv(src, filt, 1)
    assert check_against_f64(oracle, got, sbuf, fb, 1) < TOL
    si = workloads.small_ints((H, W, C), 853, -2, 2).astype(np.float16)
    fi = workloads.small_ints((N, 3, 3, C), 854, -2, 2).astype(np.float16)
    got, sbuf, fb = gpu_hconv(si, fi, 0)
    ref, _ = oracle.conv2_f64_f16(sbuf, fb, 0)
    assert np.array_equal(got.astype(np.float64), ref)


@pytest.mark.parametrize("case", [(14, 14, 128, 40, 3, 3), (12, 10, 120, 70, 3, 3), (7, 7, 512, 130, 3, 3), (9, 5, 64, 16, 5, 5)])
def test_small_images_split_the_walk_over_k(gpu, oracle, case):
    # few 128-pixel tiles and many K steps: ranges of K steps run as separate workgroups and meet in an fp32 workspace;
    # bias, ReLU and the rounding happen in the finishing kernel.  Integer data exact, real data within the fp16 rule.
    H, W, C, N, kh, kw = case
    si = workloads.small_ints((H, W, C), 861, -1, 1).astype(np.float16)
    fi = workloads.small_ints((N, kh, kw, C), 862, -1, 1).astype(np.float16)
    for flag in (1, 0):
        got, sbuf, fb = gpu_hconv(si, fi, flag)
        ref, _ = oracle.conv2_f64_f16(sbuf, fb, flag)
        assert np.array_equal(got.astype(np.float64), ref)
    src = workloads.normal((H, W, C), 863).astype(np.float16)
    filt = workloads.normal((N, kh, kw, C), 864, sigma=0.05).astype(np.float16)
    bias = workloads.normal((N,), 865).astype(np.float16)
    for b, r in ((None, False), (bias, True)):
        got, sbuf, fb = gpu_hconv(src, filt, 1, bias16=b, relu=r)
        assert check_against_f64(oracle, got, sbuf, fb, 1, bias16=b, relu=r) < TOL


def test_split_walk_over_k_is_the_same_on_every_run(gpu, oracle):
    # 14x14x512 under 512 filters of 3x3: two 128-pixel tiles by four filter tiles and 72 K steps -- split over K.  The
    # ranges' planes are added in range order, so real-valued data give the same bits on every run.
    src = workloads.normal((14, 14, 512), 866).astype(np.float16)
    filt = workloads.normal((512, 3, 3, 512), 867, sigma=0.05).astype(np.float16)
    first, sbuf, fb = gpu_hconv(src, filt, 1)
    for _ in range(3):
        again, _, _ = gpu_hconv(src, filt, 1)
        assert np.array_equal(again.view(np.uint16), first.view(np.uint16))
    assert check_against_f64(oracle, first, sbuf, fb, 1) < TOL
    prev = capi.lib().decx_hip_set_splitk_mode(1)
    try:
        atomic, _, _ = gpu_hconv(src, filt, 1)
    finally:
        capi.lib().decx_hip_set_splitk_mode(prev)
    assert check_against_f64(oracle, atomic, sbuf, fb, 1) < TOL
    # the two ways of combining the ranges add the same fp32 partial sums in another order: a few fp32 ulps of the sum's
    # scale apart at most, which the one rounding to binary16 turns into at most one binary16 ulp of the result
    ref, scale = oracle.conv2_f64_f16(sbuf, fb, 1)
    diff = np.abs(atomic.astype(np.float64) - first.astype(np.float64))
    assert np.all(diff <= 2.0 ** -10 * np.abs(ref) + 1e-5 * scale + 2.0 ** -24)


# channel pitch a multiple of 64 halves: a K step lies inside one tap, which is what the LDS-DMA kernel needs.  It is the
# default from about 200 tiles of 256 pixels on; variant 13 takes it for any image, 12 keeps the register-staged kernel, 14
# takes the kernel that loads a tap row's pixels once for all of its taps (filters 3, 5 or 7 wide).
DMA_CASES = [(20, 22, 64, 6, 3, 3), (16, 16, 64, 128, 3, 3), (33, 17, 128, 130, 1, 1), (12, 40, 64, 5, 5, 3), (7, 7, 64, 1, 7, 7),
             (64, 48, 64, 200, 3, 3), (30, 26, 192, 70, 3, 3), (40, 37, 60, 33, 3, 3), (40, 44, 64, 20, 5, 5), (36, 60, 64, 9, 7, 7),
             (300, 20, 128, 140, 3, 5)]


# 18 takes the kernel on 16x16x32 matrix instructions with patch-shaped tiles (256 filters wide above 128 filters), 19 keeps it out
@pytest.mark.parametrize("variant", [18, 14, 13, 12, 19])
@pytest.mark.parametrize("flag", [1, 0])
@pytest.mark.parametrize("case", DMA_CASES + [(50, 35, 64, 300, 3, 3), (17, 90, 128, 257, 1, 3)])
def test_dma_kernel_and_register_kernel_on_the_same_cases(gpu, oracle, case, flag, variant):
    H, W, C, N, kh, kw = case
    if flag == 0 and (H <= 2 * (kh // 2) or W <= 2 * (kw // 2)):
        pytest.skip("no valid region")
    si = workloads.small_ints((H, W, C), 871, -1, 1).astype(np.float16)
    fi = workloads.small_ints((N, kh, kw, C), 872, -1, 1).astype(np.float16)
    got, sbuf, fb = gpu_hconv(si, fi, flag, variant=variant)
    ref, scale = oracle.conv2_f64_f16(sbuf, fb, flag)
    assert scale.max() < 2048
    assert np.array_equal(got.astype(np.float64), ref)
    src = workloads.uniform_01((H, W, C), 873).astype(np.float16)
    filt = workloads.normal((N, kh, kw, C), 874, sigma=0.05).astype(np.float16)
    bias = workloads.normal((N,), 875).astype(np.float16)
    got, sbuf, fb = gpu_hconv(src, filt, flag, bias16=bias, relu=True, variant=variant)
    assert check_against_f64(oracle, got, sbuf, fb, flag, bias16=bias, relu=True) < TOL


@pytest.mark.parametrize("variant", [0, 18, 14, 13, 12])
@pytest.mark.parametrize("case", [(20, 21, 64, 40, 17, 17, 1), (40, 38, 64, 130, 17, 17, 0), (30, 18, 64, 130, 9, 11, 1),
                                  (24, 24, 128, 64, 11, 3, 1), (19, 40, 64, 24, 2, 4, 1), (33, 33, 24, 10, 17, 1, 1)])
def test_large_and_even_filter_extents(gpu, oracle, case, variant):
    # the reference's lowering takes filters of up to 17 x 17 (conv2_mk_im2col.h:278-306); even extents centre on
    # element kh / 2, kw / 2 like the odd ones.  Only four channels of the filters are non-zero, so that sums of {-1, 0, 1}
    # products stay exact in binary16 under 289 taps.
    H, W, C, N, kh, kw, flag = case
    si = workloads.small_ints((H, W, C), 881, -1, 1).astype(np.float16)
    fi = workloads.small_ints((N, kh, kw, C), 882, -1, 1).astype(np.float16)
    fi[:, :, :, 4:] = 0
    got, sbuf, fb = gpu_hconv(si, fi, flag, variant=variant)
    ref, scale = oracle.conv2_f64_f16(sbuf, fb, flag)
    assert scale.max() < 2048
    assert np.array_equal(got.astype(np.float64), ref)
    src = workloads.uniform_01((H, W, C), 883).astype(np.float16)
    filt = workloads.normal((N, kh, kw, C), 884, sigma=0.02).astype(np.float16)
    got, sbuf, fb = gpu_hconv(src, filt, flag, variant=variant)
    assert check_against_f64(oracle, got, sbuf, fb, flag) < TOL


def test_error_codes(gpu):
    L = capi.lib()
    d = capi.DeviceBuffer(1 << 16)
    args = lambda **kw: [kw.get("src", d.ptr), 8, 8, kw.get("dpitch", 8), 64, d.ptr, 4, 3, 3, 3 * 4 * 8, 4 * 8, d.ptr, 8, 64,
                         kw.get("flag", 1), None, 0]
    assert L.decx_hip_conv2_im2col_f16(*args(flag=7)) == 0x0b          # DECX_FAIL_ErrorFlag
    assert L.decx_hip_conv2_im2col_f16(*args(dpitch=4)) == 0x0d    # channel pitch not a multiple of 8
    assert L.decx_hip_conv2_im2col_f16(*args(src=None)) == 0x0d
    assert L.decx_hip_conv2_im2col_f16(*args()) == 0
