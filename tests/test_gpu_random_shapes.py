"""Seeded sweep over random small problems: every combination of ragged M / N / K (including K shorter than one, two or
three K steps, which take the peeled paths of the pipelined loop), pitch padding, tile shape, "+ C" and the ReLU epilogue
must reproduce the oracle's fused chain bit for bit; random convolutions likewise."""
import numpy as np
import pytest

from backup_1_amd import workloads
from gpu_helpers import gpu_conv, gpu_hconv, gpu_hgemm, gpu_sgemm

pytestmark = pytest.mark.gpu


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.mark.parametrize("seed", range(12))
def test_random_gemms_bit_exact(gpu, oracle, seed):
    rng = np.random.Generator(np.random.PCG64(7000 + seed))
    for case in range(10):
        M, N = int(rng.integers(1, 420)), int(rng.integers(1, 420))
        K = int(rng.choice([int(rng.integers(1, 70)), int(rng.integers(1, 700))]))
        variant = int(rng.integers(0, 29))
        align = int(rng.choice([8, 8, 4, 1]))          # DECX pitch, a 16-byte pitch, an unaligned pitch
        with_c, relu = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        A, B = workloads.normal((M, K), 100 * seed + case), workloads.normal((K, N), 100 * seed + case + 50)
        C = workloads.normal((M, N), 100 * seed + case + 77) if with_c else None
        ref = oracle.sgemm_chain(A, B, C)
        if relu:
            ref = oracle.relu(ref)
        got = gpu_sgemm(A, B, C=C, align=align, variant=variant, relu=relu)
        assert np.array_equal(bits(got), bits(ref)), (M, K, N, variant, align, with_c, relu)


@pytest.mark.parametrize("seed", range(8))
def test_random_convolutions_bit_exact(gpu, oracle, seed):
    rng = np.random.Generator(np.random.PCG64(8000 + seed))
    for case in range(6):
        kh, kw = int(rng.choice([1, 3, 5, 7])), int(rng.choice([1, 3, 5, 7]))
        H, W = int(rng.integers(kh, 40)), int(rng.integers(kw, 40))
        C, N = int(rng.integers(1, 40)), int(rng.integers(1, 150))
        if rng.integers(0, 3) == 0:
            C, N = int(rng.choice([32, 64, 96])), 4 * int(rng.integers(1, 40))      # what the LDS-DMA kernels (29, 30, 31) take
        flag, variant = int(rng.integers(0, 2)), int(rng.choice(list(range(14)) + [15, 16, 17, 23, 29, 30, 31]))
        src = workloads.normal((H, W, C), 300 * seed + case)
        filt = workloads.normal((N, kh, kw, C), 300 * seed + case + 150)
        ref = oracle.conv2_chain(src, filt, flag)
        assert np.array_equal(bits(gpu_conv(src, filt, flag, variant=variant)), bits(ref)), (H, W, C, N, kh, kw, flag, variant)


@pytest.mark.parametrize("seed", range(8))
def test_random_fp16_convolutions_exact_on_small_integers(gpu, oracle, seed):
    # every fp16 convolution kernel (12: register-staged, 13: LDS-DMA, 14: tap rows in LDS, 18: 16x16x32 blocks on patches, 0: the library's choice,
    # which includes the split over K) on random shapes; channel counts that make the channel pitch a multiple of 64 halves
    # half of the time, since only those reach kernels 13 and 14.  Values in {-1, 0, 1}: sums stay exact in binary16.
    rng = np.random.Generator(np.random.PCG64(9000 + seed))
    for case in range(6):
        kh, kw = int(rng.choice([1, 3, 5, 7])), int(rng.choice([1, 3, 3, 5, 7]))
        H, W = int(rng.integers(kh, 70)), int(rng.integers(kw, 70))
        C = int(rng.choice([64, 128, 57])) if rng.integers(0, 2) else int(rng.integers(1, 70))
        N = int(rng.integers(1, 200))
        flag, variant = int(rng.integers(0, 2)), int(rng.choice([0, 12, 13, 14, 18]))
        if flag == 0 and (H <= 2 * (kh // 2) or W <= 2 * (kw // 2)):
            flag = 1
        src = workloads.small_ints((H, W, C), 500 * seed + case, -1, 1).astype(np.float16)
        filt = workloads.small_ints((N, kh, kw, C), 500 * seed + case + 250, -1, 1).astype(np.float16)
        if kh * kw * C >= 2048:
            filt[:, :, :, 16:] = 0                       # keep every sum below 2048
        relu = bool(rng.integers(0, 2))
        got, sbuf, fb = gpu_hconv(src, filt, flag, relu=relu, variant=variant)
        ref, scale = oracle.conv2_f64_f16(sbuf, fb, flag)
        assert scale.max() < 2048
        want = np.maximum(ref, 0.0) if relu else ref
        assert np.array_equal(got.astype(np.float64), want), (H, W, C, N, kh, kw, flag, variant, relu)


@pytest.mark.parametrize("seed", range(10))
def test_random_fp16_gemms_exact_on_small_integers(gpu, seed):
    # every fp16 GEMM kernel (register-staged 1, 2; LDS-DMA tiles on 32x32x16 blocks 3 - 10; on 16x16x32 blocks 15, 16, and 17,
    # the walk over several tiles per workgroup, which falls back to 15 on ragged products; 11: split over K; 0: the
    # library's choice) on ragged M / N / K, with K shorter than one, two or three K steps among them, DECX pitches,
    # 16-byte pitches and unaligned ones, with and without "+ C".  Values in {-2 .. 2} and K <= 500: every sum is an
    # integer below 2048 in magnitude, exact in binary16, so the bits must equal the fp64 product's.
    rng = np.random.Generator(np.random.PCG64(9500 + seed))
    for case in range(10):
        M, N = int(rng.integers(1, 600)), int(rng.integers(1, 600))
        K = int(rng.choice([int(rng.integers(1, 100)), int(rng.integers(1, 500))]))
        variant = int(rng.choice([0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 15, 16, 17]))
        align = int(rng.choice([16, 16, 8, 1]))
        with_c = bool(rng.integers(0, 2))
        A = workloads.small_ints((M, K), 700 * seed + case, -2, 2)
        B = workloads.small_ints((K, N), 700 * seed + case + 350, -2, 2)
        C = workloads.small_ints((M, N), 700 * seed + case + 500, -40, 40) if with_c else None
        want = A.astype(np.float64) @ B.astype(np.float64) + (C if with_c else 0.0)
        assert np.abs(want).max() <= 2048
        h = lambda x: x.astype(np.float16).view(np.uint16)
        got = gpu_hgemm(h(A), h(B), h(C) if with_c else None, align=align, variant=variant)
        assert np.array_equal(got.view(np.float16).astype(np.float64), want), (M, K, N, variant, align, with_c)


@pytest.mark.parametrize("shape", [(3_000_000, 8, 8), (8, 8, 3_000_000), (16, 1_000_000, 16), (1, 1, 70_000), (70_000, 1, 1),
                                   (1, 500_000, 1), (100_000, 40, 1), (1, 40, 100_000), (65_537, 3, 129), (250, 70_000, 6),
                                   # tall results at most 256 wide, each on the tile the picker has for that width and K
                                   (70_001, 600, 96), (60_003, 100, 100), (60_000, 130, 64), (45_000, 1030, 128), (33_333, 520, 200),
                                   (52_000, 515, 250), (41_000, 300, 33), (120_000, 520, 24), (90_000, 70, 50)])
def test_extreme_aspect_ratios_exact_on_small_integers(gpu, shape):
    # millions of rows or columns under a few k, one row under a million k: tile counts, grids and chain lengths far from
    # the squares.  Values in {-1, 0, 1} with at most a third of them non-zero in A keep every sum exact in both precisions.
    M, K, N = shape
    A = workloads.small_ints((M, K), 41, -1, 1)
    B = workloads.small_ints((K, N), 42, -1, 1)
    if K > 2000:
        A[:, 2000:] = 0                                 # |sum| <= 2000: exact in binary16 as well
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.array_equal(gpu_sgemm(A, B).astype(np.float64), want), shape
    h = lambda x: x.astype(np.float16).view(np.uint16)
    assert np.array_equal(gpu_hgemm(h(A), h(B)).view(np.float16).astype(np.float64), want), shape
