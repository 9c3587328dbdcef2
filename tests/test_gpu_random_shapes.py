"""Seeded sweep over random small problems: every combination of ragged M / N / K (including K shorter than one, two or
three K steps, which take the peeled paths of the pipelined loop), pitch padding, tile shape, "+ C" and the ReLU epilogue
must reproduce the oracle's fused chain bit for bit; random convolutions likewise."""
import numpy as np
import pytest

from backup_1_amd import workloads
from gpu_helpers import gpu_conv, gpu_hconv, gpu_sgemm

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
            C, N = int(rng.choice([32, 64, 96])), 4 * int(rng.integers(1, 40))      # what the LDS-DMA kernel (29, 30) takes
        flag, variant = int(rng.integers(0, 2)), int(rng.choice(list(range(14)) + [15, 16, 17, 23, 29, 30]))
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
