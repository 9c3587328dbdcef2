"""Seeded synthetic inputs for the five benchmark configurations of the dense-contraction path.

Generation is numpy PCG64 with explicit transforms, so this container and the GPU box produce identical bytes.
Matrices follow the reference's convention: A is M rows x K, B is K rows x N, row-major
(test/test/CUDA_GEMM/CUDA_GEMM.cpp:20-22 creates them as (width, height) = (K, M), (N, K), (N, M)).
"""
import numpy as np


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def uniform_pm1(shape, seed):
    """i.i.d. uniform[-1, 1) float32."""
    return (_rng(seed).random(shape, dtype=np.float32) * np.float32(2.0) - np.float32(1.0)).astype(np.float32)


def uniform_01(shape, seed):
    return _rng(seed).random(shape, dtype=np.float32)


def normal(shape, seed, sigma=1.0):
    return (_rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(sigma)).astype(np.float32)


def small_ints(shape, seed, lo=-8, hi=8):
    """Integers in [lo, hi] as float32: every partial sum of a product stays exact in fp32 while K*hi*hi < 2^24,
    so any summation order (scalar chain, AVX2, MFMA) must give the same bits."""
    return _rng(seed).integers(lo, hi + 1, size=shape).astype(np.float32)


def gemm_square(n, seed=1234):
    """configs 1, 2, 5: square GEMM operands, uniform[-1,1]."""
    return uniform_pm1((n, n), seed), uniform_pm1((n, n), seed + 1)


def gemm_ragged(seed=4321, M=3000, K=1500, N=4500):
    """config 3: ragged general GEMM, normal(0,1)."""
    return normal((M, K), seed), normal((K, N), seed + 1)


def conv_case(seed=777, H=224, W=224, C=64, N=128, kh=3, kw=3):
    """config 4: input uniform[0,1] HxWxC channel-innermost, N filters kh x kw x C normal(0, 0.05)."""
    return uniform_01((H, W, C), seed), normal((N, kh, kw, C), seed + 1, sigma=0.05)


def known_answer_pattern(M, K, N):
    """The only known-answer input the reference's own tests hold (CUDA_GEMM.cpp:24-42):
    A[i][j] = float(j*0.1), B[i][j] = float(i*0.1) (double product, then stored as float); the demo prints the value
    every element "should be" as a float running sum of the double terms 0.1*i*0.1*i, i.e. approximately
    0.01*(K-1)K(2K-1)/6.  Returns (A, B, printed_value, closed_form)."""
    ramp = (np.arange(K, dtype=np.float64) * 0.1).astype(np.float32)
    A = np.tile(ramp[None, :], (M, 1))
    B = np.tile(ramp[:, None], (1, N))
    printed = np.float32(0.0)
    for i in range(K):
        printed = np.float32(np.float64(printed) + 0.1 * i * 0.1 * i)
    closed = 0.01 * (K - 1) * K * (2 * K - 1) / 6.0
    return np.ascontiguousarray(A), np.ascontiguousarray(B), float(printed), closed
