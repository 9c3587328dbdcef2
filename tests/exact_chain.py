"""Exact-arithmetic model of the reference's accumulation, independent of the C++ oracle.

acc_{k+1} = round_to_binary32(a_k * b_k + acc_k) with the product and the sum formed exactly (python Fractions)
and a single round-to-nearest-even at the end: that is what fmaf / _mm256_fmadd_ps do
(reference: srcs/GEMM/CUDA/GEMM_kernel_def.cuh:33-55, srcs/GEMM/CPU/sgemm_calc_kernel.h:24-29).
Normal-range values only (no subnormal / overflow handling), which is all the tests feed it.
"""
from fractions import Fraction

import numpy as np


def round_f32(x):
    """Correctly rounded (nearest-even) binary32 value of the Fraction x, returned as a Fraction."""
    if x == 0:
        return Fraction(0)
    s = -1 if x < 0 else 1
    x = abs(x)
    e = 0
    # find e with 2^23 <= x / 2^e < 2^24
    while x / Fraction(2) ** e >= 2 ** 24:
        e += 1
    while x / Fraction(2) ** e < 2 ** 23:
        e -= 1
    assert e >= -149 + 0 and e <= 104, "outside the normal binary32 range"
    q = round(x / Fraction(2) ** e)       # python rounds Fractions half-to-even
    return s * q * Fraction(2) ** e


def fma_chain(a_vals, b_vals, acc0=0.0):
    acc = Fraction(float(acc0))
    for a, b in zip(a_vals, b_vals):
        acc = round_f32(Fraction(float(a)) * Fraction(float(b)) + acc)
    return np.float32(float(acc))


def gemm_exact_chain(A, B, C=None):
    M, K = A.shape
    _, N = B.shape
    D = np.empty((M, N), dtype=np.float32)
    for i in range(M):
        for j in range(N):
            D[i, j] = fma_chain(A[i, :], B[:, j], 0.0 if C is None else C[i, j])
    return D
