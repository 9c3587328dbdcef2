#!/usr/bin/env python3
"""Writes the fixtures of this directory.  Run from the repository root: python tests/golden/make_fixtures.py

reference_known_answer.json
    The one known-answer vector the reference's own tests hold for this path, as data: the operand pattern of
    test/test/CUDA_GEMM/CUDA_GEMM.cpp:24-42 (A[i][j] = float(j*0.1), B[i][j] = float(i*0.1)), the sizes its main() runs
    (:114-115, <2048, 2048, 2048>), and the value the demo prints as what every element "should be": a float running sum of
    the double terms 0.1*i*0.1*i, next to the closed form 0.01*(K-1)K(2K-1)/6.  Nothing of the reference is executed.

chain_vectors.npz
    Small seeded inputs with the outputs of the CPU oracle (oracle/), which tests/test_oracle.py pins against that known
    answer, closed forms and an exact-rational model of the fused chain.  They freeze the pinned arithmetic as data, so
    that the GPU tests can compare bit patterns without the oracle and a later change to the oracle cannot go unnoticed:
      gemm_*   37x53 times 53x29 (+ C), normal(0,1);  conv_*  9x11x6 tensor, 5 filters 3x5x6, both border modes;
      relu_*   special values through forward / record / backward;  half_*  float -> binary16 -> float;
      hconv_*  10x13x8 binary16 tensor, 6 filters 3x3x8 (bit patterns), with the fp64 sums of products and of their
               absolute values in both border modes;  hgemm_*  33x40 times 40x21 binary16 with fp64 products likewise.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from backup_1_amd import workloads  # noqa: E402


def main():
    K = 2048
    printed = np.float32(0.0)
    for i in range(K):
        printed = np.float32(np.float64(printed) + 0.1 * i * 0.1 * i)
    known = {
        "source": "test/test/CUDA_GEMM/CUDA_GEMM.cpp:24-42 (pattern, printed expectation), :114-115 (sizes)",
        "M": 2048, "K": K, "N": 2048,
        "A": "A[i][j] = float(j * 0.1)", "B": "B[i][j] = float(i * 0.1)",
        "printed_expectation_float32": float(printed),
        "closed_form": 0.01 * (K - 1) * K * (2 * K - 1) / 6.0,
    }
    with open(os.path.join(HERE, "reference_known_answer.json"), "w") as f:
        json.dump(known, f, indent=1)
        f.write("\n")

    v = {}
    A, B, C = workloads.normal((37, 53), 9001), workloads.normal((53, 29), 9002), workloads.normal((37, 29), 9003)
    v["gemm_A"], v["gemm_B"], v["gemm_C"] = A, B, C
    v["gemm_AB"] = oracle.sgemm_chain(A, B, fast=False)
    v["gemm_AB_plus_C"] = oracle.sgemm_chain(A, B, C, fast=False)
    src, filt = workloads.normal((9, 11, 6), 9004), workloads.normal((5, 3, 5, 6), 9005)
    v["conv_src"], v["conv_filt"] = src, filt
    v["conv_same"] = oracle.conv2_chain(src, filt, 1)
    v["conv_valid"] = oracle.conv2_chain(src, filt, 0)
    x = workloads.normal((64,), 9006)
    x[:12] = [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, 1e-45, -1e-45, 3.4e38, -3.4e38, 1.17549435e-38, -1.17549435e-38]
    g = workloads.normal((64,), 9007)
    v["relu_x"], v["relu_g"] = x, g
    v["relu_forward"] = oracle.relu(x)
    fwd, rec = oracle.relu_rec(x)
    v["relu_rec_map"] = rec
    v["relu_backward"] = oracle.relu_backward(g, rec)
    h = np.array([0.0, -0.0, 1.0, 0.1, 65504.0, 65520.0, 1e-8, 6.1e-5, 5.96e-8, 2049.0, 2051.0, -3.14159, np.inf], np.float32)
    v["half_in"] = h
    v["half_bits"] = oracle.float_to_half(h)
    v["half_back"] = oracle.half_to_float(v["half_bits"])
    hs = workloads.uniform_01((10, 13, 8), 9008).astype(np.float16)
    hf = workloads.normal((6, 3, 3, 8), 9009, sigma=0.25).astype(np.float16)
    v["hconv_src_bits"], v["hconv_filt_bits"] = hs.view(np.uint16), hf.view(np.uint16)
    v["hconv_same_f64"], v["hconv_same_abs"] = oracle.conv2_f64_f16(v["hconv_src_bits"], v["hconv_filt_bits"], 1)
    v["hconv_valid_f64"], v["hconv_valid_abs"] = oracle.conv2_f64_f16(v["hconv_src_bits"], v["hconv_filt_bits"], 0)
    ha = oracle.float_to_half(workloads.uniform_pm1((33, 40), 9010))
    hb = oracle.float_to_half(workloads.uniform_pm1((40, 21), 9011))
    v["hgemm_A_bits"], v["hgemm_B_bits"] = ha, hb
    v["hgemm_f64"], v["hgemm_abs"] = oracle.gemm_f64_rows_f16(ha, hb, np.arange(33, dtype=np.int32))
    np.savez(os.path.join(HERE, "chain_vectors.npz"), **v)
    print("wrote reference_known_answer.json and chain_vectors.npz (%d arrays)" % len(v))


if __name__ == "__main__":
    main()
