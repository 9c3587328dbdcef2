"""The GPU path against the committed fixtures of tests/golden/ alone (no oracle at run time): fp32 GEMM, A*B + C, the
convolution in both border modes and the ReLU family must reproduce the frozen bit patterns; the binary16 GEMM and
convolution (fp32 accumulation) must stay within 2e-3 of the frozen fp64 results."""
import os

import numpy as np
import pytest

from backup_1_amd import capi
from gpu_helpers import gpu_conv, gpu_hconv, gpu_hgemm, gpu_sgemm

pytestmark = pytest.mark.gpu

V = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "chain_vectors.npz"))


def same_bits(a, b):
    nan = np.isnan(b)
    return np.array_equal(np.isnan(a), nan) and np.array_equal(a[~nan].view(np.uint32), b[~nan].view(np.uint32))


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14])
def test_gemm_and_conv_reproduce_the_fixtures(gpu, variant):
    assert same_bits(gpu_sgemm(V["gemm_A"], V["gemm_B"], variant=variant), V["gemm_AB"])
    assert same_bits(gpu_sgemm(V["gemm_A"], V["gemm_B"], C=V["gemm_C"], variant=variant), V["gemm_AB_plus_C"])
    assert same_bits(gpu_conv(V["conv_src"], V["conv_filt"], 1, variant=variant), V["conv_same"])
    assert same_bits(gpu_conv(V["conv_src"], V["conv_filt"], 0, variant=variant), V["conv_valid"])


def test_relu_family_reproduces_the_fixtures(gpu):
    x, g = V["relu_x"], V["relu_g"]
    n = x.size
    L = gpu.lib()
    d_x, d_y, d_g, d_gx = (capi.DeviceBuffer.from_numpy(x), capi.DeviceBuffer(n * 4), capi.DeviceBuffer.from_numpy(g),
                           capi.DeviceBuffer(n * 4))
    d_map = capi.DeviceBuffer(n // 8)
    gpu.check(L.decx_hip_relu_f32(d_x.ptr, d_y.ptr, n))
    assert same_bits(d_y.download((n,), np.float32), V["relu_forward"])
    gpu.check(L.decx_hip_relu_f32_rec(d_x.ptr, d_y.ptr, d_map.ptr, n))
    assert same_bits(d_y.download((n,), np.float32), V["relu_forward"])
    assert np.array_equal(d_map.download((n // 8,), np.uint8), V["relu_rec_map"])
    gpu.check(L.decx_hip_relu_f32_backward(d_g.ptr, d_gx.ptr, d_map.ptr, n))
    assert same_bits(d_gx.download((n,), np.float32), V["relu_backward"])


def _within_fp16_rule(got16, ref, scale):
    # 2e-3 of sum |a||b| for the fp32 accumulation, plus the one rounding of the result to binary16
    return np.all(np.abs(got16.astype(np.float64) - ref) <= 2e-3 * scale + 2.0 ** -11 * np.abs(ref) + 2.0 ** -24)


def test_half_precision_paths_stay_within_tolerance_of_the_fixtures(gpu):
    src, filt = V["hconv_src_bits"].view(np.float16), V["hconv_filt_bits"].view(np.float16)
    for flag, name in ((1, "same"), (0, "valid")):
        got, _, _ = gpu_hconv(src, filt, flag)
        assert _within_fp16_rule(got, V["hconv_%s_f64" % name], V["hconv_%s_abs" % name])
    got = gpu_hgemm(V["hgemm_A_bits"], V["hgemm_B_bits"]).view(np.float16)
    assert _within_fp16_rule(got, V["hgemm_f64"], V["hgemm_abs"])
