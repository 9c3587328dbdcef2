"""fp16-in / fp32-accumulate GEMM parity on the GPU (decx_hip_hgemm_f32acc) against an fp64 host product.

Tolerance of the path: |x - r| <= 2e-3 relative, taken as max |x - r| / sum_k|a||b| with r the fp64 product of the
binary16 operands.  Integer data gives a stricter check: the fp32 accumulation is exact, so the result must equal the
exact product rounded once to binary16.
"""
import numpy as np
import pytest

from backup_1_amd import capi, workloads
from gpu_helpers import gpu_hgemm, rel_err_vs_abs_scale

pytestmark = pytest.mark.gpu

TOL = 2e-3


def to_bits(x):
    return x.astype(np.float16).view(np.uint16)


def from_bits(b):
    return b.view(np.float16).astype(np.float64)


SHAPES = [(1, 1, 1), (3, 5, 7), (31, 17, 33), (32, 32, 32), (128, 32, 128), (129, 33, 130), (256, 256, 256),
          (300, 70, 500), (257, 1500, 255), (64, 8, 1000), (1000, 3, 64), (513, 129, 259)]


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 15, 16, 17])
@pytest.mark.parametrize("shape", SHAPES)
def test_integer_exact_all_tiles(gpu, shape, variant):
    M, K, N = shape
    A = workloads.small_ints((M, K), 3000 + M, -4, 4)
    B = workloads.small_ints((K, N), 4000 + N, -4, 4)
    got = gpu_hgemm(to_bits(A), to_bits(B), variant=variant)
    with np.errstate(over="ignore"):
        want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float16).view(np.uint16)   # one RNE rounding
    assert np.array_equal(got, want)


@pytest.mark.parametrize("shape", [(5, 7, 9), (130, 33, 77)])
def test_unaligned_pitch(gpu, shape):
    M, K, N = shape
    A = workloads.small_ints((M, K), 13, -4, 4)
    B = workloads.small_ints((K, N), 14, -4, 4)
    got = gpu_hgemm(to_bits(A), to_bits(B), align=1)
    assert np.array_equal(got, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float16).view(np.uint16))


def test_a_times_b_plus_c(gpu):
    M, K, N = 200, 150, 300
    A, B = workloads.small_ints((M, K), 21, -3, 3), workloads.small_ints((K, N), 22, -3, 3)
    C = workloads.small_ints((M, N), 23, -50, 50)
    want = (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float16).view(np.uint16)
    for variant in (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 15, 16):
        assert np.array_equal(gpu_hgemm(to_bits(A), to_bits(B), to_bits(C), variant=variant), want)


@pytest.mark.parametrize("shape", [(64, 4096, 200), (40, 20000, 130), (130, 2048, 257), (16, 65536, 64)])
def test_split_k_for_few_tiles_and_long_k(gpu, oracle, shape):
    # few 128x128 tiles and K >= 2048: K ranges as separate workgroups, fp32 partial sums in a workspace, one rounding at
    # the end (variant 0 chooses it, 11 forces it).  Integer data: every partial sum is exact, so the result is the exact
    # product rounded once, whatever the order; real data: within the fp16 rule against fp64.
    M, K, N = shape
    A, B = workloads.small_ints((M, K), 31, -1, 1), workloads.small_ints((K, N), 32, -1, 1)
    C = workloads.small_ints((M, N), 33, -20, 20)
    with np.errstate(over="ignore"):
        want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float16).view(np.uint16)
        want_c = (A.astype(np.float64) @ B.astype(np.float64) + C).astype(np.float16).view(np.uint16)
    for variant in (0, 11):
        assert np.array_equal(gpu_hgemm(to_bits(A), to_bits(B), variant=variant), want)
        assert np.array_equal(gpu_hgemm(to_bits(A), to_bits(B), to_bits(C), variant=variant), want_c)
    Ar, Br = to_bits(workloads.uniform_pm1((M, K), 34)), to_bits(workloads.uniform_pm1((K, N), 35))
    rows = np.arange(0, M, 3, dtype=np.int32)
    ref, scale = oracle.gemm_f64_rows_f16(Ar, Br, rows)
    for variant in (0, 11, 2):
        got = from_bits(gpu_hgemm(Ar, Br, variant=variant))[rows]
        assert np.max((np.abs(got - ref) - np.abs(ref) / 2048.0) / scale) < TOL, variant


def test_split_k_is_the_same_on_every_run(gpu, oracle):
    # one workspace plane per K range, added in range order: real-valued data give the same bits on every run, as every
    # path of the reference does (its long-K kernel is one chain, GEMM_long_linear_region.cuh:35-55).  The atomic mode
    # keeps the tolerance only.
    M, K, N = 64, 65536, 1024
    A, B = to_bits(workloads.uniform_pm1((M, K), 36)), to_bits(workloads.uniform_pm1((K, N), 37))
    first = gpu_hgemm(A, B)
    for _ in range(3):
        assert np.array_equal(gpu_hgemm(A, B), first)
    rows = np.arange(0, M, 5, dtype=np.int32)
    ref, scale = oracle.gemm_f64_rows_f16(A, B, rows)
    assert np.max((np.abs(from_bits(first)[rows] - ref) - np.abs(ref) / 2048.0) / scale) < TOL
    prev = capi.lib().decx_hip_set_splitk_mode(1)
    try:
        assert prev == 0
        atomic = from_bits(gpu_hgemm(A, B))[rows]
    finally:
        assert capi.lib().decx_hip_set_splitk_mode(prev) == 1
    assert np.max((np.abs(atomic - ref) - np.abs(ref) / 2048.0) / scale) < TOL
    # a product that is not split must not care about the mode: the same bits under either
    unsplit = gpu_hgemm(A[:, :512], B[:512], variant=8)
    prev = capi.lib().decx_hip_set_splitk_mode(1)
    try:
        assert np.array_equal(gpu_hgemm(A[:, :512], B[:512], variant=8), unsplit)
    finally:
        capi.lib().decx_hip_set_splitk_mode(prev)


@pytest.mark.parametrize("shape", [(4352, 128, 4352), (4352, 384, 4608), (1024, 256, 69632 + 256), (4096, 640, 8192)])
def test_one_workgroup_per_cu_walking_its_tiles(gpu, oracle, shape):
    # variant 17: more whole 256x256 tiles than compute units, one workgroup per CU walks several of them as one stream
    # of K steps (the next tile's first loads are issued during the last steps of the tile before).  Every accumulator
    # sees the same k-blocks in the same order as in the one-tile-per-workgroup build: the same bits, with and without C;
    # integer data exact; real data within the fp16 rule against fp64.
    M, K, N = shape
    info = capi.device_info()
    assert (M // 256) * (N // 256) > info["compute_units"]
    Ai, Bi = workloads.small_ints((M, K), 51, -3, 3), workloads.small_ints((K, N), 52, -3, 3)
    want = (Ai.astype(np.float64) @ Bi.astype(np.float64)).astype(np.float16).view(np.uint16)
    assert np.array_equal(gpu_hgemm(to_bits(Ai), to_bits(Bi), variant=17), want)
    del Ai, Bi, want
    A, B = to_bits(workloads.uniform_pm1((M, K), 53)), to_bits(workloads.uniform_pm1((K, N), 54))
    C = to_bits(workloads.uniform_pm1((M, N), 55))
    one_tile = gpu_hgemm(A, B, variant=15)
    walked = gpu_hgemm(A, B, variant=17)
    assert np.array_equal(walked, one_tile)
    assert np.array_equal(gpu_hgemm(A, B, C, variant=17), gpu_hgemm(A, B, C, variant=15))
    plan = capi.lib().decx_hip_hgemm_plan(M, N, K, 1, (K + 15) // 16 * 16, (N + 15) // 16 * 16, 1, None)
    assert plan == 17 or shape != (4096, 640, 8192)
    if plan == 17:            # where the automatic choice takes the walk by itself
        assert np.array_equal(gpu_hgemm(A, B), one_tile) and np.array_equal(gpu_hgemm(A, B, C), gpu_hgemm(A, B, C, variant=15))
    rows = np.random.Generator(np.random.PCG64(56)).choice(M, size=24, replace=False).astype(np.int32)
    ref, scale = oracle.gemm_f64_rows_f16(A, B, rows)
    assert rel_err_vs_abs_scale(from_bits(walked[rows]), ref, scale) < TOL


def test_rounding_to_half_is_nearest_even(gpu):
    # single products that are exact in fp32 and lie exactly half-way between two binary16 numbers
    A = np.array([[683.0], [293.0], [439.0]], dtype=np.float32)
    B = np.array([[3.0, 7.0, 14.0]], dtype=np.float32)
    got = gpu_hgemm(to_bits(A), to_bits(B)).view(np.float16).astype(np.float32)
    assert got[0, 0] == 2048.0      # 2049: tie between 2048 (even mantissa) and 2050
    assert got[1, 1] == 2052.0      # 2051: tie between 2050 and 2052 (even mantissa)
    assert got[2, 2] == 6144.0      # 6146: tie between 6144 (even mantissa) and 6148


@pytest.mark.parametrize("case", [(1024, 1024, 1024), (777, 1333, 901)])
def test_random_vs_fp64(gpu, oracle, case):
    M, K, N = case
    A, B = workloads.uniform_pm1((M, K), 61), workloads.uniform_pm1((K, N), 62)
    Ab, Bb = oracle.float_to_half(A), oracle.float_to_half(B)
    rows = np.arange(0, M, max(1, M // 50), dtype=np.int32)
    ref, scale = oracle.gemm_f64_rows_f16(Ab, Bb, rows)
    for variant in (1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 15, 16):
        got = from_bits(gpu_hgemm(Ab, Bb, variant=variant))[rows]
        err = rel_err_vs_abs_scale(got, ref, scale)
        print("%s variant %d: max |x-r|/sum|a||b| = %.3e (bound %.1e)" % (case, variant, err, TOL))
        assert err < TOL
        # elementwise: within half a binary16 ulp of the fp64 value plus the fp32 accumulation error
        assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -11 + scale * 1e-6 + 1e-7)


def test_config5_8192_cube_sampled_rows(gpu, oracle):
    n = 8192
    A, B = workloads.gemm_square(n, seed=5)
    Ab, Bb = oracle.float_to_half(A), oracle.float_to_half(B)
    del A, B
    got = gpu_hgemm(Ab, Bb)
    rows = np.random.Generator(np.random.PCG64(63)).choice(n, size=64, replace=False).astype(np.int32)
    ref, scale = oracle.gemm_f64_rows_f16(Ab, Bb, rows)
    g = from_bits(got[rows])
    err = rel_err_vs_abs_scale(g, ref, scale)
    print("8192^3 fp16: max |x-r|/sum|a||b| on 64 rows = %.3e (bound %.1e); max |x-r|/max|r| = %.3e" %
          (err, TOL, np.max(np.abs(g - ref)) / np.max(np.abs(ref))))
    assert err < TOL
    assert np.all(np.abs(g - ref) <= np.abs(ref) * 2.0 ** -11 + scale * 1e-6 + 1e-7)
    # full-size integer property: C @ 1 == A @ (B @ 1) exactly while every C element is exact in binary16 (|c| <= 2048)
    Ai = workloads.small_ints((n, n), 64, -1, 1) * (workloads.uniform_01((n, n), 65) < 0.02)
    Bi = workloads.small_ints((n, n), 66, -1, 1)
    goti = from_bits(gpu_hgemm(to_bits(Ai), to_bits(Bi)))
    assert np.max(np.abs(goti)) <= 2048
    assert np.array_equal(goti.sum(axis=1), Ai.astype(np.float64) @ Bi.astype(np.float64).sum(axis=1))
    assert np.array_equal(goti.sum(axis=0), Ai.astype(np.float64).sum(axis=0) @ Bi.astype(np.float64))


@pytest.mark.parametrize("variant", [0, 2, 4, 7, 15, 16])
def test_batched_hgemm_one_launch(gpu, variant):
    batch, M, K, N = 3, 256, 128, 512
    A = workloads.small_ints((batch, M, K), 91, -3, 3)
    B = workloads.small_ints((batch, K, N), 92, -3, 3)
    dA, dB = gpu.DeviceBuffer.from_numpy(to_bits(A)), gpu.DeviceBuffer.from_numpy(to_bits(B))
    dD = gpu.DeviceBuffer(batch * M * N * 2)
    L = gpu.lib()
    prev = L.decx_hip_set_hgemm_variant(variant)
    try:
        gpu.check(L.decx_hip_hgemm_f32acc_batched(dA.ptr, K, M * K, dB.ptr, N, K * N, None, 0, 0, dD.ptr, N, M * N, M, N, K, batch))
    finally:
        L.decx_hip_set_hgemm_variant(prev)
    got = dD.download((batch, M, N), np.uint16)
    want = np.einsum("bik,bkj->bij", A.astype(np.float64), B.astype(np.float64)).astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)
