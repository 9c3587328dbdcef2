"""fp32 GEMM parity on the GPU, through the C ABI (decx_hip_sgemm), against the CPU oracle.

The kernel feeds the matrix pipe its k indices in ascending order, and v_mfma_f32_32x32x2_f32 is two steps of a
single-accumulator fused multiply-add chain, so the result is the reference's arithmetic exactly.  Checks:
  * bit-equality with the oracle's fmaf chain on real-valued seeded data (every configuration, every tile shape, with
    and without "+ C"); the stated tolerance of the path, max |x - r| / sum_k|a||b| <= 1e-5 * sqrt(K), is implied;
  * small-integer data against exact integer arithmetic: pins the oracle-independent truth of indexing, ragged edges,
    the K tail and pitches;
  * the split-K entry point, whose K ranges are added in no fixed order, keeps the tolerance form.
"""
import numpy as np
import pytest

from backup_1_amd import workloads
from gpu_helpers import gpu_sgemm, rel_err_vs_abs_scale, pitched

pytestmark = pytest.mark.gpu

TOL = lambda K: 1e-5 * np.sqrt(K)            # stated tolerance of the path
TIGHT = lambda K: 4e-7 * np.sqrt(K) + 2e-7   # working bound: a few ulp of random-walk rounding


def exact_int_product(A, B):
    return (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)


SHAPES = [(1, 1, 1), (3, 5, 7), (31, 17, 33), (32, 16, 32), (128, 16, 128), (129, 17, 130), (256, 256, 256),
          (300, 70, 500), (257, 1500, 255), (64, 8, 1000), (1000, 3, 64), (513, 129, 259)]


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28])
@pytest.mark.parametrize("shape", SHAPES)
def test_integer_exact_all_tiles(gpu, shape, variant):
    M, K, N = shape
    A = workloads.small_ints((M, K), 1000 + M)
    B = workloads.small_ints((K, N), 2000 + N)
    got = gpu_sgemm(A, B, variant=variant)
    assert np.array_equal(got, exact_int_product(A, B))


@pytest.mark.parametrize("shape", [(5, 7, 9), (130, 33, 77), (256, 64, 250)])
def test_unaligned_pitch_uses_elementwise_loader(gpu, shape):
    M, K, N = shape
    A = workloads.small_ints((M, K), 11)
    B = workloads.small_ints((K, N), 12)
    assert np.array_equal(gpu_sgemm(A, B, align=1), exact_int_product(A, B))


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28])
def test_a_times_b_plus_c(gpu, oracle, variant):
    M, K, N = 200, 150, 300
    A, B, C = workloads.small_ints((M, K), 21), workloads.small_ints((K, N), 22), workloads.small_ints((M, N), 23, -100, 100)
    want = exact_int_product(A, B) + C
    assert np.array_equal(gpu_sgemm(A, B, C, variant=variant), want)
    assert np.array_equal(gpu_sgemm(A, B, C, variant=variant, inplace=True), want)       # GEMM.h:206 passes dst as C
    assert np.array_equal(gpu_sgemm(np.zeros_like(A), B, C, variant=variant), C)          # A = 0  =>  dst = C
    Ar, Br, Cr = workloads.normal((M, K), 24), workloads.normal((K, N), 25), workloads.normal((M, N), 26)
    # the chain starts from C (GEMM.cuh:223), so does the kernel: same bits
    assert np.array_equal(gpu_sgemm(Ar, Br, Cr, variant=variant).view(np.uint32), oracle.sgemm_chain(Ar, Br, Cr).view(np.uint32))
    assert np.array_equal(gpu_sgemm(Ar, Br, Cr, variant=variant, inplace=True).view(np.uint32),
                          oracle.sgemm_chain(Ar, Br, Cr).view(np.uint32))


@pytest.mark.parametrize("variant", [11, 12, 13, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28])
def test_block_chain_kernel_walks_every_k_layout(gpu, oracle, variant):
    # sgemm_chain16.hpp: chunks of 64 k through 2, 4 or 8 register sets and 3 LDS buffers, a ragged last chunk apart;
    # sgemm_dma_tile.hpp: steps of 32 or 64 k through 4 or 3 LDS buffers walked in one unrolled pass entered part-way;
    # K around every boundary of those schedules, M and N off the 16 / 32 grid, with and without C and ReLU
    M, N = 45, 83
    for K in (1, 3, 4, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 191, 192, 255, 256, 257, 448, 511, 512, 513, 575, 576, 577, 640, 1023,
              1024, 1025, 1088, 1152, 1153):
        A, B, C = workloads.normal((M, K), 500 + K), workloads.normal((K, N), 600 + K), workloads.normal((M, N), 700 + K)
        assert np.array_equal(gpu_sgemm(A, B, variant=variant).view(np.uint32), oracle.sgemm_chain(A, B).view(np.uint32)), K
        got = gpu_sgemm(A, B, C, variant=variant, relu=True)
        assert np.array_equal(got.view(np.uint32), oracle.relu(oracle.sgemm_chain(A, B, C)).view(np.uint32)), K


def test_long_k_is_the_references_chain_bit_for_bit(gpu, oracle):
    # the shape class of GEMM_Long_Lr (few rows, very long K): automatic choice, and both block-chain shapes
    M, K, N = 24, 40000, 40
    A, B = workloads.normal((M, K), 51), workloads.normal((K, N), 52)
    ref = oracle.sgemm_chain(A, B)
    for variant in (0, 11, 12, 13, 18, 19, 20, 21, 22, 23, 24, 25):
        assert np.array_equal(gpu_sgemm(A, B, variant=variant).view(np.uint32), ref.view(np.uint32)), variant


def test_reference_known_answer_pattern(gpu):
    # test/test/CUDA_GEMM/CUDA_GEMM.cpp:59-109 on GPU_Matrix, main runs <2048,2048,2048>; a 512-row slab keeps it quick
    M, K, N = 512, 2048, 2048
    A, B, printed, closed = workloads.known_answer_pattern(M, K, N)
    got = gpu_sgemm(A, B)
    assert np.all(got == got[0, 0])
    assert abs(float(got[0, 0]) - closed) / closed < TOL(K)
    assert abs(float(got[0, 0]) - printed) / printed < TOL(K)


def test_permutation_matrix_moves_columns_exactly(gpu):
    M, K = 300, 260
    A = workloads.normal((M, K), 31)
    perm = np.random.Generator(np.random.PCG64(32)).permutation(K)
    P = np.zeros((K, K), dtype=np.float32)
    P[perm, np.arange(K)] = 1.0
    assert np.array_equal(gpu_sgemm(A, P).view(np.uint32), A[:, perm].view(np.uint32))


def test_config1_1024_cube_vs_chain(gpu, oracle):
    A, B = workloads.gemm_square(1024)
    ref = oracle.sgemm_chain(A, B)
    for variant in range(0, 29):
        assert np.array_equal(gpu_sgemm(A, B, variant=variant).view(np.uint32), ref.view(np.uint32)), variant


def test_config3_ragged_vs_chain_and_integer_exact(gpu, oracle):
    M, K, N = 3000, 1500, 4500
    Ai, Bi = workloads.small_ints((M, K), 41), workloads.small_ints((K, N), 42)
    assert np.array_equal(gpu_sgemm(Ai, Bi), exact_int_product(Ai, Bi))
    A, B = workloads.gemm_ragged()
    ref = oracle.sgemm_chain(A, B)
    for variant in (0, 7, 2, 11, 12, 13, 14, 15, 18, 19, 20, 21, 22, 24, 25):
        assert np.array_equal(gpu_sgemm(A, B, variant=variant).view(np.uint32), ref.view(np.uint32)), variant


@pytest.mark.parametrize("n", [4096, 8192])
def test_config2_large_squares(gpu, oracle, n):
    # full-size properties that do not need an O(n^3) host product:
    #   integer data:  C @ 1 == A @ (B @ 1)  and  1^T @ C == (1^T @ A) @ B, exactly (all values are small integers)
    #   plus sampled rows against the oracle chain, bit for bit, on integer and on the seeded real-valued data.
    Ai, Bi = workloads.small_ints((n, n), 51, -4, 4), workloads.small_ints((n, n), 52, -4, 4)
    got = gpu_sgemm(Ai, Bi).astype(np.float64)
    A64, B64 = Ai.astype(np.float64), Bi.astype(np.float64)
    assert np.array_equal(got.sum(axis=1), A64 @ B64.sum(axis=1))
    assert np.array_equal(got.sum(axis=0), A64.sum(axis=0) @ B64)
    rows = np.random.Generator(np.random.PCG64(53)).choice(n, size=24, replace=False).astype(np.int32)
    assert np.array_equal(got[rows].astype(np.float32), oracle.sgemm_chain_rows(Ai, Bi, rows))
    del got, A64, B64
    A, B = workloads.gemm_square(n)
    got = gpu_sgemm(A, B)
    assert np.array_equal(got[rows].view(np.uint32), oracle.sgemm_chain_rows(A, B, rows).view(np.uint32))


def test_bad_arguments_are_reported_not_executed(gpu):
    L = gpu.lib()
    buf = gpu.DeviceBuffer(4096)
    assert L.decx_hip_sgemm(buf.ptr, 8, buf.ptr, 8, None, 0, buf.ptr, 8, 0, 8, 8) == 0x03       # empty matrix
    assert L.decx_hip_sgemm(buf.ptr, 4, buf.ptr, 8, None, 0, buf.ptr, 8, 8, 8, 8) == 0x0d       # lda < K
    assert L.decx_hip_sgemm(None, 8, buf.ptr, 8, None, 0, buf.ptr, 8, 8, 8, 8) == 0x0d
    assert gpu.last_error().strip() != ""


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_batched_gemm_one_launch(gpu, variant):
    # decx_hip_sgemm_batched: every problem of the batch against the exact integer product, with and without C
    batch, M, K, N = 5, 130, 70, 200
    A = workloads.small_ints((batch, M, K), 71)
    B = workloads.small_ints((batch, K, N), 72)
    C = workloads.small_ints((batch, M, N), 73, -50, 50)
    pad = lambda x: (x + 7) // 8 * 8
    lda, ldb, ldd = pad(K), pad(N), pad(N)
    Ab = np.full((batch, M, lda), np.nan, np.float32); Ab[:, :, :K] = A
    Bb = np.full((batch, K, ldb), np.nan, np.float32); Bb[:, :, :N] = B
    Cb = np.full((batch, M, ldd), np.nan, np.float32); Cb[:, :, :N] = C
    dA, dB, dC = (gpu.DeviceBuffer.from_numpy(x) for x in (Ab, Bb, Cb))
    dD = gpu.DeviceBuffer.from_numpy(np.full((batch, M, ldd), -5.0, np.float32))
    L = gpu.lib()
    prev = L.decx_hip_set_sgemm_variant(variant)
    try:
        gpu.check(L.decx_hip_sgemm_batched(dA.ptr, lda, M * lda, dB.ptr, ldb, K * ldb, None, 0, 0, dD.ptr, ldd, M * ldd, M, N, K, batch))
        got = dD.download((batch, M, ldd), np.float32)
        want = np.einsum("bik,bkj->bij", A.astype(np.float64), B.astype(np.float64))
        assert np.array_equal(got[:, :, :N], want.astype(np.float32)) and np.all(got[:, :, N:] == -5.0)
        gpu.check(L.decx_hip_sgemm_batched(dA.ptr, lda, M * lda, dB.ptr, ldb, K * ldb, dC.ptr, ldd, M * ldd, dD.ptr, ldd, M * ldd, M, N, K, batch))
        got = dD.download((batch, M, ldd), np.float32)
        assert np.array_equal(got[:, :, :N], (want + C).astype(np.float32))
    finally:
        L.decx_hip_set_sgemm_variant(prev)
    assert L.decx_hip_sgemm_batched(dA.ptr, lda, 10, dB.ptr, ldb, K * ldb, None, 0, 0, dD.ptr, ldd, M * ldd, M, N, K, batch) == 0x0d


def test_gemm3_host_pipeline(gpu):
    # decx_hip_gemm3_host_f32: host arrays in, host arrays out, through the three-stream pipeline
    count, M, K, N = 7, 96, 40, 120
    A = workloads.small_ints((count, M, K), 81)
    B = workloads.small_ints((count, K, N), 82)
    C = workloads.small_ints((count, M, N), 83, -50, 50)
    D = np.zeros((count, M, N), np.float32)
    L = gpu.lib()
    p = lambda a: a.ctypes.data
    gpu.check(L.decx_hip_gemm3_host_f32(p(A), K, M * K, p(B), N, K * N, None, 0, 0, p(D), N, M * N, M, N, K, count))
    want = np.einsum("bik,bkj->bij", A.astype(np.float64), B.astype(np.float64))
    assert np.array_equal(D, want.astype(np.float32))
    gpu.check(L.decx_hip_gemm3_host_f32(p(A), K, M * K, p(B), N, K * N, p(C), N, M * N, p(D), N, M * N, M, N, K, count))
    assert np.array_equal(D, (want + C).astype(np.float32))


@pytest.mark.parametrize("shape", [(96, 40, 120), (2048 + 300, 72, 264), (5000, 33, 100), (2100, 40, 2300), (300, 24, 5000),
                                   (9000, 16, 3100)])
def test_host_resident_gemm_pipeline(gpu, shape):
    # decx_hip_gemm_host_f32: pitched host matrices in, pitched host matrix out; above 512 rows of A / columns of B the
    # operands go up as several panels, and the result is computed and brought back region by region
    M, K, N = shape
    A, B = workloads.small_ints((M, K), 91), workloads.small_ints((K, N), 92)
    C = workloads.small_ints((M, N), 93, -50, 50)
    Ab, lda = pitched(A, 8)
    Bb, ldb = pitched(B, 8)
    Cb, ldc = pitched(C, 8)
    ldd = ldc
    Db = np.full((M, ldd), -5.0, np.float32)
    L = gpu.lib()
    p = lambda a: a.ctypes.data
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)
    gpu.check(L.decx_hip_gemm_host_f32(p(Ab), lda, p(Bb), ldb, None, 0, p(Db), ldd, M, N, K))
    assert np.array_equal(Db[:, :N], want) and np.all(Db[:, N:] == -5.0)
    gpu.check(L.decx_hip_gemm_host_f32(p(Ab), lda, p(Bb), ldb, p(Cb), ldc, p(Db), ldd, M, N, K))
    assert np.array_equal(Db[:, :N], want + C)
    Db[:, :N] = C                                          # C and dst the same host matrix
    gpu.check(L.decx_hip_gemm_host_f32(p(Ab), lda, p(Bb), ldb, p(Db), ldd, p(Db), ldd, M, N, K))
    assert np.array_equal(Db[:, :N], want + C) and np.all(Db[:, N:] == -5.0)
    assert L.decx_hip_gemm_host_f32(p(Ab), K - 1, p(Bb), ldb, None, 0, p(Db), ldd, M, N, K) == 0x0d


def test_host_resident_gemm_pipeline_fp16(gpu, oracle):
    M, K, N = 2048 + 100, 64, 1024 + 144
    A, B = workloads.small_ints((M, K), 94, -3, 3), workloads.small_ints((K, N), 95, -3, 3)
    Ah, Bh = oracle.float_to_half(A), oracle.float_to_half(B)
    D = np.zeros((M, N), np.uint16)
    p = lambda a: a.ctypes.data
    gpu.check(gpu.lib().decx_hip_gemm_host_f16(p(Ah), K, p(Bh), N, None, 0, p(D), N, M, N, K))
    assert np.array_equal(oracle.half_to_float(D), (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))


def test_host_pipelines_keep_their_device_blocks_until_release_tmp(gpu):
    # the device blocks of the host-matrix entry points stay with the library between calls (the reference's device pool,
    # MemoryPool_D.h) and go back to the runtime with decx_hip_release_tmp (de::release_all_tmp, Memory_pool.h:23-37);
    # a call of another size in between takes blocks of its own or a larger idle one, and results stay right throughout
    import ctypes
    import time
    hip = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    L = gpu.lib()
    p = lambda a: a.ctypes.data

    def call(M, K, N):
        A, B = workloads.small_ints((M, K), 96), workloads.small_ints((K, N), 97)
        D = np.zeros((M, N), np.float32)
        gpu.check(L.decx_hip_gemm_host_f32(p(A), K, p(B), N, None, 0, p(D), N, M, N, K))
        assert np.array_equal(D, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
        return free_bytes()

    gpu.check(L.decx_hip_release_tmp())
    big = (4000, 64, 4000)
    first = call(*big)
    assert call(*big) == first                          # the same call again allocates nothing
    assert call(1500, 24, 1200) < first                 # much smaller operands: blocks of their own
    assert call(*big) == call(*big)
    held = free_bytes()
    gpu.check(L.decx_hip_release_tmp())
    kept_at_least = 4 * (4000 * 64 + 64 * 4000 + 4000 * 4000)
    deadline = time.time() + 2.0                        # the runtime reports freed memory with a delay
    while free_bytes() - held < kept_at_least and time.time() < deadline:
        time.sleep(0.05)
    assert free_bytes() - held >= kept_at_least
    gpu.check(L.decx_hip_release_tmp())                 # nothing left to give back: still fine
    # temporaries of the C++ layer's host overloads: the same pool
    blk, blk2 = ctypes.c_void_p(), ctypes.c_void_p()
    gpu.check(L.decx_hip_tmp_malloc(ctypes.byref(blk), 5 << 20))
    gpu.check(L.decx_hip_tmp_free(blk))
    gpu.check(L.decx_hip_tmp_malloc(ctypes.byref(blk2), 4 << 20))
    assert blk2.value == blk.value                      # a block of a similar size is taken again
    gpu.check(L.decx_hip_tmp_free(blk2))
    assert L.decx_hip_tmp_free(blk2) == 0x0d and L.decx_hip_tmp_free(None) == 0
    assert L.decx_hip_tmp_malloc(None, 16) == 0x0d and L.decx_hip_tmp_malloc(ctypes.byref(blk), 0) == 0x0d
    gpu.check(L.decx_hip_release_tmp())
    assert call(*big) <= first + kept_at_least          # and the pipelines work on after a release


def _splitk(gpu, A, B, C=None, splits=0, inplace=False):
    M, K = A.shape
    _, N = B.shape
    pad = lambda x: (x + 7) // 8 * 8
    lda, ldb, ldd = pad(K), pad(N), pad(N)
    Ab = np.full((M, lda), np.nan, np.float32); Ab[:, :K] = A
    Bb = np.full((K, ldb), np.nan, np.float32); Bb[:, :N] = B
    dA, dB = gpu.DeviceBuffer.from_numpy(Ab), gpu.DeviceBuffer.from_numpy(Bb)
    Db = np.full((M, ldd), -9.0, np.float32)
    dC = None
    if C is not None:
        Cb = np.full((M, ldd), np.nan, np.float32); Cb[:, :N] = C
        if inplace:
            Db[:, :N] = C
        else:
            dC = gpu.DeviceBuffer.from_numpy(Cb)
    dD = gpu.DeviceBuffer.from_numpy(Db)
    cptr = dD.ptr if (C is not None and inplace) else (dC.ptr if dC else None)
    gpu.check(gpu.lib().decx_hip_sgemm_splitk(dA.ptr, lda, dB.ptr, ldb, cptr, ldd, dD.ptr, ldd, M, N, K, splits))
    out = dD.download((M, ldd), np.float32)
    assert np.all(out[:, N:] == -9.0), "split-K wrote into the pitch padding"
    return out[:, :N].copy()


@pytest.mark.parametrize("shape", [(16, 65536, 64), (48, 16384, 200), (300, 5000, 130), (1024, 1024, 1024), (7, 100, 5),
                                   (512, 8200, 256)])
def test_splitk_integer_exact_and_tolerance(gpu, oracle, shape):
    # decx_hip_sgemm_splitk (GEMM_Long_Lr): atomics make the order of the K ranges free, integers stay exact
    M, K, N = shape
    A = workloads.small_ints((M, K), 301, -3, 3)
    B = workloads.small_ints((K, N), 302, -3, 3)
    C = workloads.small_ints((M, N), 303, -40, 40)
    want = exact_int_product(A, B)
    for splits in (0, 3, 64):
        assert np.array_equal(_splitk(gpu, A, B, splits=splits), want)
    assert np.array_equal(_splitk(gpu, A, B, C), want + C)
    assert np.array_equal(_splitk(gpu, A, B, C, inplace=True), want + C)
    Ar, Br = workloads.uniform_pm1((M, K), 304), workloads.uniform_pm1((K, N), 305)
    rows = np.arange(0, M, max(1, M // 16), dtype=np.int32)
    ref = oracle.sgemm_chain_rows(Ar, Br, rows)
    _, scale = oracle.gemm_f64_rows_f32(Ar, Br, rows)
    err = rel_err_vs_abs_scale(_splitk(gpu, Ar, Br)[rows], ref, scale)
    assert err < TIGHT(K) < TOL(K)
