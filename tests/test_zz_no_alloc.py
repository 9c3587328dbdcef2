"""decx_hip_hgemm_f32acc_noalloc: the fp16 GEMM's K-range route on the workspace that is built into the library, for
callers that cannot allocate device memory.  Checked through the C ABI against decx_hip_hgemm_f32acc on the same inputs:
bit-equal (both add the ranges' planes in range order, and take the same number of ranges), and within the fp16 rule
against fp64.  Two calls in a row share the one workspace, the second with a smaller input: nothing of the first call may
leak into it."""
import numpy as np
import pytest

from backup_1_amd import capi, workloads
from gpu_helpers import gpu_hgemm, pitched

pytestmark = pytest.mark.gpu

TOL = 2e-3


def noalloc_hgemm(Abits, Bbits, Cbits=None, splits=0):
    M, K = Abits.shape
    _, N = Bbits.shape
    Ab, lda = pitched(Abits, 16)
    Bb, ldb = pitched(Bbits, 16)
    ldd = (N + 15) // 16 * 16
    dA, dB = capi.DeviceBuffer.from_numpy(Ab), capi.DeviceBuffer.from_numpy(Bb)
    dD = capi.DeviceBuffer.from_numpy(np.full((M, ldd), 0x5555, dtype=np.uint16))
    dC, ldc = None, 0
    if Cbits is not None:
        Cb, ldc = pitched(Cbits, 16)
        dC = capi.DeviceBuffer.from_numpy(Cb)
    capi.check(capi.lib().decx_hip_hgemm_f32acc_noalloc(dA.ptr, lda, dB.ptr, ldb, dC.ptr if dC else None, ldc, dD.ptr, ldd,
                                                        M, N, K, splits))
    out = dD.download((M, ldd), np.uint16)
    assert np.all(out[:, N:] == 0x5555), "kernel wrote into the pitch padding of dst"
    return out[:, :N].copy()


def bits(x):
    return x.astype(np.float16).view(np.uint16)


def free_device_bytes():
    """hipMemGetInfo, read straight from the HIP runtime the library is linked against."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def test_the_entry_point_allocates_no_device_memory(gpu):
    # operands and result are the caller's; between their allocation and their release the free device memory must not
    # move, whatever the number of K ranges, on the first call of the process on this entry point as on later ones
    shapes = [(200, 16384, 520, 0), (40, 4096, 136, 0), (256, 8192, 512, 16), (64, 65536, 1024, 0)]
    bufs = []
    for M, K, N, _ in shapes:
        A, B = bits(workloads.uniform_pm1((M, K), 7)), bits(workloads.uniform_pm1((K, N), 8))
        bufs.append((capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(B), capi.DeviceBuffer(M * N * 2)))
    capi.sync()
    before = free_device_bytes()
    for (M, K, N, splits), (dA, dB, dD) in zip(shapes, bufs):
        capi.check(capi.lib().decx_hip_hgemm_f32acc_noalloc(dA.ptr, K, dB.ptr, N, None, 0, dD.ptr, N, M, N, K, splits))
        assert free_device_bytes() == before, (M, K, N, splits)


def test_two_calls_in_a_row_match_the_allocating_entry_point(gpu, oracle):
    # first a product that takes many K ranges and most of a plane, then a smaller one with fewer ranges
    for (M, K, N), seed in (((200, 16384, 520), 70), ((40, 4096, 130), 80)):
        A, B = bits(workloads.uniform_pm1((M, K), seed)), bits(workloads.uniform_pm1((K, N), seed + 1))
        C = bits(workloads.uniform_pm1((M, N), seed + 2))
        want = gpu_hgemm(A, B)                       # decx_hip_hgemm_f32acc: splits K by itself on these shapes
        got = noalloc_hgemm(A, B)
        assert np.array_equal(got, want), (M, K, N)
        assert np.array_equal(noalloc_hgemm(A, B, C), gpu_hgemm(A, B, C)), (M, K, N)
        rows = np.arange(0, M, 3, dtype=np.int32)
        ref, scale = oracle.gemm_f64_rows_f16(A, B, rows)
        g = got.view(np.float16).astype(np.float64)[rows]
        assert np.max((np.abs(g - ref) - np.abs(ref) / 2048.0) / scale) < TOL
    # integer-valued data: exact whatever the number of ranges, also when it is given
    Ai = workloads.small_ints((70, 3000), 90, -1, 1)
    Bi = workloads.small_ints((3000, 90), 91, -1, 1)
    want = (Ai.astype(np.float64) @ Bi.astype(np.float64)).astype(np.float16).view(np.uint16)
    for splits in (0, 1, 5, 47):
        assert np.array_equal(noalloc_hgemm(bits(Ai), bits(Bi), splits=splits), want), splits


def test_refuses_what_does_not_fit_the_workspace(gpu):
    L = capi.lib()
    d = capi.DeviceBuffer(1 << 20)
    limit = 32 << 20
    # 4096 x 4096 floats = 64 MiB for a single range
    rc = L.decx_hip_hgemm_f32acc_noalloc(d.ptr, 4096, d.ptr, 4096, None, 0, d.ptr, 4096, 4096, 4096, 4096, 1)
    assert rc == 0x0d and "static workspace" in capi.last_error() and str(limit) in capi.last_error()
    # fits with 2 ranges, not with 3: 2048 x 1536 x 4 B = 12 MiB per range
    rc = L.decx_hip_hgemm_f32acc_noalloc(d.ptr, 8192, d.ptr, 1536, None, 0, d.ptr, 1536, 2048, 1536, 8192, 3)
    assert rc == 0x0d and "static workspace" in capi.last_error()
    # unaligned operands are refused too (the K-range kernel needs the vector loads)
    rc = L.decx_hip_hgemm_f32acc_noalloc(d.ptr + 2, 64, d.ptr, 64, None, 0, d.ptr, 64, 32, 32, 32, 0)
    assert rc == 0x0d
    rc = L.decx_hip_hgemm_f32acc_noalloc(None, 64, d.ptr, 64, None, 0, d.ptr, 64, 32, 32, 32, 0)
    assert rc == 0x0d
