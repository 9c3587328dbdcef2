"""Leading dimensions so wide that a matrix spans more than 4 GiB: row offsets leave 32 bits.  The containers of the
reference cannot make such a pitch (pitch = width rounded up, Matrix.h:253-267), a caller that hands sub-matrices of a
large buffer to the C ABI can.  Only the rows used are written and read, so the tests stay cheap."""
import numpy as np
import pytest

from backup_1_amd import capi, workloads

pytestmark = pytest.mark.gpu


def put(arr, pitch):
    rows, cols = arr.shape
    item = arr.dtype.itemsize
    buf = capi.DeviceBuffer(rows * pitch * item)
    host = np.ascontiguousarray(arr)
    capi.check(capi.lib().decx_hip_memcpy2d(buf.ptr, pitch * item, host.ctypes.data, cols * item, cols * item, rows, capi.H2D))
    return buf


def get(buf, rows, cols, pitch, dtype):
    out = np.empty((rows, cols), dtype=dtype)
    item = out.dtype.itemsize
    capi.check(capi.lib().decx_hip_memcpy2d(out.ctypes.data, cols * item, buf.ptr, pitch * item, cols * item, rows, capi.D2H))
    return out


@pytest.mark.parametrize("variant", [0, 2, 7, 11, 13])
def test_fp32_rows_past_four_gib(gpu, oracle, variant):
    M, K, N, pitch = 300, 200, 260, 1 << 23          # row 128 of every operand starts 4 GiB into its buffer
    A = workloads.normal((M, K), 901)
    B = workloads.normal((K, N), 902)
    C = workloads.normal((M, N), 903)
    dA, dB, dC = put(A, pitch), put(B, pitch), put(C, pitch)
    dD = capi.DeviceBuffer(M * pitch * 4)
    prev = capi.lib().decx_hip_set_sgemm_variant(variant)
    try:
        capi.sgemm(dA.ptr, pitch, dB.ptr, pitch, dD.ptr, pitch, M, N, K, dC.ptr, pitch)
    finally:
        capi.lib().decx_hip_set_sgemm_variant(prev)
    assert np.array_equal(get(dD, M, N, pitch, np.float32).view(np.uint32), oracle.sgemm_chain(A, B, C).view(np.uint32))


# 6M halves: a 256-row tile of A spans 3 GiB, offsets use the upper half of 32 bits; 16M halves: the tile spans 8 GiB,
# which the 32-bit offsets of the LDS-DMA tile cannot hold -- the library must take another kernel by itself
@pytest.mark.parametrize("variant", [0, 7])
@pytest.mark.parametrize("pitch", [6 * 1024 * 1024, 1 << 24])
def test_fp16_wide_pitch(gpu, pitch, variant):
    M, K, N = 300, 200, 260
    A = workloads.small_ints((M, K), 911, -4, 4)
    B = workloads.small_ints((K, N), 912, -4, 4)
    dA = put(A.astype(np.float16).view(np.uint16), pitch)
    dB = put(B.astype(np.float16).view(np.uint16), pitch)
    dD = capi.DeviceBuffer(M * pitch * 2)
    prev = capi.lib().decx_hip_set_hgemm_variant(variant)
    try:
        capi.hgemm(dA.ptr, pitch, dB.ptr, pitch, dD.ptr, pitch, M, N, K)
    finally:
        capi.lib().decx_hip_set_hgemm_variant(prev)
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float16).view(np.uint16)
    assert np.array_equal(get(dD, M, N, pitch, np.uint16), want)


@pytest.mark.parametrize("variant", [26, 27, 28, 20, 18, 0])
def test_fp32_lds_dma_tiles_at_their_widest_pitch(gpu, oracle, variant):
    # pitches of 2^21 - 4 floats, the widest the LDS-DMA tiles take: row 255 of a 256-row tile of A starts 2^31 - 4080 bytes
    # after the tile's first row, the last 32-bit byte offset these kernels form.  (One float wider and the library takes
    # another kernel: tests/test_kernel_choice.py.)  Two tile rows, so that the second tile's base lies beyond 2 GiB.
    M, K, N, pitch = 300, 72, 260, (1 << 21) - 4
    A = workloads.normal((M, K), 921)
    B = workloads.normal((K, N), 922)
    dA, dB = put(A, pitch), put(B, pitch)
    dD = capi.DeviceBuffer(M * 264 * 4)
    prev = capi.lib().decx_hip_set_sgemm_variant(variant)
    try:
        if variant:
            assert capi.lib().decx_hip_sgemm_plan(M, N, K, 1, pitch, pitch, 1) == variant      # the tile under test does run
        capi.sgemm(dA.ptr, pitch, dB.ptr, pitch, dD.ptr, 264, M, N, K)
    finally:
        capi.lib().decx_hip_set_sgemm_variant(prev)
    assert np.array_equal(get(dD, M, N, 264, np.float32).view(np.uint32), oracle.sgemm_chain(A, B).view(np.uint32))
