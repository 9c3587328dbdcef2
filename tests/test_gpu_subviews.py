"""Operands that are column ranges of wider device matrices: pointer moved right by c0 columns, leading dimension = the
parent's pitch.  The host-matrix pipeline of the library passes such views of B itself (one column panel at a time), and
a caller of the C ABI may.  Everything of the parent outside the view is NaN, so a fetch that strays into a neighbouring
panel and reaches a stored result shows; the allocation ends with the parent's last row, which is the case the loaders'
column bound (N rounded up to the fetch width, not the pitch) exists for."""
import numpy as np
import pytest

from backup_1_amd import capi, workloads

pytestmark = pytest.mark.gpu


def parent_with_view(view, c0, parent_cols, nan):
    parent = np.full((view.shape[0], parent_cols), nan, dtype=view.dtype)
    parent[:, c0:c0 + view.shape[1]] = view
    return capi.DeviceBuffer.from_numpy(parent)


# (M, K, N, c0 of B, parent pitch of B): the last shape is a scaled-down copy of the pipeline's case (last panel of a
# 3000-wide B); variants cover the 32x32x2 tiles, the block-chain shapes, the LDS-DMA tiles and the automatic choice
@pytest.mark.parametrize("variant", [0, 2, 7, 9, 11, 12, 13, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28])
@pytest.mark.parametrize("shape", [(96, 64, 40, 24, 64), (130, 72, 100, 8, 108), (256, 128, 952, 2048, 3000)])
def test_fp32_b_is_a_column_range(gpu, oracle, variant, shape):
    M, K, N, c0, pb = shape
    A, B = workloads.normal((M, K), 950), workloads.normal((K, N), 951)
    ca, pa = 16, 16 + K + (-K) % 4 + 8                    # A too is a view: columns [16, 16 + K) of a wider parent
    dA = parent_with_view(A, ca, pa, np.nan)
    dB = parent_with_view(B, c0, pb, np.nan)
    ldd = (N + 7) // 8 * 8
    dD = capi.DeviceBuffer.from_numpy(np.full((M, ldd), -5.0, dtype=np.float32))
    prev = capi.lib().decx_hip_set_sgemm_variant(variant)
    try:
        capi.sgemm(dA.ptr + 4 * ca, pa, dB.ptr + 4 * c0, pb, dD.ptr, ldd, M, N, K)
    finally:
        capi.lib().decx_hip_set_sgemm_variant(prev)
    out = dD.download((M, ldd), np.float32)
    assert np.array_equal(out[:, :N].view(np.uint32), oracle.sgemm_chain(A, B).view(np.uint32))
    assert np.all(out[:, N:] == -5.0)


@pytest.mark.parametrize("variant", [0, 2, 7, 8, 15, 16])
@pytest.mark.parametrize("shape", [(96, 64, 40, 24, 64), (256, 128, 952, 2048, 3000), (256, 256, 1000, 1024, 2024)])
def test_fp16_b_is_a_column_range(gpu, variant, shape):
    M, K, N, c0, pb = shape
    A = workloads.small_ints((M, K), 960, -4, 4).astype(np.float16)
    B = workloads.small_ints((K, N), 961, -4, 4).astype(np.float16)
    nan16 = np.uint16(0x7e00)
    ca, pa = 32, 32 + K + (-K) % 8 + 16
    dA = parent_with_view(A.view(np.uint16), ca, pa, nan16)
    dB = parent_with_view(B.view(np.uint16), c0, pb, nan16)
    ldd = (N + 15) // 16 * 16
    dD = capi.DeviceBuffer.from_numpy(np.full((M, ldd), 0x5555, dtype=np.uint16))
    prev = capi.lib().decx_hip_set_hgemm_variant(variant)
    try:
        capi.hgemm(dA.ptr + 2 * ca, pa, dB.ptr + 2 * c0, pb, dD.ptr, ldd, M, N, K)
    finally:
        capi.lib().decx_hip_set_hgemm_variant(prev)
    out = dD.download((M, ldd), np.uint16)
    want = (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float16).view(np.uint16)
    assert np.array_equal(out[:, :N], want)
    assert np.all(out[:, N:] == 0x5555)
