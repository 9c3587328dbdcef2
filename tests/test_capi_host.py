"""CPU-only checks of the C-ABI library: it loads, exports every declared symbol, and refuses work before init."""
import ctypes
import os
import re

import pytest

from backup_1_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "decx_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(decx_hip_[a-z0-9_]+)\s*\(", header)))
    assert declared == sorted(capi.SYMBOLS)
    L = ctypes.CDLL(capi.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), name


def test_compute_entry_points_refuse_before_init():
    import torch  # noqa: F401  (only to learn whether this box has a GPU; the library itself never uses torch)
    L = capi.lib()
    if L.decx_hip_is_init():
        pytest.skip("library already initialised in this process")
    # the decx::cuP.is_init gate (GEMM.h:63): error 0x01 and the reference's message
    assert L.decx_hip_sgemm(None, 8, None, 8, None, 0, None, 8, 8, 8, 8) == 0x01
    assert "initialized first" in capi.last_error()
    assert L.decx_hip_hgemm_f32acc(None, 16, None, 16, None, 0, None, 16, 8, 8, 8) == 0x01
    assert L.decx_hip_conv2_im2col_f32(None, 4, 4, 4, 16, None, 1, 3, 3, 48, 16, None, 4, 16, 1) == 0x01
    p = ctypes.c_void_p()
    assert L.decx_hip_malloc(ctypes.byref(p), 16) == 0x01
    assert L.decx_hip_timer_start() == 0x01


def test_init_without_device_fails_cleanly():
    import torch
    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present")
    dev = ctypes.c_int(-1)
    rc = capi.lib().decx_hip_init(ctypes.byref(dev))
    assert rc != 0 and not capi.lib().decx_hip_is_init()
    assert capi.last_error().strip() != ""


def test_every_hip_source_is_in_the_makefile():
    # the library is one translation unit per kernel family: a source missing from SRCS would silently drop its entry points
    csrc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "backup_1_amd", "csrc")
    mk = open(os.path.join(csrc, "Makefile")).read().replace("\\\n", " ")
    srcs = next(l for l in mk.splitlines() if l.startswith("SRCS")).split(":=")[1].split()
    assert sorted(srcs) == sorted(f for f in os.listdir(csrc) if f.endswith(".hip"))


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


# widths of the tiles the GEMM kernels are built with (sgemm_launch.hpp, sgemm_chain16.hpp, hgemm.hip) and the width
# of their vector fetches: 4 floats, 8 halves
B_TILE_WIDTHS = {4: (16, 32, 64, 128, 192, 256), 8: (64, 128, 256)}


@pytest.mark.parametrize("unit", (4, 8))
def test_b_loaders_stay_inside_a_column_range_of_a_wider_matrix(unit):
    """B may be columns [c0, c0 + N) of a parent matrix (pointer moved right, parent pitch): the last row of that view
    ends with the parent's allocation, so no fetch may go beyond column roundup(N, unit) - 1 of the view, whatever the
    tile width.  A bound taken from the pitch instead (fetch up to ldb - unit) would leave the parent's last row by up
    to c0 columns."""
    L = capi.lib()
    for tile_n in B_TILE_WIDTHS[unit]:
        for N in list(range(1, 3 * tile_n + 2)) + [952, 3000, 4500, 8191, 8192]:
            extent = L.decx_hip_b_read_extent(N, tile_n, unit)
            assert extent == (N + unit - 1) // unit * unit - 1, (N, tile_n, unit, extent)
    # the case that showed the defect: K = 1024 rows of a parent with pitch 3000 = exactly 3000 pages of 4 KiB, last
    # column panel c0 = 2048 with 952 columns, 64-wide tiles: the fetch must end inside the parent's last row
    K, ldb_parent, c0, cols = 1024, 3000, 2048, 952
    extent = L.decx_hip_b_read_extent(cols, 64, 4)
    last_element = (K - 1) * ldb_parent + c0 + extent
    assert last_element < K * ldb_parent
    assert L.decx_hip_b_read_extent(0, 64, 4) == -1 and L.decx_hip_b_read_extent(8, 60, 8) == -1
