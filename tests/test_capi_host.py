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
