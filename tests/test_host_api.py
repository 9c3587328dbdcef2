"""Runs the C++ API test program (tests/host/test_decx_api.cpp, built by backup_1_amd/host/Makefile): the DECX-named
classes and functions over the C ABI, exercised the way the reference's demos do, with assertions."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "build", "test_decx_api")


def _run(mode, timeout):
    assert os.path.exists(BIN), "build it with `make -C backup_1_amd/host` (or __graft_entry__.build())"
    r = subprocess.run([BIN, mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)
    print(r.stdout)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "0 failure(s)" in r.stdout


def test_cpp_api_cpu_side():
    _run("cpu", 300)


@pytest.mark.gpu
def test_cpp_api_gpu_side():
    _run("gpu", 300)
