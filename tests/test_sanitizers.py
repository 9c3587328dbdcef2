"""The host-side C++ (the DECX-named API layer, de::cpu::sgemm with its atomic-counter workers, and the oracle with its
packaged-task thread pool) compiled under ThreadSanitizer and AddressSanitizer and run over the CPU checks of
tests/host/test_decx_api.cpp.  CPU only: the program never initialises a device.  The reference's counterparts of these
pieces are where its host-side races live (core/thread_management/thread_pool.h:73-100: workers and the submitting
thread share the queue without a common lock; core/memory_management/MemoryPool_D.h:24: unsynchronised global pool)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
pytestmark = pytest.mark.sanitizer


@pytest.mark.parametrize("san", ["thread", "address"])
def test_host_code_is_clean_under(san):
    host = os.path.join(ROOT, "backup_1_amd", "host")
    if not os.path.exists(os.path.join(ROOT, "backup_1_amd", "libdecx_hip.so")):
        pytest.fail("libdecx_hip.so is missing: build it with `make -C backup_1_amd/csrc`")
    r = subprocess.run(["make", "-C", host, "san", "SAN=" + san], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    exe = os.path.join(ROOT, "tests", "build", "test_decx_api_" + san)
    env = dict(os.environ)
    # leaks: the API hands out heap objects that the reference's conventions never delete (factories return references)
    env["ASAN_OPTIONS"] = "detect_leaks=0:abort_on_error=0"
    env["TSAN_OPTIONS"] = "halt_on_error=0:exitcode=66"
    r = subprocess.run([exe, "cpu-small"], capture_output=True, text=True, env=env, timeout=600)
    report = r.stdout[-4000:] + r.stderr[-6000:]
    assert "WARNING: ThreadSanitizer" not in r.stderr and "ERROR: AddressSanitizer" not in r.stderr, report
    assert r.returncode == 0, report
    assert "cpu-small: 0 failure(s)" in r.stdout, report
