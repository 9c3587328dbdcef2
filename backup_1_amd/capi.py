"""ctypes binding of libdecx_hip.so, the C ABI declared in include/decx_hip.h.

This is what the tests and bench.py call.  There is no CPU fallback: if the shared library is missing or the
device is not an MI355X the calls raise.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdecx_hip.so")

H2D, D2H, D2D = 1, 2, 3
CONV_NO_COMPENSATE, CONV_ZERO_COMPENSATE = 0, 1

# every symbol include/decx_hip.h declares; tests check the library exports all of them
SYMBOLS = [
    "decx_hip_init", "decx_hip_is_init", "decx_hip_device_info", "decx_hip_malloc", "decx_hip_free", "decx_hip_memset",
    "decx_hip_host_malloc", "decx_hip_host_free", "decx_hip_memcpy2d", "decx_hip_memcpy", "decx_hip_sync",
    "decx_hip_sgemm", "decx_hip_sgemm_async", "decx_hip_hgemm_f32acc", "decx_hip_hgemm_f32acc_async",
    "decx_hip_conv2_im2col_f32", "decx_hip_conv2_im2col_f32_async", "decx_hip_timer_start", "decx_hip_timer_stop",
    "decx_hip_last_error", "decx_hip_set_sgemm_variant", "decx_hip_set_hgemm_variant", "decx_hip_stream",
    "decx_hip_sgemm_splitk", "decx_hip_sgemm_batched", "decx_hip_hgemm_f32acc_batched", "decx_hip_gemm3_host_f32", "decx_hip_gemm3_host_f16",
    "decx_hip_conv2_im2col_f32_fused", "decx_hip_conv2_im2col_f16", "decx_hip_conv2_im2col_f16_async", "decx_hip_sgemm_relu", "decx_hip_relu_f32", "decx_hip_relu_f32_async",
    "decx_hip_relu_f32_rec", "decx_hip_relu_f32_backward", "decx_hip_gemm_host_f32", "decx_hip_gemm_host_f16",
    "decx_hip_b_read_extent", "decx_hip_sgemm_plan", "decx_hip_sgemm_plan_split", "decx_hip_hgemm_plan", "decx_hip_hgemm_plan_split", "decx_hip_conv_plan_split", "decx_hip_conv_patch_offsets_fit", "decx_hip_set_splitk_mode", "decx_hip_hgemm_f32acc_noalloc", "decx_hip_release_tmp", "decx_hip_tmp_malloc", "decx_hip_tmp_free",
]


class DecxHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("decx_hip error 0x%x: %s" % (code, message.strip()))
        self.code = code


_lib = None


def lib():
    """Load libdecx_hip.so (built by backup_1_amd/csrc/Makefile).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `make -C backup_1_amd/csrc` (hipcc, gfx950)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        P, I, Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        PP, PI, PF, PZ = ctypes.POINTER(P), ctypes.POINTER(I), ctypes.POINTER(ctypes.c_float), ctypes.POINTER(Z)
        sig = {
            "decx_hip_init": ([PI], I), "decx_hip_is_init": ([], I), "decx_hip_device_info": ([PI, PI, PZ], I),
            "decx_hip_malloc": ([PP, Z], I), "decx_hip_free": ([P], I), "decx_hip_memset": ([P, I, Z], I),
            "decx_hip_host_malloc": ([PP, Z], I), "decx_hip_host_free": ([P], I),
            "decx_hip_memcpy2d": ([P, Z, P, Z, Z, Z, I], I), "decx_hip_memcpy": ([P, P, Z, I], I),
            "decx_hip_sync": ([], I),
            "decx_hip_sgemm": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_sgemm_async": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_hgemm_f32acc": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_hgemm_f32acc_async": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_conv2_im2col_f32": ([P, I, I, I, Z, P, I, I, I, Z, Z, P, I, Z, I], I),
            "decx_hip_conv2_im2col_f32_async": ([P, I, I, I, Z, P, I, I, I, Z, Z, P, I, Z, I], I),
            "decx_hip_stream": ([], P), "decx_hip_release_tmp": ([], I), "decx_hip_tmp_malloc": ([ctypes.POINTER(ctypes.c_void_p), Z], I),
            "decx_hip_tmp_free": ([P], I),
            "decx_hip_sgemm_splitk": ([P, I, P, I, P, I, P, I, I, I, I, I], I),
            "decx_hip_sgemm_batched": ([P, I, Z, P, I, Z, P, I, Z, P, I, Z, I, I, I, I], I),
            "decx_hip_hgemm_f32acc_batched": ([P, I, Z, P, I, Z, P, I, Z, P, I, Z, I, I, I, I], I),
            "decx_hip_gemm3_host_f32": ([P, I, Z, P, I, Z, P, I, Z, P, I, Z, I, I, I, I], I),
            "decx_hip_gemm3_host_f16": ([P, I, Z, P, I, Z, P, I, Z, P, I, Z, I, I, I, I], I),
            "decx_hip_conv2_im2col_f32_fused": ([P, I, I, I, Z, P, I, I, I, Z, Z, P, I, Z, I, P, I], I),
            "decx_hip_conv2_im2col_f16": ([P, I, I, I, Z, P, I, I, I, Z, Z, P, I, Z, I, P, I], I),
            "decx_hip_conv2_im2col_f16_async": ([P, I, I, I, Z, P, I, I, I, Z, Z, P, I, Z, I, P, I], I),
            "decx_hip_sgemm_relu": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_gemm_host_f32": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_gemm_host_f16": ([P, I, P, I, P, I, P, I, I, I, I], I),
            "decx_hip_relu_f32": ([P, P, Z], I), "decx_hip_relu_f32_async": ([P, P, Z], I),
            "decx_hip_relu_f32_rec": ([P, P, P, Z], I), "decx_hip_relu_f32_backward": ([P, P, P, Z], I),
            "decx_hip_timer_start": ([], I), "decx_hip_timer_stop": ([PF], I),
            "decx_hip_last_error": ([], ctypes.c_char_p),
            "decx_hip_set_sgemm_variant": ([I], I), "decx_hip_set_hgemm_variant": ([I], I),
            "decx_hip_b_read_extent": ([I, I, I], I),
            "decx_hip_sgemm_plan": ([I, I, I, I, ctypes.c_long, ctypes.c_long, I], I),
            "decx_hip_sgemm_plan_split": ([I, I, I, I, ctypes.c_long, ctypes.c_long, I, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)], I),
            "decx_hip_hgemm_plan_split": ([I, I, I, I, ctypes.c_long, ctypes.c_long, I, ctypes.POINTER(ctypes.c_int)], I),
            "decx_hip_conv_plan_split": ([I, I, I, I, I, I, I, ctypes.POINTER(ctypes.c_int)], I),
            "decx_hip_hgemm_plan": ([I, I, I, I, ctypes.c_long, ctypes.c_long, I, PI], I),
            "decx_hip_conv_patch_offsets_fit": ([I, I, I, Z, I, I, I, I], I),
            "decx_hip_set_splitk_mode": ([I], I),
            "decx_hip_hgemm_f32acc_noalloc": ([P, I, P, I, P, I, P, I, I, I, I, I], I),
        }
        for name, (args, res) in sig.items():
            fn = getattr(L, name)
            fn.argtypes, fn.restype = args, res
        _lib = L
    return _lib


PROBE_LIB_PATH = os.path.join(_HERE, "libdecx_hip_probe.so")
_probe = None


def probe_lib():
    """Load libdecx_hip_probe.so, the measurement instruments (`make -C backup_1_amd/csrc probes`): ablation builds of
    the large fp16 tile kernel and the calibration copy kernel.  Only bench.py's `ladder` and `copy` legs use it."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_LIB_PATH):
            raise FileNotFoundError("%s is missing: build it with `make -C backup_1_amd/csrc probes`" % PROBE_LIB_PATH)
        L = ctypes.CDLL(PROBE_LIB_PATH)
        P, I, Z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        L.decx_probe_hgemm.argtypes, L.decx_probe_hgemm.restype = [I, I, P, P, I, P, I, P, I, I, I, I, I, I], I
        L.decx_probe_copy.argtypes, L.decx_probe_copy.restype = [P, P, P, Z], I
        _probe = L
    return _probe


def stream():
    return lib().decx_hip_stream()


def last_error():
    return lib().decx_hip_last_error().decode("utf-8", "replace")


def check(rc):
    if rc != 0:
        raise DecxHipError(rc, last_error())


def init():
    dev = ctypes.c_int(-1)
    check(lib().decx_hip_init(ctypes.byref(dev)))
    return dev.value


def device_info():
    cu, khz, mem = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    check(lib().decx_hip_device_info(ctypes.byref(cu), ctypes.byref(khz), ctypes.byref(mem)))
    return {"compute_units": cu.value, "clock_khz": khz.value, "hbm_bytes": mem.value}


def sync():
    check(lib().decx_hip_sync())


class DeviceBuffer:
    """A device allocation made through the C ABI, with numpy upload / download helpers."""

    def __init__(self, nbytes):
        p = ctypes.c_void_p()
        check(lib().decx_hip_malloc(ctypes.byref(p), nbytes))
        self.ptr, self.nbytes = p.value, nbytes

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        buf.upload(arr)
        return buf

    def upload(self, arr):
        arr = np.ascontiguousarray(arr)
        assert arr.nbytes <= self.nbytes
        check(lib().decx_hip_memcpy(self.ptr, arr.ctypes.data, arr.nbytes, H2D))

    def download(self, shape, dtype):
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        check(lib().decx_hip_memcpy(out.ctypes.data, self.ptr, out.nbytes, D2H))
        return out

    def fill(self, byte):
        check(lib().decx_hip_memset(self.ptr, byte, self.nbytes))

    def free(self):
        if self.ptr:
            check(lib().decx_hip_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def sgemm(dA, lda, dB, ldb, dD, ldd, M, N, K, dC=None, ldc=0, blocking=True):
    fn = lib().decx_hip_sgemm if blocking else lib().decx_hip_sgemm_async
    check(fn(dA, lda, dB, ldb, dC, ldc, dD, ldd, M, N, K))


def hgemm(dA, lda, dB, ldb, dD, ldd, M, N, K, dC=None, ldc=0, blocking=True):
    fn = lib().decx_hip_hgemm_f32acc if blocking else lib().decx_hip_hgemm_f32acc_async
    check(fn(dA, lda, dB, ldb, dC, ldc, dD, ldd, M, N, K))


def conv2_im2col(dsrc, H, W, dpitch, src_row_stride, dfilt, N, kh, kw, filt_stride, filt_row_stride, ddst, dst_dpitch,
                 dst_row_stride, flag, blocking=True):
    fn = lib().decx_hip_conv2_im2col_f32 if blocking else lib().decx_hip_conv2_im2col_f32_async
    check(fn(dsrc, H, W, dpitch, src_row_stride, dfilt, N, kh, kw, filt_stride, filt_row_stride, ddst, dst_dpitch,
             dst_row_stride, flag))


def timer_start():
    check(lib().decx_hip_timer_start())


def timer_stop():
    ms = ctypes.c_float()
    check(lib().decx_hip_timer_stop(ctypes.byref(ms)))
    return ms.value
