#!/usr/bin/env python3
"""Benchmark of the dense-contraction path on one MI355X.

A "step" is one de::cuda::GEMM-on-GPU_Matrix equivalent: one call of decx_hip_sgemm on device-resident operands.
Headline workload (the configuration the metric is quoted on): fp32 square GEMM, M = N = K = 8192, row-major,
entries uniform[-1,1] from a fixed seed.  The same JSON line also carries, under "also", the other configurations the
metric names (fp16 8192^3 with fp32 accumulation, fp32 4096^3, the ragged 3000x1500x4500 GEMM, the fused im2col
convolution), each timed the same way, and a CPU baseline (the restated DECX_cpu thread-pool SGEMM from oracle/) timed
on this box's host cores on a bounded slab of the headline workload.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MATRIX_TFLOPS = 157.3     # MI355X dense fp32 MFMA
PEAK_FP16_MATRIX_TFLOPS = 2516.6    # MI355X dense fp16 MFMA (2.5 PFLOP/s)
PEAK_HBM_GBPS = 8000.0              # MI355X HBM3E
# HBM-side bytes per launch of the headline kernel come from the FETCH_SIZE / WRITE_SIZE counter runs recorded in
# profiles/traffic.json (kernel, bytes, the commit they were measured at).  Counters cannot be read from inside this
# script; the figure is only reported for the workload and tile shape it was measured on, with its source beside it.
TRAFFIC_FILE = os.path.join("profiles", "traffic.json")
# the kernel that runs the headline product, by --sgemm-variant (0 = the library's own choice, which is shape 26 there)
HEADLINE_KERNELS = {0: "sgemm_dma_kernel<256x256x16, 4x2 waves, LDS-DMA loads>", 26: "sgemm_dma_kernel<256x256x16, 4x2 waves, LDS-DMA loads>",
                    7: "sgemm_tile_kernel<256x256x16, 4x2 waves>", 1: "sgemm_tile_kernel<256x256x16, 2x2 waves>"}


def measured_traffic(size, sgemm_variant):
    """(bytes per launch, where the figure comes from) of the headline kernel, or (None, reason)."""
    try:
        with open(os.path.join(ROOT, TRAFFIC_FILE)) as f:
            table = json.load(f)["kernels"]
    except (OSError, ValueError, KeyError) as e:
        return None, "%s unreadable: %s" % (TRAFFIC_FILE, e)
    for name, rec in table.items():
        if rec.get("size") == size and sgemm_variant in rec.get("sgemm_variants", []):
            return rec["traffic_bytes"], "%s: %s, measured at commit %s" % (TRAFFIC_FILE, name, rec.get("measured_at_commit"))
    return None, "no counter run recorded for this size and tile shape"


def verify_sgemm_rows(capi, dD, ldd, A, B, nrows, seed):
    """Bit-compare `nrows` sampled rows of the device result with the oracle's fused chain (outside any timed region;
    the oracle is only the checker)."""
    import oracle
    M, N = A.shape[0], B.shape[1]
    rows = np.sort(np.random.Generator(np.random.PCG64(seed)).choice(M, size=min(nrows, M), replace=False)).astype(np.int32)
    got = dD.download((M, ldd), np.float32)[rows, :N]
    want = oracle.sgemm_chain_rows(A, B, rows)
    return bool(np.array_equal(got.view(np.uint32), want.view(np.uint32))), int(rows.size)


def verify_hgemm_rows(capi, dD, ldd, Abits, Bbits, nrows, seed):
    """Sampled rows of the binary16 result against fp64 on the same binary16 inputs: max |x - r| / sum |a||b| (less
    the half-ulp of the final rounding) must stay below 2e-3."""
    import oracle
    M, N = Abits.shape[0], Bbits.shape[1]
    rows = np.sort(np.random.Generator(np.random.PCG64(seed)).choice(M, size=min(nrows, M), replace=False)).astype(np.int32)
    got = dD.download((M, ldd), np.uint16)[rows, :N].view(np.float16).astype(np.float64)
    ref, scale = oracle.gemm_f64_rows_f16(Abits, Bbits, rows)
    err = float(np.max((np.abs(got - ref) - np.abs(ref) / 2048.0) / scale))
    return err < 2e-3, max(err, 0.0), int(rows.size)


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


# Side workloads only (the headline runs exactly --warmup + --steps launches): lower bounds on the warm-up and on the
# timed region, in milliseconds of back-to-back launches.  A sub-millisecond kernel launched after a host-side pause
# starts on a chip that has clocked down and speeds up over the first tens of milliseconds (config 4 of the convolution:
# 0.079 ms per launch at first, 0.069 ms from about 250 launches on), so a few dozen launches measure the ramp.
SIDE_MIN_WARM_MS = 0.0
SIDE_MIN_TIMED_MS = 0.0


def time_launches(capi, launch, steps, warmup):
    """Returns (wall ms per step, HIP-event ms per step) for back-to-back launches on the library's stream: `warmup`
    untimed and `steps` timed ones, both extended to the SIDE_MIN_* durations when those are set."""
    t0 = time.perf_counter()
    for _ in range(warmup):
        launch()
    capi.sync()
    if SIDE_MIN_WARM_MS > 0:
        while (time.perf_counter() - t0) * 1e3 < SIDE_MIN_WARM_MS:
            for _ in range(max(warmup, 1)):
                launch()
            capi.sync()
    if SIDE_MIN_TIMED_MS > 0 and warmup > 0:
        t1 = time.perf_counter()
        for _ in range(warmup):
            launch()
        capi.sync()
        pilot_ms = (time.perf_counter() - t1) * 1e3 / warmup
        steps = max(steps, min(int(SIDE_MIN_TIMED_MS / max(pilot_ms, 1e-3)) + 1, 5000))
    t0 = time.perf_counter()
    capi.timer_start()
    for _ in range(steps):
        launch()
    ev_ms = capi.timer_stop()
    capi.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms / steps, ev_ms / steps


def bench_sgemm(capi, workloads, M, K, N, steps, warmup, seed, dist="uniform", verify_rows=0):
    if dist == "uniform":
        A, B = workloads.uniform_pm1((M, K), seed), workloads.uniform_pm1((K, N), seed + 1)
    else:
        A, B = workloads.normal((M, K), seed), workloads.normal((K, N), seed + 1)
    pad8 = lambda x: (x + 7) // 8 * 8
    lda, ldb, ldd = pad8(K), pad8(N), pad8(N)
    Ab = np.zeros((M, lda), np.float32); Ab[:, :K] = A
    Bb = np.zeros((K, ldb), np.float32); Bb[:, :N] = B
    dA, dB = capi.DeviceBuffer.from_numpy(Ab), capi.DeviceBuffer.from_numpy(Bb)
    dD = capi.DeviceBuffer(M * ldd * 4)
    launch = lambda: capi.sgemm(dA.ptr, lda, dB.ptr, ldb, dD.ptr, ldd, M, N, K, blocking=False)
    wall, ev = time_launches(capi, launch, steps, warmup)
    flops = 2.0 * M * N * K
    med, mn = per_launch_stats(capi, launch, 10)
    out = {"ms_wall": wall, "ms_kernel": ev, "tflops": flops / (wall * 1e-3) / 1e12, "tflops_kernel": flops / (ev * 1e-3) / 1e12,
           "flops": flops, "A": A, "B": B, "ms_median": med, "ms_min": mn}
    if verify_rows:
        # the result of the launches just timed, checked after the timed region
        out["verified"], out["verified_rows"] = verify_sgemm_rows(capi, dD, ldd, A, B, verify_rows, seed + 2)
    return out


def bench_hgemm(capi, workloads, n, steps, warmup, seed, shape=None, verify_rows=0):
    M, K, N = shape if shape else (n, n, n)
    A = workloads.uniform_pm1((M, K), seed).astype(np.float16).view(np.uint16)
    B = workloads.uniform_pm1((K, N), seed + 1).astype(np.float16).view(np.uint16)
    dA, dB = capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(B)
    dD = capi.DeviceBuffer(M * N * 2)
    launch = lambda: capi.hgemm(dA.ptr, K, dB.ptr, N, dD.ptr, N, M, N, K, blocking=False)
    wall, ev = time_launches(capi, launch, steps, warmup)
    flops = 2.0 * M * N * K
    out = {"ms_wall": wall, "ms_kernel": ev, "tflops": flops / (wall * 1e-3) / 1e12, "tflops_kernel": flops / (ev * 1e-3) / 1e12}
    if verify_rows:
        out["verified"], out["max_rel_err"], out["verified_rows"] = verify_hgemm_rows(capi, dD, N, A, B, verify_rows, seed + 2)
    return out


def bench_two_launch_ab(capi, seed=2024, count=40):
    """Seeded random sizes (M, N in 1500..9000, K in 512..8192): each product as the library runs it (two launches where
    decx_hip_*_plan_split says so) against the same product kept in one launch (variants 34 / 20), fp32 and fp16;
    operands uniform in (-1, 1) uploaded once per size from a 64 MB host block, results compared (fp32: equal bits)."""
    import ctypes
    L = capi.lib()
    rng = np.random.Generator(np.random.PCG64(seed))
    block = (np.random.Generator(np.random.PCG64(seed + 1)).random(1 << 24, dtype=np.float32) * 2 - 1)
    def fill(dev, count_elems, half):
        src = block.astype(np.float16) if half else block
        size = src.itemsize
        for start in range(0, count_elems, src.size):
            n = min(src.size, count_elems - start)
            capi.check(L.decx_hip_memcpy(dev.ptr + start * size, src.ctypes.data, n * size, 1))
    def timed(launch):
        for _ in range(3):
            launch()
        capi.sync()
        best = 1e9
        for _ in range(3):
            capi.timer_start()
            for _ in range(8):
                launch()
            best = min(best, capi.timer_stop() / 8)
        return best
    rows = []
    while len(rows) < count:
        M, N = int(rng.integers(1500, 9000)), int(rng.integers(1500, 9000))
        K = int(rng.choice([512, 1024, 1500, 2048, 4096, 8192]))
        if 1.0 * M * N * K > 3.0e11:
            continue
        for half in (False, True):
            unit, size = (16, 2) if half else (8, 4)
            lda, ldb = (K + unit - 1) // unit * unit, (N + unit - 1) // unit * unit
            tile, by_columns = ctypes.c_int(0), ctypes.c_int(0)
            first = (L.decx_hip_hgemm_plan_split(M, N, K, 1, lda, ldb, 1, ctypes.byref(by_columns)) if half else
                     L.decx_hip_sgemm_plan_split(M, N, K, 1, lda, ldb, 1, ctypes.byref(tile), ctypes.byref(by_columns)))
            if first <= 0:
                continue
            dA, dB = capi.DeviceBuffer(M * lda * size), capi.DeviceBuffer(K * ldb * size)
            dD, dE = capi.DeviceBuffer(M * ldb * size), capi.DeviceBuffer(M * ldb * size)
            fill(dA, M * lda, half)
            fill(dB, K * ldb, half)
            gemm, knob, one_launch = ((capi.hgemm, L.decx_hip_set_hgemm_variant, 20) if half else
                                      (capi.sgemm, L.decx_hip_set_sgemm_variant, 34))
            t = {}
            for v, dst in ((0, dD), (one_launch, dE), (0, dD), (one_launch, dE)):
                knob(v)
                t[v] = min(t.get(v, 1e9), timed(lambda: gemm(dA.ptr, lda, dB.ptr, ldb, dst.ptr, ldb, M, N, K, blocking=False)))
            knob(0)
            dt = np.uint16 if half else np.uint32
            a, b = dD.download((M, ldb), dt)[:, :N], dE.download((M, ldb), dt)[:, :N]
            if half:
                same = bool(np.max(np.abs(a.view(np.float16).astype(np.float32) - b.view(np.float16).astype(np.float32))) <= 4e-3 * np.sqrt(K))
            else:
                same = bool(np.array_equal(a, b))
            rows.append({"what": "%s %dx%dx%d (MxKxN)" % ("fp16" if half else "fp32", M, K, N),
                         "first_launch": "%d %s" % (first, "columns" if by_columns.value else "rows") + ("" if half else " on tile %d" % tile.value),
                         "two_launches_ms": round(t[0], 5), "one_launch_ms": round(t[one_launch], 5), "ratio": round(t[0] / t[one_launch], 4),
                         "tflops": round(2.0 * M * N * K / t[0] / 1e9, 1), "one_launch_tflops": round(2.0 * M * N * K / t[one_launch] / 1e9, 1),
                         "results_agree": same})
            for d in (dA, dB, dD, dE):
                d.free()
    return rows


LADDER_BUILDS = [(0, "2 LDS stages of 64 k, one tile per workgroup"), (1, "4 LDS stages of 32 k"), (2, "5 LDS stages of 32 k"),
                 (3, "2 LDS stages of 64 k, one workgroup per CU walks its tiles as one stream of K steps"),
                 (5, "2 LDS stages of 64 k, 4 waves of 128 x 128 (one per SIMD) instead of 8 of 128 x 64"),
                 (6, "4 LDS stages of 32 k, 4 waves of 128 x 128")]
LADDER_RUNGS = [(7, "matrix instructions only"), (5, "+ LDS fragment reads"), (12, "+ global->LDS loads that never move on (cache hits)"),
                (4, "+ global->LDS loads (whole K walk, no stores)"), (0, "whole kernel")]
LADDER_ORDERS = [(16, "whole kernel, matrix instructions row block by row block, columns ascending"),
                 (32, "whole kernel, matrix instructions column block by column block")]


def bench_fp16_ladder(capi, workloads, steps, warmup, n=8192):
    """The large fp16 tile kernel in several builds with parts of its K walk left out (libdecx_hip_probe.so), on
    uniform[-1,1] operands and on all-zero ones: what each part costs, and what the operand values cost (the same
    instructions on zeros draw less power, so the chip clocks higher).  Every rung issues the same matrix
    instructions: 2 n^3 flop."""
    probe, stream = capi.probe_lib(), capi.stream()
    A = workloads.uniform_pm1((n, n), 5).astype(np.float16).view(np.uint16)
    B = workloads.uniform_pm1((n, n), 6).astype(np.float16).view(np.uint16)
    dA, dB = capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(B)
    dZ = capi.DeviceBuffer(n * n * 2)
    dZ.fill(0)
    dD = capi.DeviceBuffer(n * n * 2)
    out = []
    cases = [(kind, kname, ab, what) for kind, kname in LADDER_BUILDS for ab, what in LADDER_RUNGS]
    cases += [(0, LADDER_BUILDS[0][1], ab, what) for ab, what in LADDER_ORDERS]
    for kind, kname, ablate, what in cases:
        row = {"build": kind, "build_what": kname, "ablate": ablate, "what": what}
        for tag, a, b in (("uniform", dA, dB), ("zeros", dZ, dZ)):
            def launch():
                rc = probe.decx_probe_hgemm(kind, ablate, stream, a.ptr, n, b.ptr, n, dD.ptr, n, n, n, n, 8, 0)
                if rc != 0:
                    raise RuntimeError("decx_probe_hgemm(kind %d, ablate %d) returned %d" % (kind, ablate, rc))
            wall, ev = time_launches(capi, launch, steps, warmup)
            row["tflops_" + tag] = round(2.0 * n ** 3 / (ev * 1e-3) / 1e12, 1)
            row["ms_" + tag] = round(ev, 4)
        out.append(row)
    return out


def bench_conv(capi, workloads, steps, warmup, H=224, W=224, C=64, N=128):
    kh = kw = 3
    src, filt = workloads.conv_case(H=H, W=W, C=C, N=N)
    fb = np.zeros((N, kh, 4, C), np.float32); fb[:, :, :kw, :] = filt       # TensorArray: wpitch = ceil4(kw)
    dS, dF = capi.DeviceBuffer.from_numpy(src), capi.DeviceBuffer.from_numpy(fb)
    dD = capi.DeviceBuffer(H * W * N * 4)
    launch = lambda: capi.conv2_im2col(dS.ptr, H, W, C, W * C, dF.ptr, N, kh, kw, kh * 4 * C, 4 * C, dD.ptr, N, W * N, 1,
                                       blocking=False)
    wall, ev = time_launches(capi, launch, steps, warmup)
    flops = 2.0 * H * W * N * kh * kw * C
    return {"ms_wall": wall, "ms_kernel": ev, "tflops": flops / (wall * 1e-3) / 1e12, "tflops_kernel": flops / (ev * 1e-3) / 1e12}


def bench_hconv(capi, workloads, steps, warmup, H=224, W=224, C=64, N=128):
    """config 4 in binary16 with fp32 accumulation (decx_hip_conv2_im2col_f16_async); same flop count as bench_conv."""
    kh = kw = 3
    src, filt = workloads.conv_case(H=H, W=W, C=C, N=N)
    fb = np.zeros((N, kh, 4, C), np.float16); fb[:, :, :kw, :] = filt.astype(np.float16)
    dS, dF = capi.DeviceBuffer.from_numpy(src.astype(np.float16).view(np.uint16)), capi.DeviceBuffer.from_numpy(fb.view(np.uint16))
    dD = capi.DeviceBuffer(H * W * N * 2)
    launch = lambda: capi.check(capi.lib().decx_hip_conv2_im2col_f16_async(
        dS.ptr, H, W, C, W * C, dF.ptr, N, kh, kw, kh * 4 * C, 4 * C, dD.ptr, N, W * N, 1, None, 0))
    wall, ev = time_launches(capi, launch, steps, warmup)
    flops = 2.0 * H * W * N * kh * kw * C
    return {"ms_wall": wall, "ms_kernel": ev, "tflops": flops / (wall * 1e-3) / 1e12, "tflops_kernel": flops / (ev * 1e-3) / 1e12}


def per_launch_stats(capi, launch, reps):
    """Each launch timed on its own between two HIP events: (median ms, min ms)."""
    ms = []
    for _ in range(reps):
        capi.timer_start()
        launch()
        ms.append(capi.timer_stop())
    ms.sort()
    return ms[len(ms) // 2], ms[0]


class PinnedArray:
    """Host memory from decx_hip_host_malloc viewed as a numpy array (what Page_Locked DECX containers hold)."""

    def __init__(self, capi, shape, dtype):
        import ctypes
        self.capi, self.nbytes = capi, int(np.prod(shape)) * np.dtype(dtype).itemsize
        p = ctypes.c_void_p()
        capi.check(capi.lib().decx_hip_host_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value
        self.array = np.ctypeslib.as_array((ctypes.c_byte * self.nbytes).from_address(self.ptr)).view(dtype).reshape(shape)

    def free(self):
        self.array = None
        self.capi.check(self.capi.lib().decx_hip_host_free(self.ptr))


def bench_host_resident_gemm(capi, A, B, reps):
    """de::cuda::GEMM(Matrix<float>...) equivalent (GEMM.h:56-131) through decx_hip_gemm_host_f32: pinned host operands,
    device allocation, uploads, kernel and download (pipelined over row panels) -- the PCIe-inclusive figure."""
    M, K = A.shape
    N = B.shape[1]
    hA, hB, hD = PinnedArray(capi, (M, K), np.float32), PinnedArray(capi, (K, N), np.float32), PinnedArray(capi, (M, N), np.float32)
    hA.array[:], hB.array[:] = A, B
    L = capi.lib()
    best = None
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        capi.check(L.decx_hip_gemm_host_f32(hA.ptr, K, hB.ptr, N, None, 0, hD.ptr, N, M, N, K))
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    for h in (hA, hB, hD): h.free()
    return {"ms": best * 1e3, "tflops": 2.0 * M * N * K / best / 1e12, "pcie_bytes": 4.0 * (M * K + K * N + M * N)}


def bench_host_resident_gemm3(capi, workloads, count, n, reps):
    """de::cuda::GEMM3(MatrixArray...) equivalent (GEMM3.h:27-36) through decx_hip_gemm3_host_f32: `count` products of n^3
    between pinned host arrays; uploads, kernels and downloads of consecutive matrices overlap on three streams."""
    hA, hB, hD = (PinnedArray(capi, (count, n, n), np.float32) for _ in range(3))
    for i in range(count):
        hA.array[i], hB.array[i] = workloads.uniform_pm1((n, n), 700 + 2 * i), workloads.uniform_pm1((n, n), 701 + 2 * i)
    best = None
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        capi.check(capi.lib().decx_hip_gemm3_host_f32(hA.ptr, n, n * n, hB.ptr, n, n * n, None, 0, 0, hD.ptr, n, n * n, n, n, n, count))
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    for h in (hA, hB, hD): h.free()
    return {"ms": best * 1e3, "tflops": 2.0 * count * n ** 3 / best / 1e12, "pcie_bytes": 12.0 * count * n * n}


def bench_host_resident_conv(capi, workloads, reps):
    """de::cuda::Conv2_MK_im2col(Tensor, TensorArray, Tensor) equivalent (conv2_mk_im2col.h:278-306): upload the
    tensor and the filters, fused kernel, download the result."""
    H = W = 224; C = 64; N = 128; kh = kw = 3
    src, filt = workloads.conv_case()
    hS, hF, hD = PinnedArray(capi, (H, W, C), np.float32), PinnedArray(capi, (N, kh, 4, C), np.float32), PinnedArray(capi, (H, W, N), np.float32)
    hS.array[:] = src
    hF.array[:] = 0
    hF.array[:, :, :kw, :] = filt
    dS, dF, dD = capi.DeviceBuffer(hS.nbytes), capi.DeviceBuffer(hF.nbytes), capi.DeviceBuffer(hD.nbytes)
    L = capi.lib()
    best = None
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        capi.check(L.decx_hip_memcpy(dS.ptr, hS.ptr, hS.nbytes, capi.H2D))
        capi.check(L.decx_hip_memcpy(dF.ptr, hF.ptr, hF.nbytes, capi.H2D))
        capi.conv2_im2col(dS.ptr, H, W, C, W * C, dF.ptr, N, kh, kw, kh * 4 * C, 4 * C, dD.ptr, N, W * N, 1)
        capi.check(L.decx_hip_memcpy(hD.ptr, dD.ptr, hD.nbytes, capi.D2H))
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    for h in (hS, hF, hD): h.free()
    return {"ms": best * 1e3, "tflops": 2.0 * H * W * N * kh * kw * C / best / 1e12}


def cpu_conv_baseline(workloads):
    """The reference has no CPU convolution; its CPU equivalent is a host im2col in the reference's k order followed by
    the restated DECX_cpu thread-pool SGEMM on the 50176 x 576 x 128 lowered problem."""
    import oracle
    H = W = 224; C = 64; N = 128; kh = kw = 3
    src, filt = workloads.conv_case()
    padded = np.zeros((H + 2, W + 2, C), np.float32)
    cols = np.zeros((H * W, kh * kw * C), np.float32)
    out = np.zeros((H * W, N), np.float32)
    Bm = np.ascontiguousarray(filt.reshape(N, kh * kw * C).T)
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        padded[1:-1, 1:-1] = src
        for ki in range(kh):
            for kj in range(kw):
                cols[:, (ki * kw + kj) * C:(ki * kw + kj + 1) * C] = padded[ki:ki + H, kj:kj + W].reshape(H * W, C)
        t1 = time.perf_counter()
        oracle.decx_cpu_sgemm(cols, Bm, out=out)
        t2 = time.perf_counter()
        if best is None or t2 - t0 < best[0]: best = (t2 - t0, t1 - t0, t2 - t1)
    flops = 2.0 * H * W * N * kh * kw * C
    return {"tflops": round(flops / best[0] / 1e12, 4), "ms": round(best[0] * 1e3, 2), "im2col_ms": round(best[1] * 1e3, 2),
            "sgemm_ms": round(best[2] * 1e3, 2), "sgemm_tflops": round(flops / best[2] / 1e12, 4),
            "what": "numpy im2col (reference k order, single thread) + restated DECX_cpu SGEMM on 50176x576x128, best of 2"}


def bench_relu(capi, workloads, steps, warmup):
    """de::nn::ReLU_f over a 8192 x 8192 fp32 matrix (256 MiB in, 256 MiB out): HBM-bound, 8 bytes per element."""
    n = 8192 * 8192
    x = workloads.normal((n,), 77)
    dX, dY = capi.DeviceBuffer.from_numpy(x), capi.DeviceBuffer(n * 4)
    launch = lambda: capi.check(capi.lib().decx_hip_relu_f32_async(dX.ptr, dY.ptr, n))
    wall, ev = time_launches(capi, launch, steps, warmup)
    return {"ms_wall": wall, "ms_kernel": ev, "gbps": 8.0 * n / (ev * 1e-3) / 1e9}


def bench_conv_fused(capi, workloads, steps, warmup):
    """config 4 with the bias + ReLU epilogue (decx_hip_conv2_im2col_f32_fused); same flop count as bench_conv."""
    H = W = 224; C = 64; N = 128; kh = kw = 3
    src, filt = workloads.conv_case()
    fb = np.zeros((N, kh, 4, C), np.float32); fb[:, :, :kw, :] = filt
    dS, dF = capi.DeviceBuffer.from_numpy(src), capi.DeviceBuffer.from_numpy(fb)
    dB = capi.DeviceBuffer.from_numpy(workloads.normal((N,), 78))
    dD = capi.DeviceBuffer(H * W * N * 4)
    import ctypes
    fn = capi.lib().decx_hip_conv2_im2col_f32_fused
    # the arguments converted once, as a C or C++ caller's are: ctypes otherwise spends a microsecond per call on them
    args = tuple(t(v) for t, v in zip(fn.argtypes, (dS.ptr, H, W, C, W * C, dF.ptr, N, kh, kw, kh * 4 * C, 4 * C, dD.ptr, N, W * N,
                                                    1, dB.ptr, 1)))
    capi.check(fn(*args))

    def launch():
        rc = fn(*args)
        if rc:
            capi.check(rc)
    best, med = time_blocking_calls(launch, steps, warmup)   # the fused entry point is synchronous: time whole calls
    flops = 2.0 * H * W * N * kh * kw * C
    return {"ms_wall": best, "ms_median": med, "tflops": flops / (best * 1e-3) / 1e12}


def time_blocking_calls(call, steps, warmup):
    """(min, median) wall milliseconds of whole synchronous calls, one after the other: like every side workload, after
    at least SIDE_MIN_WARM_MS of calls (the chip clocks up over the first tens of milliseconds) and over at least
    SIDE_MIN_TIMED_MS of them."""
    t_end = time.perf_counter() + SIDE_MIN_WARM_MS * 1e-3
    done = 0
    while done < warmup or time.perf_counter() < t_end:
        call()
        done += 1
    ms = []
    t_end = time.perf_counter() + SIDE_MIN_TIMED_MS * 1e-3
    while len(ms) < steps or time.perf_counter() < t_end:
        t0 = time.perf_counter()
        call()
        ms.append((time.perf_counter() - t0) * 1e3)
    ms.sort()
    return ms[0], ms[len(ms) // 2]


def bench_batched(capi, workloads, fp16, batch, n):
    """`batch` independent n^3 products in one launch of the batched entry point (the kernel step of GEMM3 over a
    MatrixArray); the entry point blocks, so whole calls are timed."""
    es = 2 if fp16 else 4
    mats_a, mats_b = [], []
    for i in range(batch):
        a, b = workloads.uniform_pm1((n, n), 900 + 2 * i), workloads.uniform_pm1((n, n), 901 + 2 * i)
        if fp16:
            a, b = a.astype(np.float16).view(np.uint16), b.astype(np.float16).view(np.uint16)
        mats_a.append(a); mats_b.append(b)
    dA, dB = capi.DeviceBuffer.from_numpy(np.stack(mats_a)), capi.DeviceBuffer.from_numpy(np.stack(mats_b))
    dD = capi.DeviceBuffer(batch * n * n * es)
    fn = capi.lib().decx_hip_hgemm_f32acc_batched if fp16 else capi.lib().decx_hip_sgemm_batched
    call = lambda: capi.check(fn(dA.ptr, n, n * n, dB.ptr, n, n * n, None, 0, 0, dD.ptr, n, n * n, n, n, n, batch))
    best, med = time_blocking_calls(call, 20, 5)
    flops = 2.0 * batch * n ** 3
    return {"tflops": round(flops / (best * 1e-3) / 1e12, 2), "ms_per_call_min": round(best, 4), "ms_per_call_median": round(med, 4)}


def bench_blocking_calls(capi, workloads, steps, warmup):
    """What a caller of the synchronous drop-in API (every call of the reference's API blocks) sees on kernels of tens of
    microseconds: whole calls of decx_hip_sgemm at 1024^3 beside the same kernel enqueued back to back, and the floor
    of a blocking call (a 64-float ReLU: launch + wait, next to nothing to compute)."""
    n = 1024
    A, B = workloads.uniform_pm1((n, n), 77), workloads.uniform_pm1((n, n), 78)
    dA, dB, dD = capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(B), capi.DeviceBuffer(n * n * 4)
    steps = max(steps, 200)
    best, med = time_blocking_calls(lambda: capi.sgemm(dA.ptr, n, dB.ptr, n, dD.ptr, n, n, n, n, blocking=True), steps, warmup)
    _, ev = time_launches(capi, lambda: capi.sgemm(dA.ptr, n, dB.ptr, n, dD.ptr, n, n, n, n, blocking=False), steps, warmup)
    tiny = capi.DeviceBuffer(256)
    tiny.fill(0)
    fbest, fmed = time_blocking_calls(lambda: capi.check(capi.lib().decx_hip_relu_f32(tiny.ptr, tiny.ptr, 64)), steps, warmup)
    flops = 2.0 * n ** 3
    return {"fp32_1024_blocking_call": {"ms_per_call_min": round(best, 4), "ms_per_call_median": round(med, 4),
                                        "tflops": round(flops / (best * 1e-3) / 1e12, 2),
                                        "ms_per_launch_enqueued": round(ev, 4)},
            "blocking_call_floor_relu_64_floats": {"ms_per_call_min": round(fbest, 4), "ms_per_call_median": round(fmed, 4)}}


SWEEP_FP32 = [(1024, 1024, 1024), (1536, 1536, 1536), (2048, 2048, 2048), (2560, 2560, 2560), (3072, 3072, 3072), (4096, 4096, 4096),
              (6144, 6144, 6144), (640, 640, 640), (768, 768, 768), (896, 896, 896), (1152, 1152, 1152), (1280, 1280, 1280),
              (1664, 1664, 1664), (3000, 1500, 4500), (2816, 4096, 2816), (1920, 4096, 1920), (8192, 1024, 256), (4096, 4096, 64),
              (8192, 64, 8192), (4096, 128, 4096), (8192, 2048, 8192), (2048, 8192, 2048), (1024, 8192, 1024), (512, 8192, 512),
              (384, 8192, 384), (64, 65536, 1024), (128, 16384, 1024), (196, 4608, 512), (300, 200, 260), (8192, 8192, 8192),
              # tall results at most 256 wide (the shape of a lowered convolution)
              (409600, 576, 64), (147456, 1152, 128), (82944, 864, 96), (82944, 864, 224), (100000, 4096, 128), (300000, 128, 64),
              (200000, 128, 128), (30000, 512, 48), (262144, 288, 32), (150000, 2048, 256), (200000, 1024, 32), (400000, 32, 64),
              # results that run as two launches (whole rounds of a 256-row tile, then the rest); 34 = kept in one launch
              (4352, 4096, 4352), (4096, 4096, 4608), (6950, 2048, 5308), (3497, 1500, 5226), (6324, 512, 5986)]
SWEEP_FP32_VARIANTS = [2, 3, 4, 5, 7, 8, 9, 10, 14, 15, 16, 11, 12, 13, 23, 18, 19, 20, 21, 22, 24, 25, 26, 27, 28, 34]
SWEEP_CONV = [(224, 224, 64, 128, 3), (112, 112, 128, 128, 3), (56, 56, 256, 256, 3), (28, 28, 512, 512, 3), (128, 128, 128, 128, 5),
              (512, 512, 256, 256, 3), (224, 224, 64, 64, 3), (96, 96, 128, 256, 3), (28, 28, 256, 256, 3), (14, 14, 512, 512, 3),
              (180, 180, 128, 128, 3), (208, 208, 64, 128, 3), (256, 256, 64, 128, 3), (56, 56, 64, 256, 1),
              # two launches by output rows (whole rounds of the 256x256 tile, then the rest); 34 = kept in one launch
              (300, 300, 128, 256, 3), (385, 385, 256, 256, 3)]
SWEEP_CONV_VARIANTS = [2, 3, 4, 5, 7, 9, 10, 15, 16, 17, 11, 12, 13, 23, 29, 30, 31, 33, 34]
SWEEP_FP16 = [(8192, 8192, 8192), (4096, 4096, 4096), (2048, 2048, 2048), (1024, 1024, 1024), (3000, 1500, 4500), (64, 65536, 1024),
              (512, 8192, 512), (128, 16384, 2048),
              # results that run as two launches (whole rounds of the 256x256 tile, then the rest); 20 = kept in one launch
              (4352, 4096, 4352), (4013, 8192, 4775), (7336, 4096, 6806)]
SWEEP_FP16_VARIANTS = [1, 2, 7, 8, 9, 10, 15, 16, 17, 11, 20]


def sweep_one(capi, launch, set_variant, variants, budget_ms=25.0):
    """ms per launch of `launch` under the automatic choice and under every forced variant; a variant that takes more than
    eight times the automatic choice's time is timed on one launch only.  (Interleaved A/B runs of the automatic choice and
    the same variant forced agree to 0.1 %; in a sweep the order of the variants shows as a few percent on kernels of
    tens of microseconds, hence the three placements of the automatic choice.)"""
    def timed(n):
        capi.timer_start()
        for _ in range(n):
            launch()
        return capi.timer_stop() / n
    out = {}
    variants = list(variants)
    half = len(variants) // 2
    for v in [0] + variants[:half] + [0] + variants[half:] + [0]:      # the automatic choice three times: the best of them
        set_variant(v)
        launch()
        capi.sync()
        one = timed(1)
        if v != 0 and one > 8.0 * out[0]:
            out[v] = one
            continue
        n = max(3, min(200, int(budget_ms / max(one, 1e-3))))
        timed(n)                                        # the chip's clock settles over the first milliseconds
        if v == 0:
            timed(n)
        t = min(timed(n), timed(n))
        out[v] = min(t, out[v]) if v in out else t
    set_variant(0)
    return out


def bench_shape_sweep(capi, workloads):
    """The automatic kernel choice against every forced variant, shape by shape (the evidence behind the pickers of
    sgemm_launch.hpp, hgemm.hip and the convolution launchers)."""
    L = capi.lib()
    rows = []
    def padded(x, unit):                                # the pitch of a DECX container: 8 floats, 16 halves (Matrix.h:24-27)
        return (x + unit - 1) // unit * unit
    def row_of(what, auto_variant, t):
        best = min((v for v in t if v), key=lambda v: t[v])
        return {"what": what, "auto_variant": auto_variant, "auto_ms": round(t[0], 5), "best_variant": best, "best_ms": round(t[best], 5),
                "auto_over_best": round(t[0] / t[best], 4), "ms_by_variant": {str(v): round(ms, 5) for v, ms in t.items()}}
    for M, K, N in SWEEP_FP32:
        lda, ldb = padded(K, 8), padded(N, 8)
        A, B = np.zeros((M, lda), np.float32), np.zeros((K, ldb), np.float32)
        A[:, :K], B[:, :N] = workloads.uniform_pm1((M, K), 31), workloads.uniform_pm1((K, N), 32)
        dA, dB, dD = capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(B), capi.DeviceBuffer(M * ldb * 4)
        t = sweep_one(capi, lambda: capi.sgemm(dA.ptr, lda, dB.ptr, ldb, dD.ptr, ldb, M, N, K, blocking=False), L.decx_hip_set_sgemm_variant,
                      SWEEP_FP32_VARIANTS)
        rows.append(row_of("fp32 GEMM %dx%dx%d (MxKxN)" % (M, K, N), L.decx_hip_sgemm_plan(M, N, K, 1, lda, ldb, 1), t))
        for b in (dA, dB, dD):
            b.free()
    for H, W, C, N, k in SWEEP_CONV:
        src, filt = workloads.conv_case(H=H, W=W, C=C, N=N, kh=k, kw=k)
        kp = (k + 3) // 4 * 4
        fb = np.zeros((N, k, kp, C), np.float32); fb[:, :, :k, :] = filt
        dS, dF, dD = capi.DeviceBuffer.from_numpy(src), capi.DeviceBuffer.from_numpy(fb), capi.DeviceBuffer(H * W * N * 4)
        t = sweep_one(capi, lambda: capi.conv2_im2col(dS.ptr, H, W, C, W * C, dF.ptr, N, k, k, k * kp * C, kp * C, dD.ptr, N, W * N, 1, blocking=False),
                      L.decx_hip_set_sgemm_variant, SWEEP_CONV_VARIANTS)
        rows.append(row_of("fp32 conv %dx%dx%d under %d filters %dx%d" % (H, W, C, N, k, k), "auto", t))
        for b in (dS, dF, dD):
            b.free()
    for M, K, N in SWEEP_FP16:
        lda, ldb = padded(K, 16), padded(N, 16)
        A, B = np.zeros((M, lda), np.uint16), np.zeros((K, ldb), np.uint16)
        A[:, :K] = workloads.uniform_pm1((M, K), 33).astype(np.float16).view(np.uint16)
        B[:, :N] = workloads.uniform_pm1((K, N), 34).astype(np.float16).view(np.uint16)
        dA, dB, dD = capi.DeviceBuffer.from_numpy(A), capi.DeviceBuffer.from_numpy(B), capi.DeviceBuffer(M * ldb * 2)
        t = sweep_one(capi, lambda: capi.hgemm(dA.ptr, lda, dB.ptr, ldb, dD.ptr, ldb, M, N, K, blocking=False), L.decx_hip_set_hgemm_variant,
                      SWEEP_FP16_VARIANTS)
        rows.append(row_of("fp16 GEMM %dx%dx%d (MxKxN)" % (M, K, N), L.decx_hip_hgemm_plan(M, N, K, 1, lda, ldb, 1, None), t))
        for b in (dA, dB, dD):
            b.free()
    return rows


def cpp_api_blocking_calls():
    """The same two blocking calls made from C++ through the DECX-named API (tests/build/test_decx_api timing, built by
    backup_1_amd/host/Makefile): what a DECX program sees, without the ctypes call overhead of this script."""
    import re
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tests", "build", "test_decx_api")
    if not os.path.exists(exe):
        return None
    r = subprocess.run([exe, "timing"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    out = {}
    for line in r.stdout.splitlines():
        m = re.match(r"(.+?)\s+min\s+([0-9.]+) us\s+median\s+([0-9.]+) us", line)
        if m:
            out[m.group(1).strip()] = {"us_per_call_min": float(m.group(2)), "us_per_call_median": float(m.group(3))}
    return out or None


def cpu_baseline(workloads, A, B, rows):
    """The restated DECX_cpu thread-pool SGEMM (oracle/, kind "port") on the first `rows` rows of the headline A times
    the full B: B re-pack included, 12 tasks on a pool of min(hardware threads, 16) workers, as the reference sizes it."""
    import oracle
    N = B.shape[1]
    out = np.zeros((rows, N), np.float32)
    workers = oracle.pool_size(0)
    best = None
    for _ in range(2):
        t0 = time.perf_counter()
        oracle.decx_cpu_sgemm(A[:rows], B, out=out)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    flops = 2.0 * rows * N * A.shape[1]
    # configuration 1 of the baseline file: the same routine on the fp32 1024^3 problem (de::cpu::sgemm, sgemm.h:28-60)
    A1, B1 = workloads.uniform_pm1((1024, 1024), 1), workloads.uniform_pm1((1024, 1024), 2)
    out1 = np.zeros((1024, 1024), np.float32)
    best1 = None
    for _ in range(5):
        t0 = time.perf_counter()
        oracle.decx_cpu_sgemm(A1, B1, out=out1)
        dt = time.perf_counter() - t0
        best1 = dt if best1 is None else min(best1, dt)
    return {"value": flops / best / 1e12, "unit": "TFLOP/s", "cores": min(workers, 12), "kind": "port",
            "host_cores": os.cpu_count(), "pool_workers": workers, "tasks": 12,
            "fp32_1024_cube": {"gflops": round(2.0 * 1024 ** 3 / best1 / 1e9, 1), "ms": round(best1 * 1e3, 3),
                               "what": "config 1 (M=N=K=1024, uniform[-1,1]) through the same routine, best of 5"},
            "sample": "restated DECX_cpu thread-pool SGEMM (B re-pack + 32x16x64 AVX2 FMA blocks, 12 tasks = 3x4 grid on a pool "
                      "of %d workers, so at most 12 cores work at once; host reports %d logical CPUs; AVX2+FMA, g++ -O2) on rows "
                      "0..%d of the 8192^3 fp32 workload x full B, best of 2, %.2f s" % (workers, os.cpu_count() or 0, rows - 1, best)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=8192, help="square size of the headline fp32 GEMM")
    ap.add_argument("--sgemm-variant", type=int, default=0, help="force a fp32 tile shape (0 = automatic)")
    ap.add_argument("--hgemm-variant", type=int, default=0, help="force a fp16 tile shape (0 = automatic)")
    ap.add_argument("--no-verify", action="store_true", help="skip the post-run comparison of sampled rows with the oracle")
    ap.add_argument("--only", default="", help="comma list of: headline,fp16,sq4096,small,ragged,conv,relu,host,cpu (default all); extra: ladder, copy, sweep, twolaunch")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives, no sharding); --gpus %d is not supported. "
              "value is one GPU's throughput." % args.gpus, file=sys.stderr)
        sys.exit(2)
    only = set(filter(None, args.only.split(",")))
    want = lambda k: not only or k in only

    from backup_1_amd import capi, workloads
    capi.init()
    info = capi.device_info()
    capi.lib().decx_hip_set_sgemm_variant(args.sgemm_variant)
    capi.lib().decx_hip_set_hgemm_variant(args.hgemm_variant)
    log("device: %d CUs, %.0f MHz" % (info["compute_units"], info["clock_khz"] / 1e3))

    n = args.size
    log("headline: fp32 GEMM %d^3" % n)
    head = bench_sgemm(capi, workloads, n, n, n, args.steps, args.warmup, 1234, verify_rows=0 if args.no_verify else 16)
    log("  %.3f ms/step wall, %.3f ms/launch by HIP events -> %.1f TFLOP/s" % (head["ms_wall"], head["ms_kernel"], head["tflops"]))
    if "verified" in head:
        log("  %d sampled rows of the timed result bit-equal to the oracle's chain: %s" % (head["verified_rows"], head["verified"]))

    also = {}
    # the side workloads are sub-millisecond kernels launched after a host-side pause (data generation, uploads) in which
    # the chip clocks down: give them more launches, and a longer warm-up, than the headline needs
    side_steps = max(20, min(args.steps * 3, 60))
    side_warmup = max(args.warmup, 10)
    global SIDE_MIN_WARM_MS, SIDE_MIN_TIMED_MS
    SIDE_MIN_WARM_MS, SIDE_MIN_TIMED_MS = 60.0, 30.0
    also["side_timing"] = {"min_warmup_ms": SIDE_MIN_WARM_MS, "min_timed_ms": SIDE_MIN_TIMED_MS,
                           "what": "every workload under `also` is warmed up and timed over at least this many ms of back-to-back launches"}
    if want("fp16"):
        r = bench_hgemm(capi, workloads, 8192, side_steps, side_warmup, 5, verify_rows=0 if args.no_verify else 16)
        also["fp16_8192_f32acc"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                                    "frac_of_fp16_dense_peak": round(r["tflops_kernel"] / PEAK_FP16_MATRIX_TFLOPS, 4)}
        if "verified" in r:
            also["fp16_8192_f32acc"].update({"verified": r["verified"], "verified_rows": r["verified_rows"],
                                             "max_rel_err_vs_fp64": float("%.3e" % r["max_rel_err"]), "tolerance": 2e-3})
        log("fp16 8192^3: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
    if "ladder" in only:
        also["fp16_8192_ladder"] = bench_fp16_ladder(capi, workloads, side_steps, side_warmup)
        for row in also["fp16_8192_ladder"]:
            log("fp16 ladder, build %d, %-52s %7.1f TFLOP/s on uniform[-1,1], %7.1f on zeros" % (row["build"], row["what"], row["tflops_uniform"], row["tflops_zeros"]))
    if want("sq4096"):
        r = bench_sgemm(capi, workloads, 4096, 4096, 4096, side_steps, side_warmup, 1234)
        also["fp32_4096"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                             "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("fp32 4096^3: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
    if want("small"):
        # results too small to fill the chip with 256x256 tiles: 64x64 tiles fed by LDS-DMA loads (one per CU at
        # 1024 x 1024), the one-wave-per-16x16-block kernel for the thin long-K product below
        r = bench_sgemm(capi, workloads, 1024, 1024, 1024, side_steps, side_warmup, 77)
        also["fp32_1024"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                             "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("fp32 1024^3: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        r = bench_sgemm(capi, workloads, 1024, 8192, 1024, side_steps, side_warmup, 76)
        also["fp32_1024x8192x1024"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                                       "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("fp32 1024x8192x1024: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        r = bench_sgemm(capi, workloads, 64, 65536, 1024, side_steps, side_warmup, 78)
        # one fused chain per output cannot be split over K: the bound is 8 cycles per k of a single MFMA chain
        chain_ms = 65536 / 4 * 32 / (info["clock_khz"] * 1e3) * 1e3
        also["fp32_long_k_64x65536x1024_exact_chain"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                                                          "ms_of_one_bare_mfma_chain": round(chain_ms, 4)}
        log("fp32 64x65536x1024 (exact chain): %.4f ms -> %.1f TFLOP/s (a bare MFMA chain over K: %.4f ms)"
            % (r["ms_wall"], r["tflops"], chain_ms))
        r = bench_hgemm(capi, workloads, 0, side_steps, side_warmup, 79, shape=(64, 65536, 1024))
        also["fp16_long_k_64x65536x1024_split_k"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4)}
        log("fp16 64x65536x1024 (split-K, fp32 workspace): %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        # GEMM3's kernel step: 16 products of 1024^3 in one launch (256 tiles of 256 x 256 where one product has 16)
        also["fp32_batched_16x1024_one_launch_blocking_call"] = bench_batched(capi, workloads, False, 16, 1024)
        also["fp16_batched_16x1024_one_launch_blocking_call"] = bench_batched(capi, workloads, True, 16, 1024)
        log("16 x 1024^3 in one launch: fp32 %.1f TFLOP/s, fp16 %.1f TFLOP/s" %
            (also["fp32_batched_16x1024_one_launch_blocking_call"]["tflops"], also["fp16_batched_16x1024_one_launch_blocking_call"]["tflops"]))
    if want("ragged"):
        r = bench_sgemm(capi, workloads, 3000, 1500, 4500, side_steps, side_warmup, 4321, dist="normal")
        also["fp32_ragged_3000x1500x4500"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                                              "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("fp32 ragged: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        # a size that is no multiple of any tile: 289 tiles of 256x256 run as one round + 512 rows on smaller tiles
        # (decx_hip_sgemm_plan_split); the same product kept in one launch beside it (variants 34 / 20)
        L = capi.lib()
        rows = 0 if args.no_verify else 8
        r = bench_sgemm(capi, workloads, 4352, 4096, 4352, side_steps, side_warmup, 4400, verify_rows=rows)
        prev = L.decx_hip_set_sgemm_variant(34)
        one = bench_sgemm(capi, workloads, 4352, 4096, 4352, side_steps, side_warmup, 4400)
        L.decx_hip_set_sgemm_variant(prev)
        also["fp32_4352x4096x4352_two_launches"] = {"tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
                                                    "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4),
                                                    "verified": r.get("verified"), "verified_rows": r.get("verified_rows", 0),
                                                    "one_launch_tflops": round(one["tflops"], 2), "one_launch_ms": round(one["ms_wall"], 4)}
        h = bench_hgemm(capi, workloads, 0, side_steps, side_warmup, 4410, shape=(4352, 4096, 4352), verify_rows=rows)
        prev = L.decx_hip_set_hgemm_variant(20)
        hone = bench_hgemm(capi, workloads, 0, side_steps, side_warmup, 4410, shape=(4352, 4096, 4352))
        L.decx_hip_set_hgemm_variant(prev)
        also["fp16_4352x4096x4352_two_launches"] = {"tflops": round(h["tflops"], 2), "ms_per_step": round(h["ms_wall"], 4),
                                                    "verified": h.get("verified"), "max_rel_err": h.get("max_rel_err"),
                                                    "one_launch_tflops": round(hone["tflops"], 2), "one_launch_ms": round(hone["ms_wall"], 4)}
        log("4352x4096x4352 in two launches: fp32 %.1f TFLOP/s (one launch %.1f), fp16 %.1f (one launch %.1f)"
            % (r["tflops"], one["tflops"], h["tflops"], hone["tflops"]))
    if want("conv"):
        r = bench_conv(capi, workloads, side_steps, side_warmup)
        also["fp32_conv_224x224x64_128f3x3_fused_im2col"] = {
            "tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
            "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("conv: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))

    if want("conv"):
        r = bench_hconv(capi, workloads, side_steps, side_warmup)
        also["fp16_conv_224x224x64_128f3x3_f32acc_fused_im2col"] = {
            "tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
            "frac_of_fp16_dense_peak": round(r["tflops_kernel"] / PEAK_FP16_MATRIX_TFLOPS, 4)}
        log("fp16 conv: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        # config 4 is 15 - 75 us of work, a good part of it launch, first loads and the write of the result; the same
        # kernels on an image that fills the chip for several rounds of tiles show what their K loops sustain
        big = dict(H=512, W=512, C=256, N=256)
        r = bench_conv(capi, workloads, side_steps, side_warmup, **big)
        also["fp32_conv_512x512x256_256f3x3_fused_im2col"] = {
            "tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
            "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("conv 512x512x256 -> 256: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        # and a CNN layer on a small image (the use the reference names this convolution for): few outputs, long K
        small = dict(H=56, W=56, C=256, N=256)
        r = bench_conv(capi, workloads, side_steps, side_warmup, **small)
        also["fp32_conv_56x56x256_256f3x3_fused_im2col"] = {
            "tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
            "frac_of_fp32_matrix_peak": round(r["tflops_kernel"] / PEAK_FP32_MATRIX_TFLOPS, 4)}
        log("conv 56x56x256 -> 256: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        r = bench_hconv(capi, workloads, side_steps, side_warmup, **small)
        also["fp16_conv_56x56x256_256f3x3_f32acc_fused_im2col"] = {
            "tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
            "frac_of_fp16_dense_peak": round(r["tflops_kernel"] / PEAK_FP16_MATRIX_TFLOPS, 4)}
        log("fp16 conv 56x56x256 -> 256: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        r = bench_hconv(capi, workloads, side_steps, side_warmup, **big)
        also["fp16_conv_512x512x256_256f3x3_f32acc_fused_im2col"] = {
            "tflops": round(r["tflops"], 2), "ms_per_step": round(r["ms_wall"], 4),
            "frac_of_fp16_dense_peak": round(r["tflops_kernel"] / PEAK_FP16_MATRIX_TFLOPS, 4)}
        log("fp16 conv 512x512x256 -> 256: %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))

    if want("relu"):
        r = bench_relu(capi, workloads, side_steps, side_warmup)
        also["relu_f32_8192x8192"] = {"GBps": round(r["gbps"], 1), "ms_per_step": round(r["ms_wall"], 4),
                                      "frac_of_hbm_peak": round(r["gbps"] / PEAK_HBM_GBPS, 4)}
        log("relu 8192x8192: %.4f ms -> %.0f GB/s" % (r["ms_wall"], r["gbps"]))
        r = bench_conv_fused(capi, workloads, side_steps, side_warmup)
        also["fp32_conv_bias_relu_fused_blocking_call"] = {"tflops": round(r["tflops"], 2), "ms_per_call": round(r["ms_wall"], 4),
                                                           "ms_per_call_median": round(r["ms_median"], 4)}
        log("conv + bias + relu (one kernel, blocking call): %.4f ms -> %.1f TFLOP/s" % (r["ms_wall"], r["tflops"]))
        also.update(bench_blocking_calls(capi, workloads, side_steps, side_warmup))
        cpp = cpp_api_blocking_calls()
        if cpp:
            also["cpp_api_blocking_calls"] = cpp
            for what, v in cpp.items():
                log("C++ API, blocking %s: %.1f us per call (median %.1f)" % (what, v["us_per_call_min"], v["us_per_call_median"]))
        log("fp32 1024^3 blocking call: %.4f ms (enqueued: %.4f ms per launch); floor of a blocking call: %.4f ms"
            % (also["fp32_1024_blocking_call"]["ms_per_call_min"], also["fp32_1024_blocking_call"]["ms_per_launch_enqueued"],
               also["blocking_call_floor_relu_64_floats"]["ms_per_call_min"]))

    if "sweep" in only:
        also["shape_choice_sweep"] = bench_shape_sweep(capi, workloads)
        for row in also["shape_choice_sweep"]:
            log("sweep, %-46s auto %-4s %9.5f ms | best forced %-3s %9.5f ms | auto / best %.3f"
                % (row["what"], row["auto_variant"], row["auto_ms"], row["best_variant"], row["best_ms"], row["auto_over_best"]))
    if "twolaunch" in only:
        also["two_launch_ab"] = bench_two_launch_ab(capi)
        for row in also["two_launch_ab"]:
            log("two launches, %-34s first %-26s %9.4f ms (%6.1f TFLOP/s) | one launch %9.4f ms (%6.1f) | ratio %.3f%s"
                % (row["what"], row["first_launch"], row["two_launches_ms"], row["tflops"], row["one_launch_ms"], row["one_launch_tflops"],
                   row["ratio"], "" if row["results_agree"] else "  RESULTS DIFFER"))
    if "copy" in only:
        # calibration launch for the traffic counters: 1 GiB read + 1 GiB written by a plain copy kernel
        nbytes = 1 << 30
        src, dst = capi.DeviceBuffer(nbytes), capi.DeviceBuffer(nbytes)
        src.fill(1)
        for _ in range(3):
            rc = capi.probe_lib().decx_probe_copy(capi.stream(), dst.ptr, src.ptr, nbytes)
            if rc != 0:
                raise RuntimeError("decx_probe_copy returned %d" % rc)
        also["copy_1GiB"] = {"bytes_read": nbytes, "bytes_written": nbytes}

    if want("host"):
        r = bench_host_resident_gemm(capi, head["A"], head["B"], 2)
        also["host_resident_gemm_%d_pcie_inclusive" % n] = {"tflops": round(r["tflops"], 2), "ms_per_call": round(r["ms"], 2),
                                                            "pcie_bytes": r["pcie_bytes"]}
        log("host-resident GEMM %d^3 (H2D + kernel + D2H): %.1f ms -> %.1f TFLOP/s" % (n, r["ms"], r["tflops"]))
        r = bench_host_resident_gemm3(capi, workloads, 8, 2048, 3)
        also["host_resident_gemm3_8x2048_pcie_inclusive"] = {"tflops": round(r["tflops"], 2), "ms_per_call": round(r["ms"], 2),
                                                              "pcie_bytes": r["pcie_bytes"]}
        log("host-resident GEMM3, 8 x 2048^3 (H2D + kernels + D2H): %.2f ms -> %.1f TFLOP/s" % (r["ms"], r["tflops"]))
        r = bench_host_resident_conv(capi, workloads, 5)
        also["host_resident_conv_pcie_inclusive"] = {"tflops": round(r["tflops"], 2), "ms_per_call": round(r["ms"], 3)}
        log("host-resident conv (H2D + kernel + D2H): %.3f ms -> %.1f TFLOP/s" % (r["ms"], r["tflops"]))

    cpu = None
    if want("cpu"):
        also["cpu_conv_baseline"] = cpu_conv_baseline(workloads)
        log("cpu conv baseline: %.1f ms" % also["cpu_conv_baseline"]["ms"])
        log("cpu baseline (oracle port of the DECX_cpu thread-pool SGEMM) ...")
        cpu = cpu_baseline(workloads, head["A"], head["B"], rows=min(n, 3072))
        log("  %.4f TFLOP/s on %d cores" % (cpu["value"], cpu["cores"]))

    achieved = head["tflops_kernel"]
    traffic, traffic_source = measured_traffic(n, args.sgemm_variant)
    line = {
        # the metric's name as the baseline file spells it; `value` is its first component (fp32 8192^3), the fraction of
        # peak is roofline.frac, and the fp16 and conv components are under `also`
        "metric": "GEMM TFLOP/s at 8192\u00b3 fp32 & fp16 + % of MI355X matrix peak; conv TFLOP/s",
        "metric_note": "value = fp32 8192^3 GEMM; % of peak = roofline.frac; fp16 8192^3 and conv under also",
        "value": round(head["tflops"], 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_wall"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fp32 square GEMM C=A*B, M=N=K=%d, row-major, uniform[-1,1] seed 1234, device-resident "
                               "operands (GPU_Matrix path)" % n},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_FP32_MATRIX_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MATRIX_TFLOPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": HEADLINE_KERNELS.get(args.sgemm_variant, "fp32 tile shape %d" % args.sgemm_variant), "flop_per_launch": head["flops"],
                     "avg_launch_ms_hip_events": round(head["ms_kernel"], 4),
                     "single_launch_ms_median": round(head["ms_median"], 4), "single_launch_ms_min": round(head["ms_min"], 4)},
        "verified": head.get("verified"),
        "verified_how": ("%d sampled rows of the result of the timed launches, bit-compared with the CPU oracle's fused chain "
                         "after the timed region" % head["verified_rows"]) if "verified" in head else "skipped (--no-verify)",
        "cpu_baseline": cpu,
        "also": also,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
