/*
 * Measurement instruments for libdecx_hip.so, built into a library of their own (libdecx_hip_probe.so, `make probes`):
 * nothing here is part of the product's ABI, nothing in the product loads it.  bench.py loads it for its `ladder` and
 * `copy` legs only.  None of these entry points has a counterpart in the reference.
 *
 * Every launch goes to the stream passed in (a hipStream_t; decx_hip_stream() returns the product library's) and does
 * not wait, except decx_probe_copy.  Return value: 0, or 1000 + hipError_t, or 0x0d for arguments the probe refuses.
 */
#ifndef DECX_HIP_PROBE_H_
#define DECX_HIP_PROBE_H_
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* The large fp16 GEMM tile kernel of decx_hip_hgemm_f32acc (hgemm_mfma16_kernel) in one of its builds, with parts of
 * its K walk left out, so that the cost of each part can be read off as the difference between two variants.
 *   kind  : 0 = 2 LDS stages of 64 k, one tile per workgroup (the product's build for ragged and batched products)
 *           1 = 4 stages of 32 k          2 = 5 stages of 32 k
 *           3 = kind 0 as one workgroup per compute unit that walks its tiles as one stream of K steps (the product's
 *               opt-in build for large products of whole tiles, variant 17)          4 = kind 1 in that form
 *           5 = kind 0 on 4 waves of 128 x 128 (one per SIMD, a third fewer LDS fragment reads)          6 = kind 1 on those waves
 *   ablate: a sum of 1 = no global -> LDS loads inside the K walk, 2 = no LDS -> register reads inside it (the matrix
 *           instructions keep running on the first fragments), 4 = the result is not stored, 8 = the loads never move on
 *           (they fetch the tile's first K step over and over: loads that hit the caches), 16 / 32 = the matrix
 *           instructions of a unit row block by row block with ascending columns / column block by column block,
 *           instead of the product's order (columns reversed on every other row block).  Built: 0, 4, 5, 7, 12, and
 *           16, 32, 23, 39 for kind 0.  Every variant issues the same matrix instructions; all but 0, 16, 32 leave D
 *           meaningless or untouched.
 *   group_m: tile rows per raster group of the XCD-aware tile walk (the product uses 8).
 *   grid   : kinds 3, 4: number of workgroups (<= 0: one per compute unit of the current device).
 * M, N multiples of 256 and K a multiple of 128, A and B 16-byte aligned with lda, ldb multiples of 8. */
int decx_probe_hgemm(int kind, int ablate, void* stream, const uint16_t* A, int lda, const uint16_t* B, int ldb, uint16_t* D,
                     int ldd, int M, int N, int K, int group_m, int grid);

/* A plain device-to-device streaming copy kernel of `bytes` bytes (16-byte aligned, multiple of 16): hardware traffic
 * counters read for the product's kernels are scaled by what the same counters read for this kernel, whose traffic is
 * known exactly.  Blocks until complete. */
int decx_probe_copy(void* stream, void* dst, const void* src, size_t bytes);

#ifdef __cplusplus
}
#endif
#endif
