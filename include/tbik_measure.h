/*
 * libtbik_measure.so -- machine probes of the benchmark.  NOT part of the drop-in boundary (include/tbik_hip.h is):
 * nothing here has a counterpart in the reference and no product code calls it; bench.py loads the library for its ceiling figures
 * to read a roofline fraction against a ceiling measured on the box as well as against the published peak.
 * Return values are those of tbik_hip.h (0 = ok).
 *
 *   tbik_probe_mfma_bf16: `work_groups` work-groups (one per CU: each requests 100 KiB of LDS) of `waves` (4 or 8)
 *     wavefronts run |iters| x 16 v_mfma_f32_16x16x32_bf16 each on register operands taken once from `operands`
 *     (65,536 bytes of bf16, 16-byte aligned); `out` receives work_groups * waves * 64 floats.  Work done:
 *     work_groups * waves * |iters| * 16 instructions of 16,384 flop.  iters > 0: the 4 x 4 tiles of a wave row by row;
 *     iters < 0: rows in alternating directions (every MFMA changes one operand), as the tree GEMM issues them.
 *   tbik_probe_read: one grid-stride pass of 16-byte loads over `bytes` of `src` by `work_groups` work-groups of
 *     256 threads; `out` receives work_groups * 256 32-bit words.
 */
#ifndef TBIK_MEASURE_H
#define TBIK_MEASURE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif
int tbik_probe_mfma_bf16(const void* operands, void* out, int work_groups, int waves, int iters, void* stream);
int tbik_probe_read(const void* src, int64_t bytes, void* out, int work_groups, void* stream);
#ifdef __cplusplus
}
#endif
#endif /* TBIK_MEASURE_H */
