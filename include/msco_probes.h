/* Measurement aids of the grouped-matmul backend -- a library of their own (libmsco_probes.so), so that the operator
 * library exports nothing but operators.  Neither has a counterpart in the reference; the benchmark quotes them next to
 * the kernels' rates.  Status codes are those of msco_gmm.h. */
#ifndef MSCO_PROBES_H_
#define MSCO_PROBES_H_

#include <stddef.h>
#include <stdint.h>

#include "msco_gmm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid with no counterpart in the reference: the rate the matrix pipe sustains on a given operand
 * distribution, the yardstick the benchmark quotes next to the grouped matmul's rate, and what a wavefront that is alone
 * on its SIMD can issue between MFMAs.  MSCO_PROBE_MFMA_WORKGROUPS workgroups of 256 threads run `iters` (a multiple of 8) rounds of 64
 * v_mfma_i32_16x16x64_i8 (patterns 0 - 11) or 32 v_mfma_i32_32x32x32_i8 (12 - 14) -- 2^21 int8 operations per wavefront
 * and round either way, MSCO_PROBE_MFMA_WORKGROUPS * 4 * iters * 2^21 per launch -- on operand fragments read once from
 * `operands` (MSCO_PROBE_MFMA_OPERAND_BYTES bytes of int8; every workgroup reads the same), with memory operations woven
 * in, each behind an MFMA ("slot" n = 0..63 of the round), and never wait for a result:
 *    0  MFMAs only                                   12  32 x 32 x 32: MFMAs only
 *    1  16 ds_read_b128 (slots n % 4 == 1)
 *    2  pattern 1 + 8 buffer_load_dwordx4 (n % 8 == 3)
 *    3  8 ds_write_b128 alone (n % 8 == 0)            4  16 ds_write_b64 alone (n % 4 == 0)     5  32 ds_write_b32 alone
 *    6  pattern 2 + 8 ds_write_b128 at n % 8 == 0 (a read follows one MFMA later)      13  the same on 32 x 32 x 32
 *    7  pattern 2 + 8 ds_write_b128 at n % 8 == 2 (behind a read; the next read three MFMAs later)
 *    8  pattern 2 + 16 ds_write_b64 at n % 4 == 0 (slots of their own)       14  on 32 x 32 x 32, writes at n % 4 == 2
 *    9  pattern 2 + 16 ds_write_b64 at n % 4 == 1 (sharing the reads' slots)
 *   10  pattern 8 with the loads at n % 8 == 0 (sharing a write's slot)
 *   11  pattern 2 + 32 ds_write_b32 (n % 2 == 0)
 * Patterns 6 - 11, 13, 14 carry the traffic of the persistent tile kernels' K loop.  LDS reads find zeros, buffer loads
 * re-read `operands`.  `clocks` receives two int64: core clocks and 100 MHz ticks that workgroup 0 spent in the loop.  `sink` receives
 * MSCO_PROBE_MFMA_WORKGROUPS * 256 int32 values: each thread's sum over its accumulators.  Enqueues on the stream,
 * allocates nothing. */
#define MSCO_PROBE_MFMA_WORKGROUPS 256
#define MSCO_PROBE_MFMA_OPERAND_BYTES (8 * 256 * 16)
MSCO_API int msco_probe_mfma_issue(const void *operands, void *sink, void *clocks, int32_t pattern, int32_t iters, void *stream);

/* Measurement aid with no counterpart in the reference: one launch that only reads `bytes` bytes (rounded down to a
 * multiple of 4096) front to back with `workgroups` workgroups of 256 threads, each taking one contiguous share in the
 * access pattern of the packed-layout decode kernels.  Its duration is the floor under any single-launch decode kernel
 * whose weights have that size.  `sink` receives workgroups * 256 int32 values of no meaning. */
MSCO_API int msco_probe_read(const void *src, size_t bytes, void *sink, int32_t workgroups, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* MSCO_PROBES_H_ */
