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
 * distribution with no memory traffic, the yardstick the benchmark quotes next to the grouped matmul's rate.
 * MSCO_PROBE_MFMA_WORKGROUPS workgroups of 256 threads each run `iters` rounds of the 16 v_mfma_i32_32x32x32_i8 of a
 * 128 x 128 wave tile, i.e. MSCO_PROBE_MFMA_WORKGROUPS * 4 * iters * 16 * 65536 int8 operations per launch, on operand
 * fragments read once from `operands` (MSCO_PROBE_MFMA_OPERAND_BYTES bytes of int8; every workgroup reads the same).
 * `sink` receives MSCO_PROBE_MFMA_WORKGROUPS * 256 int32 values of no meaning.  Enqueues on the stream, allocates nothing. */
#define MSCO_PROBE_MFMA_WORKGROUPS 256
#define MSCO_PROBE_MFMA_OPERAND_BYTES (8 * 256 * 16)
MSCO_API int msco_probe_mfma(const void *operands, void *sink, int32_t iters, void *stream);

/* Measurement aid with no counterpart in the reference: one launch that only reads `bytes` bytes (rounded down to a
 * multiple of 4096) front to back with `workgroups` workgroups of 256 threads, each taking one contiguous share in the
 * access pattern of the packed-layout decode kernels.  Its duration is the floor under any single-launch decode kernel
 * whose weights have that size.  `sink` receives workgroups * 256 int32 values of no meaning. */
MSCO_API int msco_probe_read(const void *src, size_t bytes, void *sink, int32_t workgroups, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* MSCO_PROBES_H_ */
