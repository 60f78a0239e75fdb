/*
 * msco_moe.h -- C ABI of the MI355X (gfx950) backend for the two operators on either side of the
 * grouped matmul in an MoE layer: the routing step that sorts (token, k) rows by expert and gathers
 * their activations, and the weighted un-permutation of the expert outputs.
 *
 *   reference kernel object (what the op glue calls)                               this ABI
 *   ----------------------------------------------------------------------------  -----------------------------
 *   internal_v2::CreateMoeInitRoutingOp(inputs, outputs, MoeInitRoutingParam)      msco_moe_init_routing_v2
 *     ops/c_api/moe_init_routing_v2/moe_init_routing_v2.cc:132-147,179-182           (+ _workspace_bytes)
 *   (none: fusion of the routing step with the activation quantisation)            msco_moe_init_routing_v2_quant
 *   internal_v2::CreateMoeTokenUnpermuteOp(inputs, outputs)                        msco_moe_token_unpermute
 *     ops/c_api/moe_token_unpermute/moe_token_unpermute.cc:93-99,118-121
 *
 * Conventions are those of msco_gmm.h: int status (0 = MSCO_OK), raw device pointers to contiguous
 * row-major buffers owned by the caller, the workspace is the caller's, nothing allocates or
 * synchronises, everything is enqueued on the given hipStream_t.
 */
#ifndef MSCO_MOE_H_
#define MSCO_MOE_H_

#include <stddef.h>
#include <stdint.h>

#include "msco_gmm.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Bytes of workspace msco_moe_init_routing_v2 needs for num_rows tokens routed to k experts each. */
MSCO_API size_t msco_moe_init_routing_v2_workspace_bytes(int64_t num_rows, int64_t k, int64_t expert_num);

/* Dropless MoE routing (the only mode the reference op accepts: active_num = 0, expert_capacity = 0,
 * drop_pad_mode = 0, moe_init_routing_v2.cc:107-109).  With n = num_rows * k flat (token, k) entries:
 *   sorted = stable argsort of expert_idx.flatten()                       (golden: tests/st/
 *   expanded_row_idx[sorted[j]] = j                                        test_custom_moe_init_routing_v2.py:38,59-60)
 *   expanded_x[j, :] = x[sorted[j] / k, :]                                 (:65)
 *   expert_tokens_count_or_cumsum = cumulative (flag 1) or per-expert (flag 2) entry counts   (:47-57)
 * x [num_rows, hidden] of elem_bytes-wide elements (1, 2 or 4; hidden * elem_bytes a multiple of 16);
 * expert_idx int32 [num_rows, k] with values in [0, expert_num) (others are clamped into the range);
 * expanded_x [n, hidden]; expanded_row_idx int32 [n]; expert_tokens_count_or_cumsum int32 [expert_num]
 * (untouched when flag = 0, may then be NULL); expert_tokens_before_capacity int32 [expert_num] is an
 * output of the drop/pad mode only and is zero-filled (may be NULL).  expert_num <= 1024. */
MSCO_API int msco_moe_init_routing_v2(const void *x, const int32_t *expert_idx, void *expanded_x,
                                      int32_t *expanded_row_idx, int32_t *expert_tokens_count_or_cumsum,
                                      int32_t *expert_tokens_before_capacity, void *workspace, size_t workspace_bytes,
                                      int64_t num_rows, int64_t hidden, int64_t k, int64_t expert_num,
                                      int32_t elem_bytes, int32_t count_or_cumsum_flag, void *stream);

/* The same routing with the activations quantised on the way: what an int8 grouped matmul behind the routing step
 * consumes.  No operator of the reference does this in one step; the arithmetic is the per-token dynamic quantisation
 * that the reference's test applies to the activations in front of its int8-activation grouped matmul
 * (dyn_quant, tests/st/test_grouped_matmul_w4.py:83-89), row by row, with t = sorted[j] / k:
 *   expanded_scale[j] = float32(max_h |x[t, h]|) / 127
 *   expanded_x[j, h]  = int8(rint(float32(x[t, h]) / expanded_scale[j]))          (rint: half to even, as np.round)
 * x [num_rows, hidden] in x_dtype (MSCO_DT_F16 or MSCO_DT_BF16), hidden a multiple of 8; expanded_x int8 [n, hidden];
 * expanded_scale float32 [n] (the grouped matmul's per_token_scale).  A row of zeros gets scale 0 and zeros (the
 * golden divides 0 by 0 there).  Everything else as in msco_moe_init_routing_v2, same workspace. */
MSCO_API int msco_moe_init_routing_v2_quant(const void *x, const int32_t *expert_idx, int8_t *expanded_x,
                                            float *expanded_scale, int32_t *expanded_row_idx,
                                            int32_t *expert_tokens_count_or_cumsum, int32_t *expert_tokens_before_capacity,
                                            void *workspace, size_t workspace_bytes, int64_t num_rows, int64_t hidden,
                                            int64_t k, int64_t expert_num, int32_t x_dtype, int32_t count_or_cumsum_flag,
                                            void *stream);

/* Weighted un-permutation: out[i, :] = sum_k probs[i, k] * permuted_tokens[sorted_indices[i * top_k + k], :],
 * accumulated in the element type exactly as the golden does (tests/st/test_custom_moe_token_unpermute.py:37-47:
 * every product and every running sum is rounded to the element type; both go through float32, as numpy's
 * half arithmetic does).  permuted_tokens [num_tokens * top_k, hidden], probs [num_tokens, top_k] and
 * out [num_tokens, hidden] in dtype (MSCO_DT_F16 as in the reference, or MSCO_DT_BF16); sorted_indices int32
 * [num_tokens * top_k]; hidden a multiple of 8; top_k <= 64. */
MSCO_API int msco_moe_token_unpermute(const void *permuted_tokens, const int32_t *sorted_indices, const void *probs,
                                      void *out, int64_t num_tokens, int64_t top_k, int64_t hidden, int32_t dtype,
                                      void *stream);

#ifdef __cplusplus
}
#endif
#endif  /* MSCO_MOE_H_ */
