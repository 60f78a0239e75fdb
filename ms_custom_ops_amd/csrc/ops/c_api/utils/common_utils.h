// Shape helpers shared by the matmul-family operators (reference: ops/c_api/utils/common_utils.cc:79-138).
#ifndef MS_CUSTOM_OPS_C_API_UTILS_COMMON_UTILS_H_
#define MS_CUSTOM_OPS_C_API_UTILS_COMMON_UTILS_H_

#include <string>

#include "ops/framework/utils.h"

namespace ms_custom_ops {
struct BatchMatMulDims {
  ShapeVector batch;     // broadcast batch dims of the output
  ShapeVector x1_batch;  // x1's own batch dims, left-padded with 1 to batch.size()
  ShapeVector x2_batch;
  int64_t m{0}, k{0}, n{0};
};

// Splits x1 [..., M, K] (or [..., K, M]) and x2 [..., K, N] (or [..., N, K]) into broadcast batch dims
// and the matrix dims; raises on rank < 2, incompatible batch dims or mismatching K.
BatchMatMulDims BatchMatMulSplitDims(const ShapeVector &x1_shape, const ShapeVector &x2_shape, bool transpose_a,
                                     bool transpose_b, const std::string &op_name);

// Output shape [..., M, N].
ShapeVector BatchMatMulMakeShape(const ShapeVector &x1_shape, const ShapeVector &x2_shape, bool transpose_a,
                                 bool transpose_b, size_t offset, const std::string &op_name);
}  // namespace ms_custom_ops
#endif  // MS_CUSTOM_OPS_C_API_UTILS_COMMON_UTILS_H_
