#include "ops/c_api/utils/common_utils.h"

#include <algorithm>

namespace ms_custom_ops {
BatchMatMulDims BatchMatMulSplitDims(const ShapeVector &x1_shape, const ShapeVector &x2_shape, bool transpose_a,
                                     bool transpose_b, const std::string &op_name) {
  constexpr size_t kMatSize = 2;
  if (x1_shape.size() < kMatSize || x2_shape.size() < kMatSize) {
    MS_LOG_EXCEPTION << "For '" << op_name << "', the dimension of 'x1' and 'x2' should be at least 2, "
                     << "but got " << x1_shape.size() << " and " << x2_shape.size();
  }
  BatchMatMulDims d;
  const size_t b1 = x1_shape.size() - kMatSize, b2 = x2_shape.size() - kMatSize;
  const size_t nb = std::max(b1, b2);
  d.x1_batch.assign(nb, 1);
  d.x2_batch.assign(nb, 1);
  std::copy(x1_shape.begin(), x1_shape.begin() + b1, d.x1_batch.begin() + (nb - b1));
  std::copy(x2_shape.begin(), x2_shape.begin() + b2, d.x2_batch.begin() + (nb - b2));
  for (size_t i = 0; i < nb; ++i) {
    const int64_t a = d.x1_batch[i], b = d.x2_batch[i];
    if (a != b && a != 1 && b != 1) {
      MS_LOG_EXCEPTION << "For '" << op_name << "', batch dimensions must be equal or one of them must be 1, "
                       << "but got " << a << " and " << b;
    }
    d.batch.push_back(a == 1 ? b : a);
  }
  d.m = transpose_a ? x1_shape[b1 + 1] : x1_shape[b1];
  d.k = transpose_a ? x1_shape[b1] : x1_shape[b1 + 1];
  const int64_t k2 = transpose_b ? x2_shape[b2 + 1] : x2_shape[b2];
  d.n = transpose_b ? x2_shape[b2] : x2_shape[b2 + 1];
  if (d.k != k2) {
    MS_LOG_EXCEPTION << "For '" << op_name << "', the K dimension of 'x1' and 'x2' must be equal, "
                     << "but got " << d.k << " and " << k2;
  }
  return d;
}

ShapeVector BatchMatMulMakeShape(const ShapeVector &x1_shape, const ShapeVector &x2_shape, bool transpose_a,
                                 bool transpose_b, size_t /*offset*/, const std::string &op_name) {
  const BatchMatMulDims d = BatchMatMulSplitDims(x1_shape, x2_shape, transpose_a, transpose_b, op_name);
  ShapeVector out = d.batch;
  out.push_back(d.m);
  out.push_back(d.n);
  return out;
}
}  // namespace ms_custom_ops
