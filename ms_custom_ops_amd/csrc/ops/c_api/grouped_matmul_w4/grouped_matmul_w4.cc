// grouped_matmul_w4(x, weight, group_list, bias, x_scale, weight_scale) -> out
//
// Grouped matmul of int8 activations with int4 weights that carry one float32 scale per (expert, K group, column).
// Interface, shape and type rules and messages follow the reference (ops/c_api/grouped_matmul_w4/
// grouped_matmul_w4.cc:50-88 shapes, :120-152 types, :254-255 the Python signature): x int8 [m, k]; weight two 4-bit
// values per byte [e, n, k / 2]; group_list int32 [e]; bias, x_scale, weight_scale float32; out float16 [m, n].  The
// tensor library here has no 4-bit type, so the packed weight arrives as an int8 or uint8 tensor.  The reference
// creates a closed kernel object that multiplies the nibbles unsigned and adds `bias` = 8 * sum_k dequantised
// weight to compensate (:183-186, test_grouped_matmul_w4.py:103-106); the backend behind msco_gmm_a8w4 multiplies
// signed nibbles, so `bias` is type- and shape-checked and not read.
#include <string>
#include <vector>

#include "msco_gmm.h"
#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
static ShapeVector InferGroupedMatmulW4OutputShape(const ShapeVector &x_shape, const ShapeVector &weight_shape,
                                                   const ShapeVector &group_list_shape) {
  if (x_shape.size() != kDim2) MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'x' must be 2D, but got:" << x_shape.size();
  if (weight_shape.size() != kDim3) {
    MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'weight' must be 3D, but got:" << weight_shape.size();
  }
  if (group_list_shape.size() != kDim1) {
    MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'group_list' must be 1D, but got:" << group_list_shape.size();
  }
  const int64_t weight_real_k_dim = weight_shape[kIndex2] << 1;   // stored as [e, n, k / 2]
  if (x_shape[kIndex1] != weight_real_k_dim) {
    MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'x' and 'weight' must have the same dimension of 'k', but got:"
                     << x_shape[kIndex1] << " and " << weight_real_k_dim;
  }
  return ShapeVector{x_shape[kIndex0], weight_shape[kIndex1]};
}

static void CheckGroupedMatmulW4Types(TypeId x, TypeId weight, TypeId group_list, TypeId bias, TypeId x_scale, TypeId weight_scale) {
  if (x != kNumberTypeInt8) MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'x' must be int8, but got:" << x;
  if (weight != kNumberTypeInt8 && weight != kNumberTypeUInt8 && weight != kNumberTypeInt4) {
    MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'weight' must be qint4x2, but got:" << weight;
  }
  if (group_list != kNumberTypeInt32) MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'group_list' must be int32, but got:" << group_list;
  if (bias != kNumberTypeFloat32) MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'bias' must be float32, but got:" << bias;
  if (x_scale != kNumberTypeFloat32) MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'x_scale' must be float32, but got:" << x_scale;
  if (weight_scale != kNumberTypeFloat32) {
    MS_LOG_EXCEPTION << "For GroupedMatmulW4, input 'weight_scale' must be float32, but got:" << weight_scale;
  }
}

static void RunGroupedMatmulW4(const ms::Tensor &x, const ms::Tensor &weight, const ms::Tensor &group_list, const ms::Tensor &bias,
                               const ms::Tensor &x_scale, const ms::Tensor &weight_scale, const ms::Tensor &out) {
  const std::string op_name = "GroupedMatmulW4";
  CheckGroupedMatmulW4Types(x.data_type(), weight.data_type(), group_list.data_type(), bias.data_type(), x_scale.data_type(),
                            weight_scale.data_type());
  CheckContiguous(op_name, {x, weight, group_list, bias, x_scale, weight_scale}, true);
  CheckContiguous(op_name, {out}, false);
  const int64_t m = x.shape()[kIndex0], k = x.shape()[kIndex1], e = weight.shape()[kIndex0], n = weight.shape()[kIndex1];
  if (group_list.shape()[kIndex0] != e) {
    MS_EXCEPTION_VALUE << "For GroupedMatmulW4, group_list must have one entry per expert (" << e << "), but got " << group_list.shape();
  }
  const ShapeVector &ws = weight_scale.shape();
  if (ws.size() != kDim3 || ws[kIndex0] != e || ws[kIndex2] != n || ws[kIndex1] <= 0 || k % ws[kIndex1] != 0) {
    MS_EXCEPTION_VALUE << "For GroupedMatmulW4, weight_scale must be [e, k / group_size, n] = [" << e << ", k / group_size, " << n
                       << "], but got " << ws;
  }
  if (x_scale.shape().size() != kDim1 || x_scale.shape()[kIndex0] != m) {
    MS_EXCEPTION_VALUE << "For GroupedMatmulW4, x_scale must be [m] = [" << m << "], but got " << x_scale.shape();
  }
  if (bias.shape().size() != kDim2 || bias.shape()[kIndex0] != e || bias.shape()[kIndex1] != n) {
    MS_EXCEPTION_VALUE << "For GroupedMatmulW4, bias must be [e, n] = [" << e << ", " << n << "], but got " << bias.shape();
  }
  const int64_t group_size = k / ws[kIndex1];
  void *stream = CurrentStream();
  int rc;
  {
    GilReleaseWithCheck release;
    rc = msco_gmm_a8w4(static_cast<const int8_t *>(x.GetDataPtr()), weight.GetDataPtr(),
                       static_cast<const int32_t *>(group_list.GetDataPtr()), static_cast<const float *>(x_scale.GetDataPtr()),
                       static_cast<const float *>(weight_scale.GetDataPtr()), out.GetDataPtr(), m, k, n, e, group_size, stream);
  }
  if (rc == MSCO_ERR_SHAPE || rc == MSCO_ERR_UNSUPPORTED) {
    MS_EXCEPTION_VALUE << "For GroupedMatmulW4, k must be a multiple of 32 and of the K-group size, the K-group size a multiple "
                       << "of 32 and k at most 8192, but got k = " << k << " and a K-group size of " << group_size;
  }
  if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << op_name << ", the backend launch failed: " << msco_status_string(rc);
}

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
class CustomGroupedMatmulW4OpFuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override {
    return {InferGroupedMatmulW4OutputShape(inputs[0].GetShape(), inputs[1].GetShape(), inputs[2].GetShape())};
  }
  TypeIdList InferType(const KernelTensorList &inputs) const override {
    CheckGroupedMatmulW4Types(inputs[0].GetType(), inputs[1].GetType(), inputs[2].GetType(), inputs[3].GetType(),
                              inputs[4].GetType(), inputs[5].GetType());
    return {kNumberTypeFloat16};
  }
};

class CustomGroupedMatmulW4 : public KernelMod {
 public:
  std::vector<size_t> Resize(const KernelTensorList &, const std::vector<ms::Tensor> &) override { return {}; }
  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &, const std::vector<ms::Tensor> &outputs,
              void *stream) override {
    LaunchStreamScope on_launch_stream(stream);   // the routine below enqueues on CurrentStream()
    RunGroupedMatmulW4(inputs[0].tensor, inputs[1].tensor, inputs[2].tensor, inputs[3].tensor, inputs[4].tensor,
                       inputs[5].tensor, outputs[0]);
    return true;
  }
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(grouped_matmul_w4, ms_custom_ops::CustomGroupedMatmulW4OpFuncImpl, ms_custom_ops::CustomGroupedMatmulW4);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
ms::Tensor pyboost_grouped_matmul_w4(const ms::Tensor &x, const ms::Tensor &weight, const ms::Tensor &group_list,
                                     const ms::Tensor &bias, const ms::Tensor &x_scale, const ms::Tensor &weight_scale) {
  const auto out_shape = InferGroupedMatmulW4OutputShape(x.shape(), weight.shape(), group_list.shape());
  ms::Tensor out = AllocateTensor(kNumberTypeFloat16, out_shape);
  RunGroupedMatmulW4(x, weight, group_list, bias, x_scale, weight_scale, out);
  return out;
}
}  // namespace ms_custom_ops

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("grouped_matmul_w4", &ms_custom_ops::pyboost_grouped_matmul_w4, "GroupedMatmulW4", pybind11::arg("x"),
        pybind11::arg("weight"), pybind11::arg("group_list"), pybind11::arg("bias"), pybind11::arg("x_scale"),
        pybind11::arg("weight_scale"));
}
