// moe_init_routing_quant(x, expert_idx, expert_num, expert_tokens_count_or_cumsum_flag)
//   -> (expanded_x int8, expanded_scale float32, expanded_row_idx, expert_tokens_count_or_cumsum)
//
// The routing step in front of an int8-activation grouped matmul with the activation quantisation done on the
// way: rows are sorted by expert as moe_init_routing_v2 sorts them (ops/c_api/moe_init_routing_v2/
// moe_init_routing_v2.cc:47-72 for the shape rules kept here) and every gathered row is quantised per token as the
// reference's test quantises the activations it feeds to the int8 path (dyn_quant, tests/st/test_grouped_matmul_w4.py:83-89).
// The reference has no operator for the pair; the outputs are what grouped_matmul_v4_cops takes as x and
// per_token_scale, and expert_tokens_count_or_cumsum (flag 1) as its group_list.
#include <string>
#include <vector>

#include "msco_moe.h"
#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
constexpr size_t kMoeQuantInputRank = 2;
constexpr int64_t kMoeQuantHiddenAlign = 8;
constexpr int64_t kMoeQuantExpertLimit = 1024;

static ShapeVector MoeInitRoutingQuantMakeShape(const std::string &op_name, const ShapeVector &x_shape,
                                                const ShapeVector &expert_idx_shape, int64_t expert_num) {
  if (x_shape.size() != kMoeQuantInputRank) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the rank of x must be " << kMoeQuantInputRank << ", but got "
                       << x_shape.size();
  }
  if (expert_idx_shape.size() != kMoeQuantInputRank) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the rank of expert_idx must be " << kMoeQuantInputRank
                       << ", but got " << expert_idx_shape.size();
  }
  const int64_t h = x_shape[kIndex1];
  if (h <= 0 || h % kMoeQuantHiddenAlign != 0) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the hidden_size of x must be a multiple of " << kMoeQuantHiddenAlign
                       << ", but got " << h;
  }
  if (expert_num <= 0 || expert_num > kMoeQuantExpertLimit) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the expert_num must be in [1, " << kMoeQuantExpertLimit
                       << "], but got " << expert_num;
  }
  if (expert_idx_shape[kIndex0] != x_shape[kIndex0]) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], x and expert_idx must have the same number of rows, but got "
                       << x_shape << " and " << expert_idx_shape;
  }
  return ShapeVector{x_shape[kIndex0] * expert_idx_shape[kIndex1], h};
}

static void RunMoeInitRoutingQuant(const ms::Tensor &x, const ms::Tensor &expert_idx, int64_t expert_num, int64_t flag,
                                   const std::vector<ms::Tensor> &outputs) {
  const std::string op_name = "MoeInitRoutingQuant";
  if (x.data_type() != kNumberTypeFloat16 && x.data_type() != kNumberTypeBFloat16) {
    MS_EXCEPTION_TYPE << "For op [" << op_name << "], x must be Float16 or BFloat16, but got " << x.data_type();
  }
  if (expert_idx.data_type() != kNumberTypeInt32) {
    MS_EXCEPTION_TYPE << "For op [" << op_name << "], expert_idx must be Int32, but got " << expert_idx.data_type();
  }
  if (flag < 0 || flag > 2) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], expert_tokens_count_or_cumsum_flag must be 0, 1 or 2, but got " << flag;
  }
  CheckContiguous(op_name, {x, expert_idx}, true);
  CheckContiguous(op_name, outputs, false);
  const int64_t num_rows = x.shape()[kIndex0], hidden = x.shape()[kIndex1], k = expert_idx.shape()[kIndex1];
  void *stream = CurrentStream();
  const size_t ws_bytes = msco_moe_init_routing_v2_workspace_bytes(num_rows, k, expert_num);
  ms::Tensor workspace;
  if (ws_bytes > 0) workspace = AllocateTensor(kNumberTypeInt8, ShapeVector{static_cast<int64_t>(ws_bytes)});
  int rc;
  {
    GilReleaseWithCheck release;
    rc = msco_moe_init_routing_v2_quant(x.GetDataPtr(), static_cast<const int32_t *>(expert_idx.GetDataPtr()),
                                        static_cast<int8_t *>(outputs[0].GetDataPtr()),
                                        static_cast<float *>(outputs[1].GetDataPtr()),
                                        static_cast<int32_t *>(outputs[2].GetDataPtr()),
                                        static_cast<int32_t *>(outputs[3].GetDataPtr()), nullptr,
                                        workspace.is_defined() ? workspace.GetDataPtr() : nullptr, ws_bytes, num_rows, hidden,
                                        k, expert_num, x.data_type() == kNumberTypeBFloat16 ? MSCO_DT_BF16 : MSCO_DT_F16,
                                        static_cast<int32_t>(flag), stream);
  }
  if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << op_name << ", the backend launch failed: " << msco_status_string(rc);
}

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
class MoeInitRoutingQuantFuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override {
    const int64_t expert_num = inputs[2].GetValueWithCheck<int64_t>();
    const ShapeVector expanded = MoeInitRoutingQuantMakeShape("MoeInitRoutingQuant", inputs[0].GetShape(), inputs[1].GetShape(), expert_num);
    return {expanded, ShapeVector{expanded[kIndex0]}, ShapeVector{expanded[kIndex0]}, ShapeVector{expert_num}};
  }
  TypeIdList InferType(const KernelTensorList &inputs) const override {
    const TypeId idx_type = inputs[1].GetType();
    return {kNumberTypeInt8, kNumberTypeFloat32, idx_type, idx_type};
  }
};

class MoeInitRoutingQuantHip : public KernelMod {
 public:
  std::vector<size_t> Resize(const KernelTensorList &, const std::vector<ms::Tensor> &) override { return {}; }
  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &, const std::vector<ms::Tensor> &outputs,
              void *stream) override {
    LaunchStreamScope on_launch_stream(stream);   // the routine below enqueues on CurrentStream()
    RunMoeInitRoutingQuant(inputs[0].tensor, inputs[1].tensor, inputs[2].GetValueWithCheck<int64_t>(),
                           inputs[3].GetValueWithCheck<int64_t>(), outputs);
    return true;
  }
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(moe_init_routing_quant, ms_custom_ops::MoeInitRoutingQuantFuncImpl, ms_custom_ops::MoeInitRoutingQuantHip);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
std::vector<ms::Tensor> moe_init_routing_quant_custom(const ms::Tensor &x, const ms::Tensor &expert_idx, int64_t expert_num,
                                                      int64_t expert_tokens_count_or_cumsum_flag) {
  const auto expanded = MoeInitRoutingQuantMakeShape("MoeInitRoutingQuant", x.shape(), expert_idx.shape(), expert_num);
  std::vector<ms::Tensor> outputs = {AllocateTensor(kNumberTypeInt8, expanded),
                                     AllocateTensor(kNumberTypeFloat32, {expanded[kIndex0]}),
                                     AllocateTensor(expert_idx.data_type(), {expanded[kIndex0]}),
                                     AllocateTensor(expert_idx.data_type(), {expert_num})};
  RunMoeInitRoutingQuant(x, expert_idx, expert_num, expert_tokens_count_or_cumsum_flag, outputs);
  return outputs;
}
}  // namespace ms_custom_ops

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("moe_init_routing_quant", &ms_custom_ops::moe_init_routing_quant_custom, "MoeInitRoutingQuant", pybind11::arg("x"),
        pybind11::arg("expert_idx"), pybind11::arg("expert_num"), pybind11::arg("expert_tokens_count_or_cumsum_flag"));
}
