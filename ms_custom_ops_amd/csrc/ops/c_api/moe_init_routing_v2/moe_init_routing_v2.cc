// moe_init_routing_v2(x, expert_idx, active_num, expert_capacity, expert_num, drop_pad_mode,
//                     expert_tokens_count_or_cumsum_flag, expert_tokens_before_capacity_flag)
//   -> (expanded_x, expanded_row_idx, expert_tokens_count_or_cumsum, expert_tokens_before_capacity)
//
// The routing step in front of the grouped matmul.  Interface, shape rules and messages follow the
// reference (ops/c_api/moe_init_routing_v2/moe_init_routing_v2.cc): x and expert_idx are 2-D (:52-58),
// hidden_size <= 7168 and a multiple of 1024 (:62-66), expert_num <= 256 (:67-70), active_num,
// expert_capacity and drop_pad_mode must be 0 (:107-109); four outputs, the index outputs in expert_idx's
// type (:117-121,127-132).  The reference creates a closed kernel object (:146,180); here the work is one
// call of msco_moe_init_routing_v2 on the framework's current stream.
#include <string>
#include <vector>

#include "msco_moe.h"
#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
constexpr size_t kMoeInitInputRank = 2;
constexpr int64_t kMoeInitHiddenLimit = 7168;
constexpr int64_t kMoeInitHiddenBase = 1024;
constexpr int64_t kMoeInitExpertLimit = 256;

static void MoeInitCheckVal(const std::string &op_name, int64_t value, int64_t expected, const std::string &name) {
  if (value != expected) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], " << name << " must be " << expected << ", but got " << value;
  }
}

static ShapeVector MoeInitRoutingV2MakeShape(const std::string &op_name, const ShapeVector &x_shape,
                                             const ShapeVector &expert_idx_shape, int64_t expert_num) {
  if (x_shape.size() != kMoeInitInputRank) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the rank of x must be " << kMoeInitInputRank << ", but got "
                       << x_shape.size();
  }
  if (expert_idx_shape.size() != kMoeInitInputRank) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the rank of expert_idx must be " << kMoeInitInputRank
                       << ", but got " << expert_idx_shape.size();
  }
  const int64_t h = x_shape[kIndex1];
  if (h > kMoeInitHiddenLimit || h % kMoeInitHiddenBase != 0) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the hidden_size of x must be less than or " << kMoeInitHiddenLimit
                       << " and be multiple of " << kMoeInitHiddenBase << ", but got " << h;
  }
  if (expert_num > kMoeInitExpertLimit) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], the expert_num must be less than or equal to "
                       << kMoeInitExpertLimit << ", but got " << expert_num;
  }
  if (expert_idx_shape[kIndex0] != x_shape[kIndex0]) {
    MS_EXCEPTION_VALUE << "For op [" << op_name << "], x and expert_idx must have the same number of rows, but got "
                       << x_shape << " and " << expert_idx_shape;
  }
  return ShapeVector{x_shape[kIndex0] * expert_idx_shape[kIndex1], h};
}

static void RunMoeInitRoutingV2(const ms::Tensor &x, const ms::Tensor &expert_idx, int64_t active_num,
                                int64_t expert_capacity, int64_t expert_num, int64_t drop_pad_mode, int64_t flag,
                                const std::vector<ms::Tensor> &outputs) {
  const std::string op_name = "MoeInitRoutingV2";
  MoeInitCheckVal(op_name, active_num, 0, "active_num");
  MoeInitCheckVal(op_name, expert_capacity, 0, "expert_capacity");
  MoeInitCheckVal(op_name, drop_pad_mode, 0, "drop_pad_mode");
  if (expert_idx.data_type() != kNumberTypeInt32) {
    MS_EXCEPTION_TYPE << "For op [" << op_name << "], expert_idx must be Int32, but got " << expert_idx.data_type();
  }
  if (expert_num <= 0) MS_EXCEPTION_VALUE << "For op [" << op_name << "], expert_num must be positive, but got " << expert_num;
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
    rc = msco_moe_init_routing_v2(x.GetDataPtr(), static_cast<const int32_t *>(expert_idx.GetDataPtr()),
                                  outputs[0].GetDataPtr(), static_cast<int32_t *>(outputs[1].GetDataPtr()),
                                  static_cast<int32_t *>(outputs[2].GetDataPtr()),
                                  static_cast<int32_t *>(outputs[3].GetDataPtr()),
                                  workspace.is_defined() ? workspace.GetDataPtr() : nullptr, ws_bytes, num_rows, hidden, k,
                                  expert_num, static_cast<int32_t>(TypeIdSize(x.data_type())), static_cast<int32_t>(flag),
                                  stream);
  }
  if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << op_name << ", the backend launch failed: " << msco_status_string(rc);
}

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
class MoeInitRoutingV2FuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override {
    const int64_t expert_num = inputs[4].GetValueWithCheck<int64_t>();
    MoeInitCheckVal("MoeInitRoutingV2", inputs[2].GetValueWithCheck<int64_t>(), 0, "active_num");
    MoeInitCheckVal("MoeInitRoutingV2", inputs[3].GetValueWithCheck<int64_t>(), 0, "expert_capacity");
    MoeInitCheckVal("MoeInitRoutingV2", inputs[5].GetValueWithCheck<int64_t>(), 0, "drop_pad_mode");
    const ShapeVector expanded = MoeInitRoutingV2MakeShape("MoeInitRoutingV2", inputs[0].GetShape(), inputs[1].GetShape(), expert_num);
    return {expanded, ShapeVector{expanded[kIndex0]}, ShapeVector{expert_num}, ShapeVector{expert_num}};
  }
  TypeIdList InferType(const KernelTensorList &inputs) const override {
    const TypeId x_type = inputs[0].GetType(), idx_type = inputs[1].GetType();
    return {x_type, idx_type, idx_type, idx_type};
  }
};

class MoeInitRoutingV2Hip : public KernelMod {
 public:
  std::vector<size_t> Resize(const KernelTensorList &, const std::vector<ms::Tensor> &) override { return {}; }
  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &, const std::vector<ms::Tensor> &outputs,
              void *stream) override {
    LaunchStreamScope on_launch_stream(stream);   // the routine below enqueues on CurrentStream()
    RunMoeInitRoutingV2(inputs[0].tensor, inputs[1].tensor, inputs[2].GetValueWithCheck<int64_t>(),
                        inputs[3].GetValueWithCheck<int64_t>(), inputs[4].GetValueWithCheck<int64_t>(),
                        inputs[5].GetValueWithCheck<int64_t>(), inputs[6].GetValueWithCheck<int64_t>(), outputs);
    return true;
  }
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(moe_init_routing_v2, ms_custom_ops::MoeInitRoutingV2FuncImpl, ms_custom_ops::MoeInitRoutingV2Hip);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
std::vector<ms::Tensor> moe_init_routing_v2_custom(const ms::Tensor &x, const ms::Tensor &expert_idx, int64_t active_num,
                                                   int64_t expert_capacity, int64_t expert_num, int64_t drop_pad_mode,
                                                   int64_t expert_tokens_count_or_cumsum_flag,
                                                   bool expert_tokens_before_capacity_flag) {
  (void)expert_tokens_before_capacity_flag;   // an output of the drop/pad mode, which the op does not accept
  const auto expanded = MoeInitRoutingV2MakeShape("MoeInitRoutingV2", x.shape(), expert_idx.shape(), expert_num);
  std::vector<ms::Tensor> outputs = {AllocateTensor(x.data_type(), expanded),
                                     AllocateTensor(expert_idx.data_type(), {expanded[kIndex0]}),
                                     AllocateTensor(expert_idx.data_type(), {expert_num}),
                                     AllocateTensor(expert_idx.data_type(), {expert_num})};
  RunMoeInitRoutingV2(x, expert_idx, active_num, expert_capacity, expert_num, drop_pad_mode,
                      expert_tokens_count_or_cumsum_flag, outputs);
  return outputs;
}
}  // namespace ms_custom_ops

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("moe_init_routing_v2", &ms_custom_ops::moe_init_routing_v2_custom, "MoeInitRoutingV2", pybind11::arg("x"),
        pybind11::arg("expert_idx"), pybind11::arg("active_num"), pybind11::arg("expert_capacity"),
        pybind11::arg("expert_num"), pybind11::arg("drop_pad_mode"), pybind11::arg("expert_tokens_count_or_cumsum_flag"),
        pybind11::arg("expert_tokens_before_capacity_flag"));
}
