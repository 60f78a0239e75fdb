// moe_token_unpermute(permuted_tokens, sorted_indices, probs, padded_mode=False, restore_shape=None)
//
// The step behind the grouped matmul: out[i] = sum_k probs[i, k] * permuted_tokens[sorted_indices[i * K + k]].
// Interface and rules follow the reference (ops/c_api/moe_token_unpermute/moe_token_unpermute.cc): both tensor
// arguments 2-D (:43-50), output [tokens, hidden] in permuted_tokens' type (:51-52,71-78), float16 only (:73-76);
// padded_mode / restore_shape are accepted and must stay at their defaults, top_k in {1, 2, 4, 8} and hidden in
// {2048, 5120, 7168} as the reference's kernel demands (moe_token_unpermute.md "特殊说明"; an unsupported hidden
// size is a "Tiling error" RuntimeError, tests/st/test_custom_moe_token_unpermute.py:100-103).  bfloat16 is an
// extension of this backend.
#include <optional>
#include <string>
#include <vector>

#include "msco_moe.h"
#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
static ShapeVector MoeTokenUnpermuteMakeShape(const ShapeVector &permuted_tokens_shape, const ShapeVector &probs_shape) {
  if (permuted_tokens_shape.size() != kDim2) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, permuted_tokens must be a 2D tensor, but got dimension: "
                     << permuted_tokens_shape.size();
  }
  if (probs_shape.size() != kDim2) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, probs must be a 2D tensor, but got dimension: " << probs_shape.size();
  }
  return ShapeVector{probs_shape[0], permuted_tokens_shape[1]};
}

static void RunMoeTokenUnpermute(const ms::Tensor &permuted_tokens, const ms::Tensor &sorted_indices, const ms::Tensor &probs,
                                 bool padded_mode, bool has_restore_shape, const ms::Tensor &out) {
  const std::string op_name = "MoeTokenUnpermute";
  const TypeId t = permuted_tokens.data_type();
  if (t != kNumberTypeFloat16 && t != kNumberTypeBFloat16) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, permuted_tokens must be a float16 tensor, but got: " << t;
  }
  if (probs.data_type() != t) MS_LOG_EXCEPTION << "For MoeTokenUnpermute, probs must have permuted_tokens' type, but got: " << probs.data_type();
  if (sorted_indices.data_type() != kNumberTypeInt32) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, sorted_indices must be an int32 tensor, but got: " << sorted_indices.data_type();
  }
  if (padded_mode || has_restore_shape) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, only padded_mode = False and restore_shape = None are supported.";
  }
  const int64_t tokens = probs.shape()[0], top_k = probs.shape()[1], hidden = permuted_tokens.shape()[1];
  if (permuted_tokens.shape()[0] != tokens * top_k || sorted_indices.numel() != tokens * top_k) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, permuted_tokens and sorted_indices must hold tokens * top_k = " << tokens * top_k
                     << " rows, but got " << permuted_tokens.shape() << " and " << sorted_indices.shape();
  }
  const bool k_ok = top_k == 1 || top_k == 2 || top_k == 4 || top_k == 8;
  const bool h_ok = hidden == 2048 || hidden == 5120 || hidden == 7168;
  if (!k_ok || !h_ok) {
    MS_LOG_EXCEPTION << "For MoeTokenUnpermute, Tiling error: top_k must be 1, 2, 4 or 8 and hidden_size 2048, 5120 or 7168, "
                        "but got top_k=" << top_k << ", hidden_size=" << hidden;
  }
  CheckContiguous(op_name, {permuted_tokens, sorted_indices, probs}, true);
  CheckContiguous(op_name, {out}, false);
  void *stream = CurrentStream();
  int rc;
  {
    GilReleaseWithCheck release;
    rc = msco_moe_token_unpermute(permuted_tokens.GetDataPtr(), static_cast<const int32_t *>(sorted_indices.GetDataPtr()),
                                  probs.GetDataPtr(), out.GetDataPtr(), tokens, top_k, hidden,
                                  t == kNumberTypeBFloat16 ? MSCO_DT_BF16 : MSCO_DT_F16, stream);
  }
  if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << op_name << ", the backend launch failed: " << msco_status_string(rc);
}

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
class MoeTokenUnpermuteFuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override {
    return {MoeTokenUnpermuteMakeShape(inputs[0].GetShape(), inputs[2].GetShape())};
  }
  TypeIdList InferType(const KernelTensorList &inputs) const override {
    const TypeId t = inputs[0].GetType();
    if (t != kNumberTypeFloat16 && t != kNumberTypeBFloat16) {
      MS_LOG_EXCEPTION << "For MoeTokenUnpermute, permuted_tokens must be a float16 tensor, but got: " << t;
    }
    return {t};
  }
};

class MoeTokenUnpermuteHip : public KernelMod {
 public:
  std::vector<size_t> Resize(const KernelTensorList &, const std::vector<ms::Tensor> &) override { return {}; }
  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &, const std::vector<ms::Tensor> &outputs,
              void *stream) override {
    LaunchStreamScope on_launch_stream(stream);   // the routine below enqueues on CurrentStream()
    const bool padded = inputs.size() > 3 && !inputs[3].IsNone() && inputs[3].GetValueWithCheck<bool>();
    const bool restore = inputs.size() > 4 && !inputs[4].IsNone();
    RunMoeTokenUnpermute(inputs[0].tensor, inputs[1].tensor, inputs[2].tensor, padded, restore, outputs.at(0));
    return true;
  }
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(moe_token_unpermute, ms_custom_ops::MoeTokenUnpermuteFuncImpl, ms_custom_ops::MoeTokenUnpermuteHip);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
ms::Tensor moe_token_unpermute_custom(const ms::Tensor &permuted_tokens, const ms::Tensor &sorted_indices,
                                      const ms::Tensor &probs, const std::optional<bool> &padded_mode,
                                      const std::optional<std::vector<int32_t>> &restore_shape) {
  auto out = AllocateTensor(permuted_tokens.data_type(), MoeTokenUnpermuteMakeShape(permuted_tokens.shape(), probs.shape()));
  RunMoeTokenUnpermute(permuted_tokens, sorted_indices, probs, padded_mode.value_or(false), restore_shape.has_value(), out);
  return out;
}
}  // namespace ms_custom_ops

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("moe_token_unpermute", &ms_custom_ops::moe_token_unpermute_custom, "MoeTokenUnpermute",
        pybind11::arg("permuted_tokens"), pybind11::arg("sorted_indices"), pybind11::arg("probs"),
        pybind11::arg("padded_mode") = false, pybind11::arg("restore_shape") = std::nullopt);
}
