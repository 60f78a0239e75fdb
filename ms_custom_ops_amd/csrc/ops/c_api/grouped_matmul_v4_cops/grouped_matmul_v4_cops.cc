// grouped_matmul_v4_cops(x, weight, bias, scale, offset, antiquant_scale, antiquant_offset,
//                        per_token_scale, group_list, activation_input, activation_quant_scale,
//                        activation_quant_offset, split_item, group_type, group_list_type, act_type,
//                        weight_format, output_dtype) -> list of tensors
//
// List-of-tensor GMM-V4 entry of the reference (ops/c_api/grouped_matmul_v4_cops/
// grouped_matmul_v4_cops.cc): same eighteen arguments and defaults (:395-405), int64 group_list with
// group_list_type 0 (cumulative) or 1 (counts), output dtype rules of InferOutputTypes (:162-203).
// The reference forwards the twelve lists to aclnnGroupedMatmulV4 (:359-363); here
//   * group_type 0 (one x [M,K], one weight [E,K,N], one output [M,N]) is one grouped launch of the
//     HIP backend: W8A8 with per-channel scale / per-token scale / int32 bias, or weight-only
//     (bf16/f16 x, int8 weight, antiquant scale and offset [E,N]); with a qint4x2 weight [E,K,N/2] (A8W4,
//     tests/st/test_grouped_matmul_v4_cops.py:429-485, and A16W4, :197-262) the nibble pairs are widened to int8 on the
//     device first (msco_unpack_int4) and the W8A8 or the weight-only launch multiplies them: exact, at the price of
//     one more pass over the weights;
//   * group_type -1 (independent x[i] @ weight[i]) is one dense launch per pair.
// Not implemented on this backend and refused with a message: float x float matmuls,
// uint64 scales with int8 output, `offset`, the activation inputs, group_type 1.  act_type selects an activation
// fused into the epilogue (0 none, 1 relu, 2 gelu_tanh, 4 fast_gelu, 5 silu: the values of CANN's GMMActType, which the
// reference passes through without naming them).
#include <optional>
#include <string>
#include <vector>

#include "ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops_func_impl.h"
#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
namespace {
struct V4Args {
  TensorVec x, weight, bias, scale, offset, antiquant_scale, antiquant_offset, per_token_scale;
  ms::Tensor group_list;
  TensorVec activation_input, activation_quant_scale, activation_quant_offset;
  int64_t split_item{0}, group_type{-1}, group_list_type{0}, act_type{0};
  std::string weight_format{"ND"};
};

const ms::Tensor &At(const TensorVec &v, size_t i) {
  static const ms::Tensor empty;
  return i < v.size() ? v[i] : empty;
}

void CheckV4Support(const V4Args &a) {
  if (a.weight_format != kNdFormat && a.weight_format != kFractalNzFormat) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", weight_format must be 'ND' or 'FRACTAL_NZ', but got '"
                     << a.weight_format << "'.";
  }
  // act_type goes to the backend as the reference hands it to aclnnGroupedMatmulV4 (grouped_matmul_v4_cops.cc:96,363):
  // 0 none, 1 relu, 2 gelu (tanh form), 4 fast gelu, 5 silu; 3 (gelu, erf form) is the value CANN itself lists as unsupported
  if (a.act_type < MSCO_ACT_NONE || a.act_type > MSCO_ACT_SILU || a.act_type == MSCO_ACT_GELU_ERF) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", act_type must be 0 (none), 1 (relu), 2 (gelu_tanh), "
                       << "4 (fast_gelu) or 5 (silu), but got " << a.act_type;
  }
  if (!a.activation_input.empty() || !a.activation_quant_scale.empty() || !a.activation_quant_offset.empty()) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName
                     << ", 'activation_input', 'activation_quant_scale' and 'activation_quant_offset' are not implemented by the HIP backend.";
  }
  if (!a.offset.empty()) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", 'offset' is not implemented by the HIP backend.";
  }
  if (a.group_list_type != 0 && a.group_list_type != 1) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", group_list_type must be 0 or 1, but got "
                       << a.group_list_type;
  }
  const TypeId xt = a.x[0].data_type(), wt = a.weight[0].data_type();
  if (wt == kNumberTypeInt4) {
    // qint4x2 weight [E, K, N / 2], one output: A8W4 with int8 x (tests/st/test_grouped_matmul_v4_cops.py:429-485) and
    // A16W4 with float16 / bfloat16 x and the antiquant inputs (:197-262)
    if ((xt != kNumberTypeInt8 && xt != kNumberTypeFloat16 && xt != kNumberTypeBFloat16) ||
        a.group_type != kGroupTypeSingleOutput || a.weight_format != kNdFormat) {
      MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", int4 weights are implemented for Int8, Float16 or "
                       << "BFloat16 'x', group_type 0 and weight_format 'ND' only, but got x dtype " << xt
                       << ", group_type " << a.group_type << ", weight_format '" << a.weight_format << "'.";
    }
    return;
  }
  if (wt != kNumberTypeInt8) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName
                     << ", the HIP backend implements the quantized paths only (int8 weight), but got weight dtype "
                     << wt;
  }
  if (xt != kNumberTypeInt8 && xt != kNumberTypeBFloat16 && xt != kNumberTypeFloat16) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", 'x' must be Int8, BFloat16 or Float16, but got " << xt;
  }
}

// One backend launch: descriptor, problem size, positional device addresses and the output.
struct OneLaunch {
  msco_gmm_desc desc{};
  GmmProblem problem{};
  const void *addrs[MSCO_IN_COUNT] = {nullptr};
  void *out{nullptr};
  // 4-bit weights: the nibble pairs (int4_bytes bytes at int4_src) are widened to int8 in a staging buffer of twice that
  // size first, and addrs[MSCO_IN_WEIGHT] is set to the staging buffer
  const void *int4_src{nullptr};
  size_t int4_bytes{0};
};
const char *const kBackendOpName = "GroupedMatmulV4";

// One launch: x [M,K], weight [E,K,N], optional per-group rows of bias / scale / antiquant.
OneLaunch BuildOne(const ms::Tensor &x, const ms::Tensor &w, const ms::Tensor &bias, const ms::Tensor &scale,
                   const ms::Tensor &aq_scale, const ms::Tensor &aq_offset, const ms::Tensor &per_token,
                   const ms::Tensor &group_list, int64_t group_list_type, const ms::Tensor &out, int64_t m, int64_t k,
                   int64_t n, int64_t e, bool packed, int64_t act_type) {
  const TypeId xt = x.data_type();
  const bool int4 = w.data_type() == kNumberTypeInt4;
  OneLaunch one;
  one.problem = GmmProblem{m, k, n, e};
  one.out = out.GetDataPtr();
  msco_gmm_desc &d = one.desc;
  const void **addrs = one.addrs;
  d.abi_version = MSCO_GMM_ABI_VERSION;
  d.x_dtype = ToBackendDtype(xt);
  d.weight_dtype = MSCO_DT_I8;
  d.out_dtype = ToBackendDtype(out.data_type());
  d.group_list_dtype = group_list.is_defined() ? ToBackendDtype(group_list.data_type()) : MSCO_DT_NONE;
  d.group_list_type = static_cast<int32_t>(group_list_type);
  d.scale_per_group = 1;
  d.weight_layout = packed ? MSCO_WL_PACKED : MSCO_WL_ROW_MAJOR;
  if (act_type != MSCO_ACT_NONE && out.data_type() == kNumberTypeInt32) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", act_type " << act_type
                       << " needs a floating-point output (give 'scale'), but the output is Int32.";
  }
  d.act_type = static_cast<int32_t>(act_type);
  addrs[MSCO_IN_X] = x.GetDataPtr();
  addrs[MSCO_IN_WEIGHT] = w.GetDataPtr();
  if (int4) {
    one.int4_src = w.GetDataPtr();
    one.int4_bytes = w.nbytes();
    addrs[MSCO_IN_WEIGHT] = nullptr;   // the staging buffer, set by the caller
  }
  addrs[MSCO_IN_GROUP_LIST] = group_list.is_defined() ? group_list.GetDataPtr() : nullptr;
  auto expect_en = [&](const ms::Tensor &t, const char *name) {
    if (t.is_defined() && t.numel() != e * n) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", '" << name << "' must have E*N = " << e * n
                         << " elements, but got shape " << t.shape();
    }
  };
  if (xt == kNumberTypeInt8) {
    if (aq_scale.is_defined() || aq_offset.is_defined()) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", antiquant inputs need a floating-point 'x'.";
    }
    const bool raw = out.data_type() == kNumberTypeInt32;
    expect_en(bias, "bias");
    expect_en(scale, "scale");
    if (int4) {
      // The reference kernel multiplies the nibbles unsigned and needs bias = 8 * sum_k w[k, n] * scale[n] (Float32,
      // tests/st/test_grouped_matmul_v4_cops.py:463) to compensate; here they are multiplied signed, so the term is
      // checked for its type and not read (the expected value of the test, :467-476, contains no bias either).
      if (bias.is_defined() && bias.data_type() != kNumberTypeFloat32) {
        MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << " with A8W4, 'bias' must be Float32, but got "
                           << bias.data_type();
      }
      if (!scale.is_defined() || out.data_type() == kNumberTypeInt32) {
        MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << " with A8W4, 'scale' must be given.";
      }
    } else if (bias.is_defined() && bias.data_type() != kNumberTypeInt32) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", the quantized path takes an Int32 'bias', but got "
                         << bias.data_type();
    }
    if (per_token.is_defined() && (per_token.data_type() != kNumberTypeFloat32 || per_token.numel() != m)) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", 'per_token_scale' must be Float32 with M = " << m
                         << " elements, but got " << per_token.data_type() << " " << per_token.shape();
    }
    d.bias_dtype = (bias.is_defined() && !int4) ? MSCO_DT_I32 : MSCO_DT_NONE;
    d.scale_dtype = (!raw && scale.is_defined()) ? ToBackendDtype(scale.data_type()) : MSCO_DT_NONE;
    d.per_token_dtype = (!raw && per_token.is_defined()) ? MSCO_DT_F32 : MSCO_DT_NONE;
    addrs[MSCO_IN_BIAS] = d.bias_dtype != MSCO_DT_NONE ? bias.GetDataPtr() : nullptr;
    addrs[MSCO_IN_SCALE] = d.scale_dtype != MSCO_DT_NONE ? scale.GetDataPtr() : nullptr;
    addrs[MSCO_IN_PER_TOKEN_SCALE] = d.per_token_dtype != MSCO_DT_NONE ? per_token.GetDataPtr() : nullptr;
  } else {
    if (!aq_scale.is_defined()) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", weight-only quantization needs 'antiquant_scale'.";
    }
    if (aq_scale.data_type() != xt || (aq_offset.is_defined() && aq_offset.data_type() != xt)) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                         << ", 'antiquant_scale' and 'antiquant_offset' must have the dtype of 'x' (" << xt << ").";
    }
    if (bias.is_defined() || scale.is_defined() || per_token.is_defined()) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                         << ", 'bias', 'scale' and 'per_token_scale' are not used by the weight-only path.";
    }
    expect_en(aq_scale, "antiquant_scale");
    expect_en(aq_offset, "antiquant_offset");
    d.antiquant_dtype = ToBackendDtype(xt);
    d.has_antiquant_offset = aq_offset.is_defined() ? 1 : 0;
    addrs[MSCO_IN_ANTIQUANT_SCALE] = aq_scale.GetDataPtr();
    addrs[MSCO_IN_ANTIQUANT_OFFSET] = aq_offset.is_defined() ? aq_offset.GetDataPtr() : nullptr;
  }
  return one;
}

// The backend launches a call consists of, in order: one for group_type 0, one per (x[i], weight[i]) pair for -1.
std::vector<OneLaunch> BuildLaunches(const V4Args &a, const TensorVec &outputs) {
  std::vector<OneLaunch> launches;
  CheckV4Support(a);
  TensorVec all = a.x;
  for (const auto *v : {&a.weight, &a.bias, &a.scale, &a.antiquant_scale, &a.antiquant_offset, &a.per_token_scale}) {
    all.insert(all.end(), v->begin(), v->end());
  }
  all.push_back(a.group_list);
  CheckContiguous("GroupedMatmulV4", all, true);
  CheckContiguous("GroupedMatmulV4", outputs, false);

  if (a.group_type == kGroupTypeSingleOutput) {
    const auto &x = a.x[0];
    const auto &w = a.weight[0];
    const bool packed = a.weight_format == kFractalNzFormat;   // [E, N / 16, ceil(K / 64), 1024] from trans_data
    if (x.shape().size() != kDim2 || (packed ? !IsPackedWeightShape(w.shape(), kDim4) : w.shape().size() != kDim3)) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", with group_type 0 'x' must be [M, K] and 'weight' "
                         << (packed ? "[E, N/16, ceil(K/64), 1024] (prepacked by trans_data)" : "[E, K, N]") << ", but got "
                         << x.shape() << " and " << w.shape();
    }
    // (qint4x2: two 4-bit values per stored element along N -- UnifyWeightShape of the reference,
    // ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:56-66,274-295)
    const int64_t n_mul = w.data_type() == kNumberTypeInt4 ? 2 : 1;
    const int64_t m = x.shape()[0], k = x.shape()[1], e = w.shape()[0], n = packed ? w.shape()[1] * 16 : w.shape()[2] * n_mul;
    const int64_t wk = packed ? (w.shape()[2] == (k + 63) / 64 ? k : w.shape()[2] * 64) : w.shape()[1];
    if (wk != k) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", the K dimension of 'x' and 'weight' must be equal, "
                         << "but got " << k << " and " << wk;
    }
    if (!a.group_list.is_defined()) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", group_type 0 needs 'group_list'.";
    }
    if (a.group_list.data_type() != kNumberTypeInt64 || a.group_list.numel() != e) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", 'group_list' must be Int64 with E = " << e
                         << " elements, but got " << a.group_list.data_type() << " " << a.group_list.shape();
    }
    launches.push_back(BuildOne(x, w, At(a.bias, 0), At(a.scale, 0), At(a.antiquant_scale, 0), At(a.antiquant_offset, 0),
                                At(a.per_token_scale, 0), a.group_list, a.group_list_type, outputs.at(0), m, k, n, e, packed,
                                a.act_type));
    return launches;
  }
  if (a.group_type != kGroupTypeMultiOutput) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", group_type " << a.group_type
                     << " is not implemented by the HIP backend (supported: -1 and 0).";
  }
  // independent problems x[i] [..., m, k] @ weight[i] [k, n]
  for (size_t i = 0; i < a.x.size(); ++i) {
    const auto &x = a.x[i];
    const auto &w = a.weight[i];
    const bool packed = a.weight_format == kFractalNzFormat;   // [N / 16, ceil(K / 64), 1024] from trans_data
    if ((packed ? !IsPackedWeightShape(w.shape(), kDim3) : w.shape().size() != kDim2) || x.shape().size() < kDim2) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", with group_type -1 every weight must be "
                         << (packed ? "[N/16, ceil(K/64), 1024] (prepacked by trans_data) " : "[K, N] ")
                         << "and every x at least 2D, but got " << x.shape() << " and " << w.shape();
    }
    const int64_t k = x.shape().back(), n = packed ? w.shape()[0] * 16 : w.shape()[1];
    const int64_t wk = packed ? (w.shape()[1] == (k + 63) / 64 ? k : w.shape()[1] * 64) : w.shape()[0];
    if (wk != k) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", the K dimension of 'x' and 'weight' must be equal, "
                         << "but got " << k << " and " << wk;
    }
    const int64_t rows = k > 0 ? x.numel() / k : 0;
    launches.push_back(BuildOne(x, w, At(a.bias, i), At(a.scale, i), At(a.antiquant_scale, i), At(a.antiquant_offset, i),
                                At(a.per_token_scale, i), ms::Tensor(), 0, outputs.at(i), rows, k, n, 1, packed, a.act_type));
  }
  return launches;
}

// 4-bit weights -> int8 in `staging` (2 * int4_bytes bytes), which becomes the launch's weight
void WidenInt4(OneLaunch &one, void *staging, void *stream) {
  const int rc = msco_unpack_int4(one.int4_src, staging, static_cast<int64_t>(one.int4_bytes), stream);
  if (rc != MSCO_OK) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", widening the 4-bit weights failed: " << msco_status_string(rc);
  }
  one.addrs[MSCO_IN_WEIGHT] = staging;
}

// Pynative: plan (cached), take the workspace from the framework's allocator, launch.
void RunGroupedMatmulV4(const V4Args &a, const TensorVec &outputs) {
  void *stream = CurrentStream();
  for (OneLaunch &one : BuildLaunches(a, outputs)) {
    auto plan = GmmPlanCache::GetInstance().GetOrCreate(kBackendOpName, one.desc, one.problem, stream);
    ms::Tensor widened;
    if (one.int4_bytes > 0) {
      widened = AllocateTensor(kNumberTypeInt8, ShapeVector{static_cast<int64_t>(2 * one.int4_bytes)});
      WidenInt4(one, widened.GetDataPtr(), stream);
    }
    ms::Tensor workspace;
    if (plan->workspace_bytes > 0) {
      workspace = AllocateTensor(kNumberTypeInt8, ShapeVector{static_cast<int64_t>(plan->workspace_bytes)});
    }
    LaunchPlan(kBackendOpName, plan, one.addrs, one.out, workspace.is_defined() ? workspace.GetDataPtr() : nullptr,
               plan->workspace_bytes, stream);
  }
}

V4Args ArgsFromGraphInputs(const KernelTensorList &inputs) {
  V4Args args;
  auto list = [&](size_t i) { return inputs[i].IsNone() ? TensorVec() : inputs[i].sequence; };
  args.x = list(kXIndex);
  args.weight = list(kWeightIndex);
  args.bias = list(kBiasIndex);
  args.scale = list(kScaleIndex);
  args.offset = list(kOffsetIndex);
  args.antiquant_scale = list(kAntiquantScaleIndex);
  args.antiquant_offset = list(kAntiquantOffsetIndex);
  args.per_token_scale = list(kPerTokenScaleIndex);
  args.group_list = inputs[kGroupListIndex].tensor;
  args.activation_input = list(kActivationInputIndex);
  args.activation_quant_scale = list(kActivationInputIndex + 1);
  args.activation_quant_offset = list(kActivationInputIndex + 2);
  args.split_item = inputs[kSplitItemIndex].GetValueWithCheck<int64_t>();
  args.group_type = inputs[kGroupTypeIndex].GetValueWithCheck<int64_t>();
  args.group_list_type = inputs[kGroupListTypeIndex].GetValueWithCheck<int64_t>();
  args.act_type = inputs[kActTypeIndex].GetValueWithCheck<int64_t>();
  args.weight_format = inputs[kWeightFormatIndex].GetValueWithCheck<std::string>();
  return args;
}
}  // namespace

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
class GroupedMatmulV4CopsHip : public KernelMod {
 public:
  // Resize = the reference's GetWorkSpaceInfo (grouped_matmul_v4_cops.cc:101-137): recover the lists and the trailing
  // scalars (the inputs arrive as twelve list slots followed by the scalars), plan every backend launch of the call and
  // return one workspace size per launch.  Only shapes, dtypes and scalars are kept: Launch reads the tensors it is
  // given, as the reference's does (:85-96).
  std::vector<size_t> Resize(const KernelTensorList &inputs, const std::vector<ms::Tensor> &outputs) override {
    group_info_ = FetchGroupInfo(inputs);
    start_idxs_ = ComputeStartIdxsFromGroupInfo(group_info_);
    std::vector<size_t> sizes;
    void *stream = CurrentStream();
    for (const OneLaunch &one : BuildLaunches(ArgsFromGraphInputs(inputs), outputs)) {
      sizes.push_back(GmmPlanCache::GetInstance().GetOrCreate(kBackendOpName, one.desc, one.problem, stream)->workspace_bytes);
      if (one.int4_bytes > 0) sizes.push_back(2 * one.int4_bytes);   // 4-bit weights widened to int8: one more slice
    }
    return sizes;
  }

  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &workspace, const std::vector<ms::Tensor> &outputs,
              void *stream) override {
    std::vector<OneLaunch> launches = BuildLaunches(ArgsFromGraphInputs(inputs), outputs);
    size_t slot = 0;   // workspace slices in Resize's order: per launch the plan's, then the widened weights if any
    for (size_t li = 0; li < launches.size(); ++li) {
      // the plan of the stream this launch goes to (a cache hit unless the stream changed since Resize)
      auto plan = GmmPlanCache::GetInstance().GetOrCreate(kBackendOpName, launches[li].desc, launches[li].problem, stream);
      const size_t i = slot++;
      if (launches[li].int4_bytes > 0) {
        const size_t w_slot = slot++;
        if (w_slot >= workspace.size() || workspace[w_slot].nbytes() < 2 * launches[li].int4_bytes) {
          MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", Launch got no workspace for the widened 4-bit weights of launch "
                           << li << ": Resize must run when shapes change.";
        }
        WidenInt4(launches[li], workspace[w_slot].GetDataPtr(), stream);
      }
      const bool have = i < workspace.size() && workspace[i].is_defined();
      if (plan->workspace_bytes > 0 && (!have || workspace[i].nbytes() < plan->workspace_bytes)) {
        MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName << ", Launch got no workspace of " << plan->workspace_bytes
                         << " bytes for launch " << li << ": Resize must run when shapes change.";
      }
      LaunchPlan(kBackendOpName, plan, launches[li].addrs, launches[li].out, have ? workspace[i].GetDataPtr() : nullptr,
                 have ? workspace[i].nbytes() : 0, stream);
    }
    return true;
  }

  const std::vector<int64_t> &start_idxs() const { return start_idxs_; }

 private:
  std::vector<int64_t> group_info_{};
  std::vector<int64_t> start_idxs_{};
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(grouped_matmul_v4_cops, ms_custom_ops::GroupedMatmulV4CopsFuncImpl,
                  ms_custom_ops::GroupedMatmulV4CopsHip);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
static TensorVec GetOptionalTensorList(const std::optional<TensorVec> &tensor_list) {
  return tensor_list.has_value() ? tensor_list.value() : TensorVec();
}

std::vector<ms::Tensor> grouped_matmul_v4_cops_custom(
  const TensorVec &x, const TensorVec &weight, const std::optional<TensorVec> &bias,
  const std::optional<TensorVec> &scale, const std::optional<TensorVec> &offset,
  const std::optional<TensorVec> &antiquant_scale, const std::optional<TensorVec> &antiquant_offset,
  const std::optional<TensorVec> &per_token_scale, const std::optional<ms::Tensor> &group_list,
  const std::optional<TensorVec> &activation_input, const std::optional<TensorVec> &activation_quant_scale,
  const std::optional<TensorVec> &activation_quant_offset, const int64_t &split_item, const int64_t &group_type,
  const int64_t &group_list_type, const int64_t &act_type, const std::string &weight_format,
  const std::optional<int64_t> &output_dtype) {
  auto output_types = InferOutputTypes(x, weight, scale, output_dtype);
  auto output_shapes = InferOutputShapes(x, weight, group_list, group_type, weight_format);
  if (output_types.size() != output_shapes.size()) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                       << ", the number of output types must be equal to the number of output shapes, "
                       << "but got output types size: " << output_types.size()
                       << ", output shapes size: " << output_shapes.size();
  }
  V4Args args;
  args.x = x;
  args.weight = weight;
  args.bias = GetOptionalTensorList(bias);
  args.scale = GetOptionalTensorList(scale);
  args.offset = GetOptionalTensorList(offset);
  args.antiquant_scale = GetOptionalTensorList(antiquant_scale);
  args.antiquant_offset = GetOptionalTensorList(antiquant_offset);
  args.per_token_scale = GetOptionalTensorList(per_token_scale);
  args.group_list = GetTensorOrEmpty(group_list);
  args.activation_input = GetOptionalTensorList(activation_input);
  args.activation_quant_scale = GetOptionalTensorList(activation_quant_scale);
  args.activation_quant_offset = GetOptionalTensorList(activation_quant_offset);
  args.split_item = split_item;
  args.group_type = group_type;
  args.group_list_type = group_list_type;
  args.act_type = act_type;
  args.weight_format = weight_format;
  CheckV4Support(args);
  if (output_types[0] == kNumberTypeInt8) {
    MS_LOG_EXCEPTION << "For " << kGroupedMatmulV4CopsName
                     << ", uint64 scales with int8 output are not implemented by the HIP backend.";
  }
  std::vector<ms::Tensor> outputs;
  for (size_t i = 0; i < output_types.size(); i++) outputs.push_back(AllocateTensor(output_types[i], output_shapes[i]));
  RunGroupedMatmulV4(args, outputs);
  return outputs;
}
}  // namespace ms_custom_ops

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("grouped_matmul_v4_cops", &ms_custom_ops::grouped_matmul_v4_cops_custom, "GroupedMatmulV4", pybind11::arg("x"),
        pybind11::arg("weight"), pybind11::arg("bias") = std::nullopt, pybind11::arg("scale") = std::nullopt,
        pybind11::arg("offset") = std::nullopt, pybind11::arg("antiquant_scale") = std::nullopt,
        pybind11::arg("antiquant_offset") = std::nullopt, pybind11::arg("per_token_scale") = std::nullopt,
        pybind11::arg("group_list") = std::nullopt, pybind11::arg("activation_input") = std::nullopt,
        pybind11::arg("activation_quant_scale") = std::nullopt, pybind11::arg("activation_quant_offset") = std::nullopt,
        pybind11::arg("split_item") = 0, pybind11::arg("group_type") = -1, pybind11::arg("group_list_type") = 0,
        pybind11::arg("act_type") = 0, pybind11::arg("weight_format") = std::string("ND"),
        pybind11::arg("output_dtype") = std::nullopt);
}
