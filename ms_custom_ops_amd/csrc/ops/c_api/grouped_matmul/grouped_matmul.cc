// grouped_matmul(x, weight, group_list, bias, scale, per_token_scale, antiquant_scale,
//                transpose_a, transpose_b, x_format)
//
// Operator entry of the reference (ops/c_api/grouped_matmul/grouped_matmul.cc): same argument
// order and defaults (:327-332), the same shape / dtype rules and messages (:53-114, :146-190) and
// the same two execution paths (graph-mode kernel module :195-241, pynative runner :253-314).
// The kernel object behind it is the gfx950 HIP backend instead of CreateGroupedMatmulOp.
//
// Differences, all on the side of doing less or saying so:
//   * only the quantized path (int8 x and weight) exists on this backend; float16 x raises;
//   * weights are consumed as stored ([E,K,N], or [E,N,K] with transpose_b), or prepacked by trans_data into the
//     backend's blocked layout ([E, N/16, ceil(K/64), 1024] int8) -- the counterpart of the reference's FRACTAL_NZ
//     pre-pass, and x_format = 1 raises;
//   * `output_dtype` is an extra, trailing, optional argument: None keeps the reference's float16
//     output, bfloat16 selects the bf16 epilogue.
#include <algorithm>
#include <optional>
#include <string>
#include <vector>

#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
enum class GroupedMatmulInputIndex : size_t {
  kGmmXIndex = 0,
  kGmmWeightIndex,
  kGmmGroupListIndex,
  kGmmBiasIndex,
  kGmmScaleIndex,
  kGmmPerTokenScaleIndex,
  kGmmAntiquantScaleIndex,
  kGmmTransposeAIndex,
  kGmmTransposeBIndex,
  kGmmXFormatIndex,
  kGmmOutputDtypeIndex,
  kGmmInputsNum,
};
static constexpr size_t I(GroupedMatmulInputIndex i) { return static_cast<size_t>(i); }

// =============================================================================
// SHAPE / TYPE RULES (shared by both modes)
// =============================================================================
void CheckInputRank(const ShapeVector &x_shape, const ShapeVector &weight_shape, const ShapeVector &group_list_shape) {
  if (x_shape.size() != kDim2) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'x' must be 2D, but got:" << x_shape.size();
  }
  if (weight_shape.size() != kDim3 && !IsPackedWeightShape(weight_shape, kDim4)) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'weight' must be 3D, but got:" << weight_shape.size();
  }
  if (group_list_shape.size() != kDim1) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'group_list' must be 1D, but got:" << group_list_shape.size();
  }
}

ShapeVector InferGroupedMatmulOutputShape(const ShapeVector &x_shape, const ShapeVector &weight_shape,
                                          const ShapeVector &group_list_shape, bool transpose_a, bool transpose_b,
                                          TypeId x_dtype) {
  CheckInputRank(x_shape, weight_shape, group_list_shape);
  const int64_t m = transpose_a ? x_shape[kIndex1] : x_shape[kIndex0];
  const int64_t k = transpose_a ? x_shape[kIndex0] : x_shape[kIndex1];
  const int64_t e = weight_shape[kIndex0];
  const bool packed = IsPackedWeightShape(weight_shape, kDim4);   // [E, N / 16, ceil(K / 64), 1024] from trans_data
  if (packed && transpose_b) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, a weight prepacked by trans_data carries its own layout; 'transpose_b' must "
                        "be false.";
  }
  const int64_t n = packed ? weight_shape[kIndex1] * 16 : (transpose_b ? weight_shape[kIndex1] : weight_shape[kIndex2]);
  const int64_t wk = packed ? (weight_shape[kIndex2] == (k + 63) / 64 ? k : weight_shape[kIndex2] * 64)
                            : (transpose_b ? weight_shape[kIndex2] : weight_shape[kIndex1]);
  if (k != wk) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'x' and 'weight' must have the same dimension of 'k', but got:" << k
                     << " and " << wk;
  }
  const int64_t k_align = (x_dtype == kNumberTypeFloat16) ? 16 : 32;
  if (k % k_align != 0) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'x' K dimension must be aligned to " << k_align << " for "
                     << (x_dtype == kNumberTypeFloat16 ? "float16" : "int8") << " input, but got: " << k;
  }
  if (n % 16 != 0) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'weight' N dimension must be aligned to 16, but got: " << n;
  }
  if (e % 8 != 0) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'weight' E dimension (group count) must be aligned to 8, but got: "
                     << e;
  }
  if (group_list_shape[kIndex0] != e) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'group_list' must have one entry per group, but got:"
                     << group_list_shape[kIndex0] << " for " << e << " groups";
  }
  return ShapeVector{m, n};
}

static void CheckOptionalDtype(TypeId actual, bool is_none, const std::vector<TypeId> &expected,
                               const std::string &input_name) {
  if (is_none) return;
  if (std::find(expected.begin(), expected.end(), actual) != expected.end()) return;
  ExceptionStream s(ExceptionStream::kRuntime);
  s << "For GroupedMatmul, input '" << input_name << "' must be one of [";
  for (size_t i = 0; i < expected.size(); ++i) s << (i ? ", " : "") << expected[i];
  s << "], but got:" << actual;
  s.Throw();
}

TypeId InferGroupedMatmulOutputType(TypeId x_dtype, TypeId weight_dtype, TypeId group_list_dtype, TypeId bias_dtype,
                                    bool bias_none, TypeId scale_dtype, bool scale_none, TypeId pts_dtype,
                                    bool pts_none, TypeId aq_dtype, bool aq_none,
                                    const std::optional<int64_t> &output_dtype) {
  if (x_dtype != kNumberTypeFloat16 && x_dtype != kNumberTypeInt8) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'x' must be float16 or int8, but got:" << x_dtype;
  }
  if (weight_dtype != x_dtype) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'weight' must be the same type as 'x', but got:" << weight_dtype;
  }
  if (group_list_dtype != kNumberTypeInt32) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'group_list' must be int32, but got:" << group_list_dtype;
  }
  CheckOptionalDtype(bias_dtype, bias_none, {kNumberTypeFloat16, kNumberTypeInt32}, "bias");
  CheckOptionalDtype(scale_dtype, scale_none, {kNumberTypeInt64, kNumberTypeUInt64, kNumberTypeFloat32}, "scale");
  CheckOptionalDtype(pts_dtype, pts_none, {kNumberTypeFloat32}, "per_token_scale");
  CheckOptionalDtype(aq_dtype, aq_none, {kNumberTypeFloat16, kNumberTypeFloat32}, "antiquant_scale");
  TypeId out = kNumberTypeFloat16;  // the reference's only output type (grouped_matmul.cc:188)
  if (output_dtype.has_value()) {
    out = static_cast<TypeId>(output_dtype.value());
    if (out != kNumberTypeFloat16 && out != kNumberTypeBFloat16) {
      MS_EXCEPTION_VALUE << "For GroupedMatmul, 'output_dtype' must be Float16 or BFloat16, but got " << out;
    }
  }
  return out;
}

// What this backend does not implement is refused up front with a precise message.
static void CheckBackendSupport(TypeId x_dtype, bool has_scale, bool has_antiquant, TypeId bias_dtype, bool bias_none,
                                int64_t x_format) {
  if (x_dtype != kNumberTypeInt8) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, the HIP backend implements the quantized int8 path only, but got x dtype:"
                     << x_dtype;
  }
  if (!has_scale) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, the quantized path needs the dequant 'scale' input.";
  }
  if (has_antiquant) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, 'antiquant_scale' ([E,K,1] weight antiquant) is not implemented by the "
                        "HIP backend; use grouped_matmul_v4_cops for weight-only quantization.";
  }
  if (!bias_none && bias_dtype != kNumberTypeInt32) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, the quantized path takes an int32 'bias', but got:" << bias_dtype;
  }
  if (x_format != static_cast<int64_t>(DataFormat::ND)) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, x_format must be 0 (ND) on the HIP backend, but got:" << x_format;
  }
}

static msco_gmm_desc MakeGroupedMatmulDesc(const TensorList &in, TypeId out_dtype, bool transpose_b) {
  msco_gmm_desc d{};
  d.abi_version = MSCO_GMM_ABI_VERSION;
  d.x_dtype = ToBackendDtype(in[MSCO_IN_X].data_type());
  d.weight_dtype = ToBackendDtype(in[MSCO_IN_WEIGHT].data_type());
  d.out_dtype = ToBackendDtype(out_dtype);
  d.group_list_dtype = ToBackendDtype(in[MSCO_IN_GROUP_LIST].data_type());
  d.group_list_type = 0;  // cumulative row ends (grouped_matmul_doc.md: "每组样本数量累加")
  d.bias_dtype = in[MSCO_IN_BIAS].is_defined() ? ToBackendDtype(in[MSCO_IN_BIAS].data_type()) : MSCO_DT_NONE;
  d.scale_dtype = in[MSCO_IN_SCALE].is_defined() ? ToBackendDtype(in[MSCO_IN_SCALE].data_type()) : MSCO_DT_NONE;
  d.per_token_dtype = in[MSCO_IN_PER_TOKEN_SCALE].is_defined() ? MSCO_DT_F32 : MSCO_DT_NONE;
  d.transpose_b = transpose_b ? 1 : 0;
  d.weight_layout = IsPackedWeightShape(in[MSCO_IN_WEIGHT].shape(), kDim4) ? MSCO_WL_PACKED : MSCO_WL_ROW_MAJOR;
  d.scale_per_group = 1;
  return d;
}

static GmmProblem MakeGroupedMatmulProblem(const TensorList &in, bool transpose_b) {
  const auto &xs = in[MSCO_IN_X].shape();
  const auto &ws = in[MSCO_IN_WEIGHT].shape();
  if (IsPackedWeightShape(ws, kDim4)) return GmmProblem{xs[0], xs[1], ws[1] * 16, ws[0]};
  return GmmProblem{xs[0], xs[1], transpose_b ? ws[1] : ws[2], ws[0]};
}

static void CheckOptionalShapes(const TensorList &in, int64_t m, int64_t n, int64_t e) {
  auto check_en = [&](const ms::Tensor &t, const char *name) {
    if (!t.is_defined()) return;
    if (t.numel() != e * n) {
      MS_LOG_EXCEPTION << "For GroupedMatmul, input '" << name << "' must have shape [E, N] = [" << e << ", " << n
                       << "], but got:" << t.shape();
    }
  };
  check_en(in[MSCO_IN_BIAS], "bias");
  check_en(in[MSCO_IN_SCALE], "scale");
  if (in[MSCO_IN_PER_TOKEN_SCALE].is_defined() && in[MSCO_IN_PER_TOKEN_SCALE].numel() != m) {
    MS_LOG_EXCEPTION << "For GroupedMatmul, input 'per_token_scale' must have shape [M] or [M, 1] with M = " << m
                     << ", but got:" << in[MSCO_IN_PER_TOKEN_SCALE].shape();
  }
}

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
static std::optional<int64_t> GetOutputDtypeArg(const KernelTensorList &inputs) {
  if (inputs.size() <= I(GroupedMatmulInputIndex::kGmmOutputDtypeIndex)) return std::nullopt;
  const auto &kt = inputs[I(GroupedMatmulInputIndex::kGmmOutputDtypeIndex)];
  if (kt.IsNone()) return std::nullopt;
  return kt.GetValueWithCheck<int64_t>();
}

class CustomGroupedMatmulOpFuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override {
    if (inputs.size() < I(GroupedMatmulInputIndex::kGmmXFormatIndex) + 1) {
      MS_LOG_EXCEPTION << "For GroupedMatmul, input size must be " << I(GroupedMatmulInputIndex::kGmmXFormatIndex) + 1
                       << ", but got " << inputs.size();
    }
    const auto &x = inputs[I(GroupedMatmulInputIndex::kGmmXIndex)];
    const auto &w = inputs[I(GroupedMatmulInputIndex::kGmmWeightIndex)];
    const auto &gl = inputs[I(GroupedMatmulInputIndex::kGmmGroupListIndex)];
    const bool ta = inputs[I(GroupedMatmulInputIndex::kGmmTransposeAIndex)].GetValueWithCheck<bool>();
    const bool tb = inputs[I(GroupedMatmulInputIndex::kGmmTransposeBIndex)].GetValueWithCheck<bool>();
    return {InferGroupedMatmulOutputShape(x.GetShape(), w.GetShape(), gl.GetShape(), ta, tb, x.GetType())};
  }

  TypeIdList InferType(const KernelTensorList &inputs) const override {
    auto at = [&](GroupedMatmulInputIndex i) -> const KernelTensor & { return inputs[I(i)]; };
    return {InferGroupedMatmulOutputType(
      at(GroupedMatmulInputIndex::kGmmXIndex).GetType(), at(GroupedMatmulInputIndex::kGmmWeightIndex).GetType(),
      at(GroupedMatmulInputIndex::kGmmGroupListIndex).GetType(), at(GroupedMatmulInputIndex::kGmmBiasIndex).GetType(),
      at(GroupedMatmulInputIndex::kGmmBiasIndex).IsNone(), at(GroupedMatmulInputIndex::kGmmScaleIndex).GetType(),
      at(GroupedMatmulInputIndex::kGmmScaleIndex).IsNone(),
      at(GroupedMatmulInputIndex::kGmmPerTokenScaleIndex).GetType(),
      at(GroupedMatmulInputIndex::kGmmPerTokenScaleIndex).IsNone(),
      at(GroupedMatmulInputIndex::kGmmAntiquantScaleIndex).GetType(),
      at(GroupedMatmulInputIndex::kGmmAntiquantScaleIndex).IsNone(), GetOutputDtypeArg(inputs))};
  }
};

class CustomGroupedMatmul : public HipGmmKernelMod {
 public:
  CustomGroupedMatmul() : HipGmmKernelMod("GroupedMatmul") {}

 protected:
  // backend order {x, weight, bias, scale, group_list, per_token_scale, antiquant_scale}, the order
  // the reference hands to its kernel object (grouped_matmul.cc:201-207)
  // transpose_a (ops/c_api/grouped_matmul/grouped_matmul.cc:73-74,216-218 of the reference): x arrives [K, M].  The
  // kernels read K-contiguous rows, so Launch turns it into [M, K] in a workspace slice of its own; here x is
  // presented with the shape it will have then.
  TensorList GetBackendInputs(const KernelTensorList &inputs) override {
    auto t = [&](GroupedMatmulInputIndex i) { return inputs[I(i)].tensor; };
    ms::Tensor x = t(GroupedMatmulInputIndex::kGmmXIndex);
    transpose_x_ = inputs[I(GroupedMatmulInputIndex::kGmmTransposeAIndex)].GetValueWithCheck<bool>();
    if (transpose_x_) {
      CheckContiguous(kernel_name_, {x}, true);
      x = x.Slice(0, ShapeVector{x.shape()[kIndex1], x.shape()[kIndex0]});
    }
    return {x,          t(GroupedMatmulInputIndex::kGmmWeightIndex),
            t(GroupedMatmulInputIndex::kGmmBiasIndex),       t(GroupedMatmulInputIndex::kGmmScaleIndex),
            t(GroupedMatmulInputIndex::kGmmGroupListIndex),  t(GroupedMatmulInputIndex::kGmmPerTokenScaleIndex),
            t(GroupedMatmulInputIndex::kGmmAntiquantScaleIndex), ms::Tensor()};
  }

  msco_gmm_desc CreateKernel(const KernelTensorList &inputs, const TensorList &in,
                             const std::vector<ms::Tensor> &outputs) override {
    const bool tb = inputs[I(GroupedMatmulInputIndex::kGmmTransposeBIndex)].GetValueWithCheck<bool>();
    const int64_t x_format = inputs[I(GroupedMatmulInputIndex::kGmmXFormatIndex)].GetValueWithCheck<int64_t>();
    CheckBackendSupport(in[MSCO_IN_X].data_type(), in[MSCO_IN_SCALE].is_defined(),
                        in[MSCO_IN_ANTIQUANT_SCALE].is_defined(), in[MSCO_IN_BIAS].data_type(),
                        !in[MSCO_IN_BIAS].is_defined(), x_format);
    const GmmProblem pb = MakeGroupedMatmulProblem(in, tb);
    CheckOptionalShapes(in, pb.m, pb.n, pb.e);
    return MakeGroupedMatmulDesc(in, outputs.at(0).data_type(), tb);
  }

  GmmProblem GetProblem(const KernelTensorList &inputs, const TensorList &in,
                        const std::vector<ms::Tensor> &) override {
    return MakeGroupedMatmulProblem(in, inputs[I(GroupedMatmulInputIndex::kGmmTransposeBIndex)].GetValueWithCheck<bool>());
  }
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(grouped_matmul, ms_custom_ops::CustomGroupedMatmulOpFuncImpl, ms_custom_ops::CustomGroupedMatmul);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
class GroupedMatmulRunner : public HipGmmPyboostRunner {
 public:
  using HipGmmPyboostRunner::HipGmmPyboostRunner;
  void SetParam(const bool &transpose_a, const bool &transpose_b, const bool &with_bias) {
    transpose_a_ = transpose_a;
    transpose_b_ = transpose_b;
    with_bias_ = with_bias;
  }
  void SetXFormat(const DataFormat &x_format) { x_format_ = x_format; }

 protected:
  msco_gmm_desc CreateKernel(const TensorList &in, const TensorList &outputs) override {
    CheckBackendSupport(in[MSCO_IN_X].data_type(), in[MSCO_IN_SCALE].is_defined(),
                        in[MSCO_IN_ANTIQUANT_SCALE].is_defined(), in[MSCO_IN_BIAS].data_type(), !with_bias_,
                        static_cast<int64_t>(x_format_));
    const GmmProblem pb = MakeGroupedMatmulProblem(in, transpose_b_);
    CheckOptionalShapes(in, pb.m, pb.n, pb.e);
    return MakeGroupedMatmulDesc(in, outputs.at(0).data_type(), transpose_b_);
  }
  GmmProblem GetProblem(const TensorList &in, const TensorList &) override {
    return MakeGroupedMatmulProblem(in, transpose_b_);
  }

 private:
  bool transpose_a_{false};
  bool transpose_b_{false};
  bool with_bias_{false};
  DataFormat x_format_{DataFormat::ND};
};

std::vector<ms::Tensor> hip_grouped_matmul(const ms::Tensor &x, const ms::Tensor &weight, const ms::Tensor &group_list,
                                           const std::optional<ms::Tensor> &bias,
                                           const std::optional<ms::Tensor> &scale,
                                           const std::optional<ms::Tensor> &per_token_scale,
                                           const std::optional<ms::Tensor> &antiquant_scale, const bool &transpose_a,
                                           const bool &transpose_b, const int &x_format,
                                           const std::optional<int64_t> &output_dtype) {
  auto op_name = "GroupedMatmul";
  auto runner = std::make_shared<GroupedMatmulRunner>(op_name);
  runner->SetParam(transpose_a, transpose_b, bias.has_value());
  runner->SetXFormat(static_cast<DataFormat>(x_format));

  auto out_shape = InferGroupedMatmulOutputShape(x.shape(), weight.shape(), group_list.shape(), transpose_a,
                                                 transpose_b, x.data_type());
  // transpose_a: x arrives [K, M]; the kernels read K-contiguous rows, so it is turned into [M, K] once
  ms::Tensor x_rows = x;
  if (transpose_a && x.data_type() == kNumberTypeInt8) {
    CheckContiguous(op_name, {x}, true);
    const int64_t k = x.shape()[kIndex0], m = x.shape()[kIndex1];
    x_rows = AllocateTensor(kNumberTypeInt8, ShapeVector{m, k});
    if (m > 0 && k > 0) {
      const int rc = msco_transpose_2d(x.GetDataPtr(), x_rows.GetDataPtr(), 1, k, m, 1, CurrentStream());
      if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << op_name << ", transposing x failed: " << msco_status_string(rc);
    }
  }
  std::vector<ms::Tensor> inputs = {x_rows,
                                    weight,
                                    GetTensorOrEmpty(bias),
                                    GetTensorOrEmpty(scale),
                                    group_list,
                                    GetTensorOrEmpty(per_token_scale),
                                    GetTensorOrEmpty(antiquant_scale),
                                    ms::Tensor()};
  auto out_type = InferGroupedMatmulOutputType(
    x.data_type(), weight.data_type(), group_list.data_type(), inputs[MSCO_IN_BIAS].data_type(), !bias.has_value(),
    inputs[MSCO_IN_SCALE].data_type(), !scale.has_value(), inputs[MSCO_IN_PER_TOKEN_SCALE].data_type(),
    !per_token_scale.has_value(), inputs[MSCO_IN_ANTIQUANT_SCALE].data_type(), !antiquant_scale.has_value(),
    output_dtype);
  std::vector<ms::Tensor> outputs = {AllocateTensor(out_type, out_shape)};
  runner->GetOrCreateKernel(inputs, outputs);
  runner->Run(inputs, outputs);
  return outputs;
}
}  // namespace ms_custom_ops

auto pyboost_grouped_matmul(const ms::Tensor &x, const ms::Tensor &weight, const ms::Tensor &group_list,
                            const std::optional<ms::Tensor> &bias, const std::optional<ms::Tensor> &scale,
                            const std::optional<ms::Tensor> &per_token_scale,
                            const std::optional<ms::Tensor> &antiquant_scale, const bool &transpose_a,
                            const bool &transpose_b, const int &x_format, const std::optional<int64_t> &output_dtype) {
  return ms_custom_ops::hip_grouped_matmul(x, weight, group_list, bias, scale, per_token_scale, antiquant_scale,
                                           transpose_a, transpose_b, x_format, output_dtype)[0];
}

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("grouped_matmul", &pyboost_grouped_matmul, "GroupedMatmul", pybind11::arg("x"), pybind11::arg("weight"),
        pybind11::arg("group_list"), pybind11::arg("bias") = std::nullopt, pybind11::arg("scale") = std::nullopt,
        pybind11::arg("per_token_scale") = std::nullopt, pybind11::arg("antiquant_scale") = std::nullopt,
        pybind11::arg("transpose_a") = false, pybind11::arg("transpose_b") = false, pybind11::arg("x_format") = 0,
        pybind11::arg("output_dtype") = std::nullopt);
}
