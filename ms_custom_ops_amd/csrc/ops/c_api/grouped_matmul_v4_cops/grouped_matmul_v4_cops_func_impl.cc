#include "ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops_func_impl.h"

#include <set>

namespace ms_custom_ops {
TypeIdList InferOutputTypes(const TensorVec &x, const TensorVec &weight, const std::optional<TensorVec> &scale,
                            const std::optional<int64_t> &output_dtype) {
  if (x.empty() || weight.empty()) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", 'x' and 'weight' must be provided.";
  }
  const TypeId x_type = x[0].data_type();
  const TypeId w_type = weight[0].data_type();
  TypeId out_type;
  if (x_type == kNumberTypeInt8 && w_type == kNumberTypeInt4) {
    out_type = kNumberTypeBFloat16;
    if (output_dtype.has_value()) {
      out_type = static_cast<TypeId>(output_dtype.value());
      if (out_type != kNumberTypeFloat16 && out_type != kNumberTypeBFloat16) {
        MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                           << " with A8W4, the output type must be in [Float16, BFloat16], but got " << out_type;
      }
    }
  } else if (!scale.has_value() || scale.value().empty()) {
    out_type = x_type == kNumberTypeInt8 ? kNumberTypeInt32 : x_type;
  } else {
    const TypeId scale_type = scale.value()[0].data_type();
    if (scale_type == kNumberTypeUInt64) {
      out_type = kNumberTypeInt8;
    } else if (scale_type == kNumberTypeBFloat16) {
      out_type = kNumberTypeBFloat16;
    } else if (scale_type == kNumberTypeFloat32) {
      out_type = kNumberTypeFloat16;
    } else {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                         << ", the scale only support Uint16, BFloat16 and Float32, but got " << scale_type;
    }
    // Backend extension: for W8A8 an explicit output_dtype of Float16 / BFloat16 wins over the
    // scale-dtype rule, so float32 scales can be combined with a bfloat16 result.
    if (x_type == kNumberTypeInt8 && w_type == kNumberTypeInt8 && output_dtype.has_value() &&
        scale_type != kNumberTypeUInt64) {
      const TypeId req = static_cast<TypeId>(output_dtype.value());
      if (req != kNumberTypeFloat16 && req != kNumberTypeBFloat16) {
        MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                           << ", the output type must be in [Float16, BFloat16], but got " << req;
      }
      out_type = req;
    }
  }
  return TypeIdList(x.size(), out_type);
}

ShapeArray InferOutputShapes(const TensorVec &x, const TensorVec &weight, const std::optional<ms::Tensor> &group_list,
                             const int64_t &group_type, const std::string &weight_format) {
  ShapeArray output_shapes;
  // FRACTAL_NZ on this backend: weights prepacked by trans_data, int8 [E, N / 16, ceil(K / 64), 1024] (no E for the
  // per-matrix form); N comes from the number of 16-column groups
  const bool packed = weight_format == kFractalNzFormat;
  auto n_of = [&](const ms::Tensor &w, size_t rank) -> int64_t {
    if (!packed) return w.shape().back();
    if (!IsPackedWeightShape(w.shape(), rank) || w.data_type() != kNumberTypeInt8) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", weight_format 'FRACTAL_NZ' takes Int8 weights "
                         << "prepacked by trans_data (last dimension 1024, rank " << rank << "), but got " << w.data_type()
                         << " " << w.shape();
    }
    return w.shape()[rank - kDim3] * 16;
  };
  if (group_type == kGroupTypeMultiOutput) {
    if (x.size() != weight.size()) {
      MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName
                         << ", when group_type is -1 and split_item is 0, x's size "
                         << "should be equal to weight, but got " << x.size() << " and " << weight.size();
    }
    for (size_t i = 0; i < x.size(); i++) {
      auto res_shape = x[i].shape();
      if (res_shape.empty() || weight[i].shape().empty()) {
        MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", 'x' and 'weight' must not be scalars.";
      }
      res_shape.back() = n_of(weight[i], kDim3);
      output_shapes.emplace_back(std::move(res_shape));
    }
    return output_shapes;
  }
  if (x.size() != kDim1 || weight.size() != kDim1) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", when split_item is 3. the size of x and weight should "
                       << "both be 1, but got x's size " << x.size() << ", and weight's size " << weight.size();
  }
  const auto &x_shape = x[0].shape();
  const auto &w_shape = weight[0].shape();
  if (x_shape.size() < kDim2 || w_shape.empty()) {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", 'x' must be at least 2D, but got " << x_shape;
  }
  const int64_t m = x_shape[x_shape.size() - kIndex2];
  int64_t n = n_of(weight[0], kDim4);
  if (weight[0].data_type() == kNumberTypeInt4) n <<= 1;
  const int64_t group_list_size = group_list.has_value() ? group_list.value().shape()[0] : 1;
  if (group_type == kGroupTypeSingleOutput) {
    output_shapes.push_back(ShapeVector{m, n});
  } else if (group_type == 1) {
    output_shapes.push_back(ShapeVector{group_list_size, m, n});
  } else {
    MS_EXCEPTION_VALUE << "For " << kGroupedMatmulV4CopsName << ", group_type must be -1, 0 or 1, but got "
                       << group_type;
  }
  return output_shapes;
}

std::vector<int64_t> FetchGroupInfo(const KernelTensorList &inputs) {
  std::vector<int64_t> sizes;
  for (size_t i = 0; i < kListTensorInputNums; i++) {
    if (i == kGroupListIndex) {
      sizes.push_back(1);
    } else if (inputs[i].IsNone()) {
      sizes.push_back(0);
    } else {
      sizes.push_back(static_cast<int64_t>(inputs[i].sequence.size()));
    }
  }
  return sizes;
}

std::vector<int64_t> ComputeStartIdxsFromGroupInfo(const std::vector<int64_t> &group_info) {
  std::vector<int64_t> start_idxs{0};
  int64_t end = 0;
  for (int64_t len : group_info) {
    end += (len == 0 ? 1 : len);
    start_idxs.push_back(end);
  }
  return start_idxs;
}

static std::optional<TensorVec> OptionalList(const KernelTensor &kt) {
  if (kt.IsNone()) return std::nullopt;
  return kt.sequence;
}

ShapeArray GroupedMatmulV4CopsFuncImpl::InferShape(const KernelTensorList &inputs) const {
  if (inputs.size() <= kOutDtypeIndex) {
    MS_LOG_EXCEPTION << "For '" << kGroupedMatmulV4CopsName << "', expected " << kOutDtypeIndex + 1
                     << " inputs, but got " << inputs.size();
  }
  for (size_t i = 0; i < kListTensorInputNums; ++i) {
    if (i != kGroupListIndex && !inputs[i].IsNone() && !inputs[i].IsSequence()) {
      MS_LOG_EXCEPTION << "For '" << kGroupedMatmulV4CopsName << "', input " << i << " must be a list of tensors.";
    }
  }
  const int64_t group_type = inputs[kGroupTypeIndex].GetValueWithCheck<int64_t>();
  std::optional<ms::Tensor> gl;
  if (!inputs[kGroupListIndex].IsNone()) {
    gl = inputs[kGroupListIndex].tensor;
    if (gl->shape().size() != kDim1) {
      MS_EXCEPTION_VALUE << "For '" << kGroupedMatmulV4CopsName << "', group_list's rank must be equal to 1, but got "
                         << gl->shape().size();
    }
  }
  const std::string weight_format =
    inputs[kWeightFormatIndex].IsNone() ? std::string(kNdFormat) : inputs[kWeightFormatIndex].GetValueWithCheck<std::string>();
  return InferOutputShapes(inputs[kXIndex].sequence, inputs[kWeightIndex].sequence, gl, group_type, weight_format);
}

TypeIdList GroupedMatmulV4CopsFuncImpl::InferType(const KernelTensorList &inputs) const {
  std::optional<int64_t> out_dtype;
  if (!inputs[kOutDtypeIndex].IsNone()) out_dtype = inputs[kOutDtypeIndex].GetValueWithCheck<int64_t>();
  return InferOutputTypes(inputs[kXIndex].sequence, inputs[kWeightIndex].sequence, OptionalList(inputs[kScaleIndex]),
                          out_dtype);
}
}  // namespace ms_custom_ops
