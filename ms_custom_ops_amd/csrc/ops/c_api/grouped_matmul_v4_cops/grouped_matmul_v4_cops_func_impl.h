// Shape / dtype inference of grouped_matmul_v4_cops, shared by the graph-mode func impl and the
// pynative entry (reference: ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops_func_impl.cc:71-236
// and grouped_matmul_v4_cops.cc:162-245).
#ifndef MS_CUSTOM_OPS_OPS_C_API_GROUPED_MATMUL_V4_COPS_FUNC_IMPL_H_
#define MS_CUSTOM_OPS_OPS_C_API_GROUPED_MATMUL_V4_COPS_FUNC_IMPL_H_

#include <string>
#include <optional>
#include <vector>

#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
constexpr auto kGroupedMatmulV4CopsName = "grouped_matmul_v4_cops";
constexpr size_t kListTensorInputNums = 12;
constexpr size_t kXIndex = 0;
constexpr size_t kWeightIndex = 1;
constexpr size_t kBiasIndex = 2;
constexpr size_t kScaleIndex = 3;
constexpr size_t kOffsetIndex = 4;
constexpr size_t kAntiquantScaleIndex = 5;
constexpr size_t kAntiquantOffsetIndex = 6;
constexpr size_t kPerTokenScaleIndex = 7;
constexpr size_t kGroupListIndex = 8;
constexpr size_t kActivationInputIndex = 9;
constexpr size_t kSplitItemIndex = 12;
constexpr size_t kGroupTypeIndex = 13;
constexpr size_t kGroupListTypeIndex = 14;
constexpr size_t kActTypeIndex = 15;
constexpr size_t kWeightFormatIndex = 16;
constexpr size_t kOutDtypeIndex = 17;
constexpr int64_t kGroupTypeMultiOutput = -1;
constexpr int64_t kGroupTypeSingleOutput = 0;

using TensorVec = std::vector<ms::Tensor>;

TypeIdList InferOutputTypes(const TensorVec &x, const TensorVec &weight, const std::optional<TensorVec> &scale,
                            const std::optional<int64_t> &output_dtype);
ShapeArray InferOutputShapes(const TensorVec &x, const TensorVec &weight, const std::optional<ms::Tensor> &group_list,
                             const int64_t &group_type, const std::string &weight_format = "ND");

// Graph mode sees the twelve list inputs flattened into one positional list; group_info[i] is the
// length of list i (0 = None, which still occupies one slot), as the reference's tuple-unfolding
// pass and FetchGroupInfo arrange it (grouped_matmul_v4_cops_func_impl.cc:30-53,
// pass/convert_tuple_input_to_dynamic_input/convert_tuple_input_to_dynamic_input.cc:29-45).
std::vector<int64_t> FetchGroupInfo(const KernelTensorList &inputs);
std::vector<int64_t> ComputeStartIdxsFromGroupInfo(const std::vector<int64_t> &group_info);

class GroupedMatmulV4CopsFuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override;
  TypeIdList InferType(const KernelTensorList &inputs) const override;
};
}  // namespace ms_custom_ops
#endif  // MS_CUSTOM_OPS_OPS_C_API_GROUPED_MATMUL_V4_COPS_FUNC_IMPL_H_
