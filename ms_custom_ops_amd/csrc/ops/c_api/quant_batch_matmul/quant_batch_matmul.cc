// quant_batch_matmul(x1, x2, scale, offset, bias, pertoken_scale, transpose_x1, transpose_x2,
//                    x2_format, output_dtype)
//
// Dense / batched W8A8 entry of the reference (ops/c_api/quant_batch_matmul/quant_batch_matmul.cc):
// same arguments and defaults (:162-168, output_dtype defaults to float16 == 42), output shape by
// BatchMatMulMakeShape (:44-56), output dtype from `output_dtype` (:57-64).  The reference forwards
// to aclnnQuantMatmulV4 (:144-145); here the dense problem is the single-group (or equal-group)
// case of the grouped HIP kernel.
//
// Not implemented on this backend and refused with a message: `offset`, int8 output, FRACTAL_NZ x2.
#include <optional>
#include <string>
#include <vector>

#include "ops/c_api/utils/common_utils.h"
#include "ops/framework/hip_backend/hip_gmm_runner.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
constexpr size_t kQbmmMatSize = 2;
constexpr size_t kQbmmInputX1 = 0;
constexpr size_t kQbmmInputX2 = 1;
constexpr size_t kQbmmInputScale = 2;
constexpr size_t kQbmmInputOffset = 3;
constexpr size_t kQbmmInputBias = 4;
constexpr size_t kQbmmInputPertokenScaleOptional = 5;
constexpr size_t kQbmmInputTransposeX1 = 6;
constexpr size_t kQbmmInputTransposeX2 = 7;
constexpr size_t kQbmmInputX2Format = 8;
constexpr size_t kQbmmInputDtype = 9;
constexpr int64_t kFloat16 = 42;

// x2 as the shape rules see it.  With x2_format "FRACTAL_NZ" x2 is a weight prepacked by trans_data, int8
// [..., N / 16, ceil(K / 64), 1024]; its logical shape is [..., K, N] with K taken from x1.
static ShapeVector QbmmLogicalX2Shape(const ShapeVector &x1_shape, const ShapeVector &x2_shape, bool transpose_x1,
                                      bool transpose_x2, const std::string &x2_format) {
  if (x2_format != kFractalNzFormat) return x2_shape;
  if (x2_shape.size() < kDim3 || x2_shape.back() != kPackedBlockBytes || x1_shape.size() < kDim2) {
    MS_EXCEPTION_VALUE << "For quant_batch_matmul, x2_format 'FRACTAL_NZ' takes an x2 prepacked by trans_data "
                       << "([..., N/16, ceil(K/64), 1024]), but got " << x2_shape;
  }
  if (transpose_x2) {
    MS_EXCEPTION_VALUE << "For quant_batch_matmul, an x2 prepacked by trans_data carries its own layout; 'transpose_x2' "
                       << "must be false.";
  }
  const int64_t k = transpose_x1 ? x1_shape[x1_shape.size() - kDim2] : x1_shape.back();
  const int64_t kb = x2_shape[x2_shape.size() - kDim2];
  ShapeVector logical(x2_shape.begin(), x2_shape.end() - kDim3);
  logical.push_back(kb == (k + 63) / 64 ? k : kb * 64);   // a mismatch surfaces as the usual K error
  logical.push_back(x2_shape[x2_shape.size() - kDim3] * 16);
  return logical;
}

static void CheckQbmmInputs(const ms::Tensor &x1, const ms::Tensor &x2, const ms::Tensor &scale,
                            const ms::Tensor &offset, const ms::Tensor &bias, const ms::Tensor &pertoken,
                            const std::string &x2_format, TypeId out_dtype, const BatchMatMulDims &d) {
  if (x2_format != kNdFormat && x2_format != kFractalNzFormat) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, the 'x2_format' is only support ['ND', 'FRACTAL_NZ'], but got "
                     << x2_format;
  }
  if (x1.data_type() != kNumberTypeInt8 || x2.data_type() != kNumberTypeInt8) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, 'x1' and 'x2' must be int8, but got " << x1.data_type() << " and "
                     << x2.data_type();
  }
  if (offset.is_defined()) MS_LOG_EXCEPTION << "For quant_batch_matmul, 'offset' is not implemented by the HIP backend.";
  if (out_dtype != kNumberTypeFloat16 && out_dtype != kNumberTypeBFloat16 && out_dtype != kNumberTypeInt32) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, 'output_dtype' must be Float16, BFloat16 or Int32 on the HIP "
                        "backend, but got " << out_dtype;
  }
  const TypeId st = scale.data_type();
  if (st != kNumberTypeFloat32 && st != kNumberTypeInt64 && st != kNumberTypeUInt64 && st != kNumberTypeBFloat16) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, 'scale' must be Float32, BFloat16, Int64 or UInt64, but got " << st;
  }
  if (scale.numel() != 1 && scale.numel() != d.n) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, 'scale' must have 1 or N = " << d.n << " elements, but got "
                     << scale.shape();
  }
  if (bias.is_defined() && (bias.data_type() != kNumberTypeInt32 || bias.numel() != d.n)) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, 'bias' must be Int32 with N = " << d.n << " elements, but got "
                     << bias.data_type() << " " << bias.shape();
  }
  if (pertoken.is_defined() && (pertoken.data_type() != kNumberTypeFloat32 || pertoken.numel() != d.m)) {
    MS_LOG_EXCEPTION << "For quant_batch_matmul, 'pertoken_scale' must be Float32 with M = " << d.m
                     << " elements, but got " << pertoken.data_type() << " " << pertoken.shape();
  }
}

// One backend launch: x [rows, K], weight [e, K, N] (or [e, N, K]), e equal groups of rows / e.
static void LaunchDense(const std::string &op_name, const ms::Tensor &x, const ms::Tensor &w, const ms::Tensor &scale,
                        const ms::Tensor &bias, const ms::Tensor &pertoken, const ms::Tensor &out, int64_t rows,
                        int64_t k, int64_t n, int64_t e, bool transpose_x2, bool packed, void *stream) {
  msco_gmm_desc d{};
  d.abi_version = MSCO_GMM_ABI_VERSION;
  d.x_dtype = MSCO_DT_I8;
  d.weight_dtype = MSCO_DT_I8;
  d.out_dtype = ToBackendDtype(out.data_type());
  d.group_list_dtype = MSCO_DT_NONE;
  const bool raw = out.data_type() == kNumberTypeInt32;  // int32 output = accumulator + bias
  d.bias_dtype = bias.is_defined() ? MSCO_DT_I32 : MSCO_DT_NONE;
  d.scale_dtype = raw ? MSCO_DT_NONE : ToBackendDtype(scale.data_type());
  d.per_token_dtype = (!raw && pertoken.is_defined()) ? MSCO_DT_F32 : MSCO_DT_NONE;
  d.transpose_b = transpose_x2 ? 1 : 0;
  d.weight_layout = packed ? MSCO_WL_PACKED : MSCO_WL_ROW_MAJOR;
  d.scale_per_group = 0;
  d.scale_is_scalar = scale.numel() == 1 ? 1 : 0;
  auto plan = GmmPlanCache::GetInstance().GetOrCreate(op_name, d, GmmProblem{rows, k, n, e}, stream);
  ms::Tensor workspace;
  if (plan->workspace_bytes > 0) {
    workspace = AllocateTensor(kNumberTypeInt8, ShapeVector{static_cast<int64_t>(plan->workspace_bytes)});
  }
  const void *addrs[MSCO_IN_COUNT] = {nullptr};
  addrs[MSCO_IN_X] = x.GetDataPtr();
  addrs[MSCO_IN_WEIGHT] = w.GetDataPtr();
  addrs[MSCO_IN_BIAS] = bias.is_defined() ? bias.GetDataPtr() : nullptr;
  addrs[MSCO_IN_SCALE] = raw ? nullptr : scale.GetDataPtr();
  addrs[MSCO_IN_PER_TOKEN_SCALE] = d.per_token_dtype != MSCO_DT_NONE ? pertoken.GetDataPtr() : nullptr;
  LaunchPlan(op_name, plan, addrs, out.GetDataPtr(), workspace.is_defined() ? workspace.GetDataPtr() : nullptr,
             plan->workspace_bytes, stream);
}

// Core routine shared by the graph-mode kernel module and the pynative entry.
void RunQuantBatchMatmul(const ms::Tensor &x1_in, const ms::Tensor &x2, const ms::Tensor &scale,
                         const ms::Tensor &offset, const ms::Tensor &bias, const ms::Tensor &pertoken,
                         bool transpose_x1, bool transpose_x2, const std::string &x2_format, const ms::Tensor &out) {
  const std::string op_name = "QuantBatchMatmul";
  const bool packed = x2_format == kFractalNzFormat;
  const BatchMatMulDims d = BatchMatMulSplitDims(
    x1_in.shape(), QbmmLogicalX2Shape(x1_in.shape(), x2.shape(), transpose_x1, transpose_x2, x2_format), transpose_x1,
    transpose_x2, op_name);
  CheckQbmmInputs(x1_in, x2, scale, offset, bias, pertoken, x2_format, out.data_type(), d);
  CheckContiguous(op_name, {x1_in, x2, scale, bias, pertoken}, true);
  CheckContiguous(op_name, {out}, false);
  void *stream = CurrentStream();
  auto prod = [](const ShapeVector &v) {
    int64_t p = 1;
    for (auto x : v) p *= x;
    return p;
  };
  const int64_t b1 = prod(d.x1_batch), b2 = prod(d.x2_batch), bo = prod(d.batch);
  if (bo == 0 || d.m == 0) return;

  ms::Tensor x1 = x1_in;
  if (transpose_x1) {  // materialise x1 as [..., M, K] once; the kernels read K-contiguous rows
    x1 = AllocateTensor(kNumberTypeInt8, ShapeVector{b1, d.m, d.k});
    const int rc = msco_transpose_2d(x1_in.GetDataPtr(), x1.GetDataPtr(), b1, d.k, d.m, 1, stream);
    if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << op_name << ", transposing x1 failed: " << msco_status_string(rc);
  }
  const bool shared_rows = !pertoken.is_defined() || bo == 1;
  if (b2 == 1 && shared_rows) {
    // every batch of x1 multiplies the same x2: one dense problem with B*M rows
    LaunchDense(op_name, x1, x2, scale, bias, pertoken, out, b1 * d.m, d.k, d.n, 1, transpose_x2, packed, stream);
    return;
  }
  if (d.x1_batch == d.x2_batch && shared_rows) {
    // batch b of x1 meets batch b of x2: B equal groups
    LaunchDense(op_name, x1, x2, scale, bias, pertoken, out, bo * d.m, d.k, d.n, bo, transpose_x2, packed, stream);
    return;
  }
  // general broadcasting: one dense launch per output batch
  const size_t nb = d.batch.size();
  for (int64_t idx = 0; idx < bo; ++idx) {
    int64_t rem = idx, i1 = 0, i2 = 0, s1 = 1, s2 = 1;
    for (int64_t ax = static_cast<int64_t>(nb) - 1; ax >= 0; --ax) {
      const int64_t c = rem % d.batch[ax];
      rem /= d.batch[ax];
      if (d.x1_batch[ax] != 1) i1 += c * s1;
      if (d.x2_batch[ax] != 1) i2 += c * s2;
      s1 *= d.x1_batch[ax];
      s2 *= d.x2_batch[ax];
    }
    const int64_t x2_elems = packed ? (d.n / 16) * ((d.k + 63) / 64) * kPackedBlockBytes : d.k * d.n;   // one matrix of x2
    LaunchDense(op_name, x1.Slice(i1 * d.m * d.k, {d.m, d.k}),
                packed ? x2.Slice(i2 * x2_elems, {d.n / 16, (d.k + 63) / 64, kPackedBlockBytes}) : x2.Slice(i2 * x2_elems, {d.k, d.n}),
                scale, bias, pertoken, out.Slice(idx * d.m * d.n, {d.m, d.n}), d.m, d.k, d.n, 1, transpose_x2, packed, stream);
  }
}

// =============================================================================
// GRAPH MODE IMPLEMENTATION
// =============================================================================
class QuantBatchMatmulCustomOpFuncImpl : public OpFuncImpl {
 public:
  ShapeArray InferShape(const KernelTensorList &inputs) const override {
    const bool transpose_x1 = inputs[kQbmmInputTransposeX1].GetValueWithCheck<bool>();
    const bool transpose_x2 = inputs[kQbmmInputTransposeX2].GetValueWithCheck<bool>();
    const std::string x2_format = inputs[kQbmmInputX2Format].IsNone() ? std::string(kNdFormat)
                                                                      : inputs[kQbmmInputX2Format].GetValueWithCheck<std::string>();
    return {BatchMatMulMakeShape(inputs[kQbmmInputX1].GetShape(),
                                 QbmmLogicalX2Shape(inputs[kQbmmInputX1].GetShape(), inputs[kQbmmInputX2].GetShape(),
                                                    transpose_x1, transpose_x2, x2_format),
                                 transpose_x1, transpose_x2, kQbmmMatSize, "QuantBatchMatmul")};
  }
  TypeIdList InferType(const KernelTensorList &inputs) const override {
    TypeId output_type = kNumberTypeFloat16;
    if (inputs.size() > kQbmmInputDtype && !inputs[kQbmmInputDtype].IsNone()) {
      output_type = static_cast<TypeId>(inputs[kQbmmInputDtype].GetValueWithCheck<int64_t>());
    }
    return {output_type};
  }
};

class QuantBatchMatmulCustomHip : public KernelMod {
 public:
  std::vector<size_t> Resize(const KernelTensorList &inputs, const std::vector<ms::Tensor> &) override {
    transpose_x1_ = inputs[kQbmmInputTransposeX1].GetValueWithCheck<bool>();
    transpose_x2_ = inputs[kQbmmInputTransposeX2].GetValueWithCheck<bool>();
    x2_format_ = inputs[kQbmmInputX2Format].GetValueWithCheck<std::string>();
    return {};  // workspace is requested from the framework inside the launch routine
  }
  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &, const std::vector<ms::Tensor> &outputs,
              void *stream) override {
    LaunchStreamScope on_launch_stream(stream);   // the routine below enqueues on CurrentStream()
    RunQuantBatchMatmul(inputs[kQbmmInputX1].tensor, inputs[kQbmmInputX2].tensor, inputs[kQbmmInputScale].tensor,
                        inputs[kQbmmInputOffset].tensor, inputs[kQbmmInputBias].tensor,
                        inputs[kQbmmInputPertokenScaleOptional].tensor, transpose_x1_, transpose_x2_, x2_format_,
                        outputs.at(0));
    return true;
  }

 private:
  bool transpose_x1_{false};
  bool transpose_x2_{false};
  std::string x2_format_{"ND"};
};
}  // namespace ms_custom_ops

REG_GRAPH_MODE_OP(quant_batch_matmul, ms_custom_ops::QuantBatchMatmulCustomOpFuncImpl,
                  ms_custom_ops::QuantBatchMatmulCustomHip);

// =============================================================================
// PYBOOST MODE IMPLEMENTATION
// =============================================================================
namespace ms_custom_ops {
ms::Tensor quant_batch_matmul_custom(const ms::Tensor &x1, const ms::Tensor &x2, const ms::Tensor &scale,
                                     const std::optional<ms::Tensor> &offset, const std::optional<ms::Tensor> &bias,
                                     const std::optional<ms::Tensor> &pertoken_scale, bool transpose_x1,
                                     bool transpose_x2, const std::string &x2_format, const int64_t output_dtype) {
  auto output_shape =
    BatchMatMulMakeShape(x1.shape(), QbmmLogicalX2Shape(x1.shape(), x2.shape(), transpose_x1, transpose_x2, x2_format),
                         transpose_x1, transpose_x2, kQbmmMatSize, "QuantBatchMatmul");
  auto out = AllocateTensor(static_cast<TypeId>(output_dtype), output_shape);
  RunQuantBatchMatmul(x1, x2, scale, GetTensorOrEmpty(offset), GetTensorOrEmpty(bias),
                      GetTensorOrEmpty(pertoken_scale), transpose_x1, transpose_x2, x2_format, out);
  return out;
}
}  // namespace ms_custom_ops

MS_CUSTOM_OPS_EXTENSION_MODULE(m) {
  m.def("quant_batch_matmul", &ms_custom_ops::quant_batch_matmul_custom, "quant_batch_matmul", pybind11::arg("x1"),
        pybind11::arg("x2"), pybind11::arg("scale"), pybind11::arg("offset") = std::nullopt,
        pybind11::arg("bias") = std::nullopt, pybind11::arg("pertoken_scale") = std::nullopt,
        pybind11::arg("transpose_x1") = false, pybind11::arg("transpose_x2") = false, pybind11::arg("x2_format") = "ND",
        pybind11::arg("output_dtype") = ms_custom_ops::kFloat16);
}
