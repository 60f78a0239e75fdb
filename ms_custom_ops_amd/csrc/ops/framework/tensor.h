// Minimal tensor view and type ids for the operator layer.
//
// The reference's operator glue is written against MindSpore's ms::Tensor / TypeId
// (ops/framework/utils.h:24, ops/framework/module.h:24).  This backend has no MindSpore: a tensor is
// a device pointer plus dtype, shape and strides, handed over by the host framework (PyTorch-ROCm
// tensors are converted by the Python package), and `owner` keeps the framework object alive.
#ifndef MS_CUSTOM_OPS_FRAMEWORK_TENSOR_H_
#define MS_CUSTOM_OPS_FRAMEWORK_TENSOR_H_

#include <pybind11/pybind11.h>

#include <cstdint>
#include <numeric>
#include <optional>
#include <string>
#include <vector>

namespace mindspore {
// Numeric values follow MindSpore's TypeId so that integer dtype arguments keep their meaning
// (quant_batch_matmul's default output_dtype is 42 == float16, quant_batch_matmul.cc:161).
enum TypeId : int {
  kTypeUnknown = 0,
  kMetaTypeNone = 9,
  kNumberTypeBool = 30,
  kNumberTypeInt8 = 32,
  kNumberTypeInt16 = 33,
  kNumberTypeInt32 = 34,
  kNumberTypeInt64 = 35,
  kNumberTypeUInt8 = 37,
  kNumberTypeUInt16 = 38,
  kNumberTypeUInt32 = 39,
  kNumberTypeUInt64 = 40,
  kNumberTypeFloat16 = 42,
  kNumberTypeFloat32 = 43,
  kNumberTypeFloat64 = 44,
  kNumberTypeBFloat16 = 45,
  kNumberTypeInt4 = 50,
};
using ShapeVector = std::vector<int64_t>;
using ShapeArray = std::vector<ShapeVector>;
using TypeIdList = std::vector<TypeId>;

inline std::string TypeIdToString(TypeId t) {
  switch (t) {
    case kMetaTypeNone: return "None";
    case kNumberTypeBool: return "Bool";
    case kNumberTypeInt8: return "Int8";
    case kNumberTypeInt16: return "Int16";
    case kNumberTypeInt32: return "Int32";
    case kNumberTypeInt64: return "Int64";
    case kNumberTypeUInt8: return "UInt8";
    case kNumberTypeUInt64: return "UInt64";
    case kNumberTypeFloat16: return "Float16";
    case kNumberTypeFloat32: return "Float32";
    case kNumberTypeFloat64: return "Float64";
    case kNumberTypeBFloat16: return "BFloat16";
    case kNumberTypeInt4: return "Int4";
    default: return "TypeId(" + std::to_string(static_cast<int>(t)) + ")";
  }
}

inline size_t TypeIdSize(TypeId t) {
  switch (t) {
    case kNumberTypeBool: case kNumberTypeInt8: case kNumberTypeUInt8: return 1;
    case kNumberTypeInt4: return 1;   // qint4x2 storage: one byte per element of the stored shape (two 4-bit values)
    case kNumberTypeInt16: case kNumberTypeUInt16: case kNumberTypeFloat16: case kNumberTypeBFloat16: return 2;
    case kNumberTypeInt32: case kNumberTypeUInt32: case kNumberTypeFloat32: return 4;
    case kNumberTypeInt64: case kNumberTypeUInt64: case kNumberTypeFloat64: return 8;
    default: return 0;
  }
}
}  // namespace mindspore

namespace ms {
using mindspore::ShapeVector;
using mindspore::TypeId;

class Tensor {
 public:
  Tensor() = default;
  Tensor(uintptr_t data, int type_id, ShapeVector shape, ShapeVector strides, pybind11::object owner)
      : data_(reinterpret_cast<void *>(data)),
        dtype_(static_cast<TypeId>(type_id)),
        shape_(std::move(shape)),
        strides_(std::move(strides)),
        owner_(std::move(owner)),
        defined_(true) {}

  bool is_defined() const { return defined_; }
  void *GetDataPtr() const { return data_; }
  TypeId data_type() const { return dtype_; }
  const ShapeVector &shape() const { return shape_; }
  const ShapeVector &strides() const { return strides_; }
  const pybind11::object &owner() const { return owner_; }
  int64_t numel() const {
    return std::accumulate(shape_.begin(), shape_.end(), static_cast<int64_t>(1), std::multiplies<int64_t>());
  }
  size_t nbytes() const { return static_cast<size_t>(numel()) * mindspore::TypeIdSize(dtype_); }
  bool is_contiguous() const {
    if (strides_.empty()) return true;
    int64_t expect = 1;
    for (int i = static_cast<int>(shape_.size()) - 1; i >= 0; --i) {
      if (shape_[i] != 1 && strides_[i] != expect) return false;
      expect *= shape_[i];
    }
    return true;
  }
  // A view on a sub-range of the same buffer (used to walk batches).
  Tensor Slice(int64_t elem_offset, ShapeVector shape) const {
    Tensor t = *this;
    t.data_ = static_cast<char *>(data_) + elem_offset * static_cast<int64_t>(mindspore::TypeIdSize(dtype_));
    t.shape_ = std::move(shape);
    t.strides_.clear();
    return t;
  }

 private:
  void *data_{nullptr};
  TypeId dtype_{mindspore::kMetaTypeNone};
  ShapeVector shape_;
  ShapeVector strides_;
  pybind11::object owner_;
  bool defined_{false};
};
}  // namespace ms
#endif  // MS_CUSTOM_OPS_FRAMEWORK_TENSOR_H_
