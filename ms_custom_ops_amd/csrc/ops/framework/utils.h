// Shared constants, error helpers and host-framework hooks of the operator layer.
// Counterpart of the reference's ops/framework/utils.h (index constants :25-52, GetTensorOrEmpty :64,
// DataFormat :122-125, GilReleaseWithCheck :181-194).
#ifndef MS_CUSTOM_OPS_FRAMEWORK_UTILS_H_
#define MS_CUSTOM_OPS_FRAMEWORK_UTILS_H_

#include <pybind11/pybind11.h>

#include <memory>
#include <optional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "ops/framework/tensor.h"

namespace ms_custom_ops {
using namespace mindspore;

constexpr size_t kIndex0{0};
constexpr size_t kIndex1{1};
constexpr size_t kIndex2{2};
constexpr size_t kIndex3{3};
constexpr size_t kDim1{1};
constexpr size_t kDim2{2};
constexpr size_t kDim3{3};
constexpr size_t kDim4{4};
constexpr size_t kNumber1{1};
constexpr size_t kNumber2{2};

constexpr auto kFractalNzFormat = "FRACTAL_NZ";
constexpr auto kNdFormat = "ND";
// Weights prepacked by trans_data(..., ND_TO_FRACTAL_NZ) travel as int8 tensors whose last dimension is one 1024-byte
// block: [E, N / 16, ceil(K / 64), 1024], or [N / 16, ceil(K / 64), 1024] for a single matrix.
constexpr int64_t kPackedBlockBytes = 1024;
inline bool IsPackedWeightShape(const std::vector<int64_t> &shape, size_t rank) {
  return shape.size() == rank && shape.back() == kPackedBlockBytes;
}

enum class DataFormat : int32_t { ND = 0, FRACTAL_NZ = 1 };

inline ms::Tensor GetTensorOrEmpty(const std::optional<ms::Tensor> &opt_tensor) {
  return opt_tensor.has_value() ? opt_tensor.value() : ms::Tensor();
}

// ---- error helpers --------------------------------------------------------------------------
// MS_LOG(EXCEPTION) in the reference surfaces as a Python RuntimeError, MS_EXCEPTION(ValueError)
// as ValueError; the two stream-style helpers below keep those call sites readable.
class ExceptionStream {
 public:
  enum Kind { kRuntime, kValue, kType };
  explicit ExceptionStream(Kind kind) : kind_(kind) {}
  template <typename T>
  ExceptionStream &operator<<(const T &v) { os_ << v; return *this; }
  ExceptionStream &operator<<(const ShapeVector &v) {
    os_ << "[";
    for (size_t i = 0; i < v.size(); ++i) os_ << (i ? ", " : "") << v[i];
    os_ << "]";
    return *this;
  }
  ExceptionStream &operator<<(TypeId t) { os_ << TypeIdToString(t); return *this; }
  [[noreturn]] void Throw() const {
    if (kind_ == kValue) throw pybind11::value_error(os_.str());
    if (kind_ == kType) throw pybind11::type_error(os_.str());
    throw std::runtime_error(os_.str());
  }

 private:
  Kind kind_;
  std::ostringstream os_;
};
struct ExceptionThrower {
  [[noreturn]] void operator=(const ExceptionStream &s) const { s.Throw(); }
};
#define MS_LOG_EXCEPTION ::ms_custom_ops::ExceptionThrower() = ::ms_custom_ops::ExceptionStream(::ms_custom_ops::ExceptionStream::kRuntime)
#define MS_EXCEPTION_VALUE ::ms_custom_ops::ExceptionThrower() = ::ms_custom_ops::ExceptionStream(::ms_custom_ops::ExceptionStream::kValue)
#define MS_EXCEPTION_TYPE ::ms_custom_ops::ExceptionThrower() = ::ms_custom_ops::ExceptionStream(::ms_custom_ops::ExceptionStream::kType)

// ---- host-framework hooks -----------------------------------------------------------------------
// The host framework (the Python package on top of PyTorch-ROCm) owns device memory and streams:
// it registers an allocator and a current-stream getter once at import.
struct FrameworkHooks {
  pybind11::object allocate;        // (type_id:int, shape:list[int]) -> ms::Tensor
  pybind11::object current_stream;  // () -> int (hipStream_t)
  static FrameworkHooks &Get() {
    static FrameworkHooks *hooks = new FrameworkHooks();  // leaked on purpose: outlives the interpreter
    return *hooks;
  }
};

ms::Tensor AllocateTensor(TypeId type, const ShapeVector &shape);
// The stream operator code enqueues on: the host framework's current stream, or -- inside a graph-mode
// KernelMod::Launch -- the stream that Launch was given (LaunchStreamScope).
void *CurrentStream();
class LaunchStreamScope {
 public:
  explicit LaunchStreamScope(void *stream);
  ~LaunchStreamScope();
  LaunchStreamScope(const LaunchStreamScope &) = delete;
  LaunchStreamScope &operator=(const LaunchStreamScope &) = delete;

 private:
  bool prev_active_;
  void *prev_stream_;
};

class GilReleaseWithCheck {
 public:
  GilReleaseWithCheck() {
    if (Py_IsInitialized() != 0 && PyGILState_Check() != 0) release_ = std::make_unique<pybind11::gil_scoped_release>();
  }
  ~GilReleaseWithCheck() { release_ = nullptr; }

 private:
  std::unique_ptr<pybind11::gil_scoped_release> release_;
};
}  // namespace ms_custom_ops
#endif  // MS_CUSTOM_OPS_FRAMEWORK_UTILS_H_
