// Operator registration surface.
//
// Same macros and registry as the reference (ops/framework/module.h:26-98): one static registrar
// object per operator translation unit, REG_GRAPH_MODE_OP for the graph-mode pair (infer
// implementation + kernel module), MS_CUSTOM_OPS_EXTENSION_MODULE for the pynative pybind
// definition, ModuleRegistry::RegisterAll from the single PYBIND11_MODULE.  MindSpore's
// MS_CUSTOM_OPS_REGISTER, OpFuncImpl and KernelMod are not available here, so this header also
// carries small in-repo equivalents: a name -> {infer, kernel factory} table and the two base
// classes with the reference's Init / Resize / Launch split (docs/ops_develop_guide.md:193-197).
#ifndef MS_CUSTOM_OPS_MODULE_H_
#define MS_CUSTOM_OPS_MODULE_H_

#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <variant>
#include <vector>

#include "ops/framework/tensor.h"
#include "ops/framework/utils.h"

using ModuleRegisterFunction = std::function<void(pybind11::module_ &)>;

class ModuleRegistry {
 public:
  static ModuleRegistry &Instance() {
    static ModuleRegistry instance;
    return instance;
  }
  // pynative definitions are installed first so a graph-mode placeholder never shadows them
  void Register(ModuleRegisterFunction func, bool pynative_node = true) {
    (pynative_node ? pynative_reg_functions_ : graph_reg_functions_).emplace_back(std::move(func));
  }
  void RegisterAll(pybind11::module_ &m) {
    for (const auto &func : pynative_reg_functions_) func(m);
    for (const auto &func : graph_reg_functions_) func(m);
  }

 private:
  ModuleRegistry() = default;
  ModuleRegistry(const ModuleRegistry &) = delete;
  ModuleRegistry &operator=(const ModuleRegistry &) = delete;
  std::vector<ModuleRegisterFunction> pynative_reg_functions_;
  std::vector<ModuleRegisterFunction> graph_reg_functions_;
};

namespace ms_custom_ops {
// One graph-mode input: a tensor, a list of tensors, a scalar attribute or None.
struct KernelTensor {
  using Scalar = std::variant<std::monostate, bool, int64_t, std::string>;
  bool is_none{true};
  ms::Tensor tensor;                 // defined for tensor inputs
  std::vector<ms::Tensor> sequence;  // non-empty for list-of-tensor inputs
  bool is_sequence{false};
  Scalar value;

  bool IsNone() const { return is_none; }
  bool IsSequence() const { return is_sequence; }
  TypeId GetType() const { return tensor.is_defined() ? tensor.data_type() : kMetaTypeNone; }
  const ShapeVector &GetShape() const { return tensor.shape(); }
  template <typename T>
  T GetValueWithCheck() const {
    if (!std::holds_alternative<T>(value)) MS_LOG_EXCEPTION << "Input scalar has an unexpected type.";
    return std::get<T>(value);
  }
};
using KernelTensorList = std::vector<KernelTensor>;

class OpFuncImpl {
 public:
  virtual ~OpFuncImpl() = default;
  virtual ShapeArray InferShape(const KernelTensorList &inputs) const = 0;
  virtual TypeIdList InferType(const KernelTensorList &inputs) const = 0;
};

class KernelMod {
 public:
  virtual ~KernelMod() = default;
  // once per instance
  virtual bool Init(const KernelTensorList &inputs, const std::vector<ms::Tensor> &outputs) { return true; }
  // whenever shapes change: shape-dependent planning, returns workspace sizes
  virtual std::vector<size_t> Resize(const KernelTensorList &inputs, const std::vector<ms::Tensor> &outputs) = 0;
  // every step
  virtual bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &workspace,
                      const std::vector<ms::Tensor> &outputs, void *stream) = 0;
};

struct OpRegistration {
  std::function<std::shared_ptr<OpFuncImpl>()> func_impl;
  std::function<std::shared_ptr<KernelMod>()> kernel_mod;
};

class OpRegistry {
 public:
  static OpRegistry &Instance() {
    static OpRegistry instance;
    return instance;
  }
  void Register(const std::string &name, OpRegistration reg) { ops_[name] = std::move(reg); }
  const OpRegistration *Find(const std::string &name) const {
    auto it = ops_.find(name);
    return it == ops_.end() ? nullptr : &it->second;
  }
  std::vector<std::string> Names() const {
    std::vector<std::string> names;
    for (const auto &kv : ops_) names.push_back(kv.first);
    return names;
  }

 private:
  std::map<std::string, OpRegistration> ops_;
};
}  // namespace ms_custom_ops

#define MS_CUSTOM_OPS_REGISTER(op, OpFuncImplClass, KernelClass)                                   \
  static const bool op##_op_registered = []() {                                                    \
    ::ms_custom_ops::OpRegistry::Instance().Register(                                              \
      #op, {[]() -> std::shared_ptr<::ms_custom_ops::OpFuncImpl> { return std::make_shared<OpFuncImplClass>(); }, \
            []() -> std::shared_ptr<::ms_custom_ops::KernelMod> { return std::make_shared<KernelClass>(); }});    \
    return true;                                                                                   \
  }()

#define REG_GRAPH_MODE_OP(op, OpFuncImplClass, KernelClass)                    \
  MS_CUSTOM_OPS_REGISTER(op, OpFuncImplClass, KernelClass);                    \
  static void op##_func() {}                                                   \
  static void op##_register(pybind11::module_ &m) {                            \
    if (!pybind11::hasattr(m, #op)) {                                          \
      m.def(#op, &op##_func);                                                  \
    }                                                                          \
  }                                                                            \
  struct op##_registrar {                                                      \
    op##_registrar() {                                                         \
      ModuleRegistry::Instance().Register(op##_register, false);               \
    }                                                                          \
  };                                                                           \
  static op##_registrar registrar_instance

#define CONCATENATE_DETAIL(x, y) x##y
#define CONCATENATE(x, y) CONCATENATE_DETAIL(x, y)

#define MS_CUSTOM_OPS_EXTENSION_MODULE(m)                                      \
  static void CONCATENATE(func_register_, __LINE__)(pybind11::module_ &);      \
  namespace {                                                                  \
  struct CONCATENATE(func_registrar_, __LINE__) {                              \
    CONCATENATE(func_registrar_, __LINE__)() {                                 \
      ModuleRegistry::Instance().Register(                                     \
          CONCATENATE(func_register_, __LINE__));                              \
    }                                                                          \
  };                                                                           \
  static CONCATENATE(func_registrar_, __LINE__)                                \
      CONCATENATE(registrar_instance_, __LINE__);                              \
  }                                                                            \
  static void CONCATENATE(func_register_, __LINE__)(pybind11::module_ & m)

#endif  // MS_CUSTOM_OPS_MODULE_H_
