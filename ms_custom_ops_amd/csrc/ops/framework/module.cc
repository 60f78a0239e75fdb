// The single pybind11 module (reference: ops/framework/module.cc:19-22) plus the pieces MindSpore
// would provide: the Tensor binding, the framework hooks, and a small graph-mode executor that runs
// a registered op through infer -> KernelMod::Init -> Resize -> Launch.
#include "ops/framework/module.h"

#include <map>
#include <memory>
#include <mutex>
#include <sstream>

#include "ops/framework/hip_backend/hip_gmm_runner.h"

namespace py = pybind11;

namespace ms_custom_ops {
ms::Tensor AllocateTensor(TypeId type, const ShapeVector &shape) {
  auto &hooks = FrameworkHooks::Get();
  if (hooks.allocate.is_none() || !hooks.allocate) {
    MS_LOG_EXCEPTION << "No device allocator is registered: import the ms_custom_ops_amd package (it registers the "
                        "host framework's allocator) before calling an operator.";
  }
  py::gil_scoped_acquire gil;
  return hooks.allocate(static_cast<int>(type), shape).cast<ms::Tensor>();
}

namespace {
thread_local bool t_launch_stream_active = false;
thread_local void *t_launch_stream = nullptr;
}  // namespace

LaunchStreamScope::LaunchStreamScope(void *stream) : prev_active_(t_launch_stream_active), prev_stream_(t_launch_stream) {
  t_launch_stream_active = true;
  t_launch_stream = stream;
}
LaunchStreamScope::~LaunchStreamScope() {
  t_launch_stream_active = prev_active_;
  t_launch_stream = prev_stream_;
}

void *CurrentStream() {
  if (t_launch_stream_active) return t_launch_stream;
  auto &hooks = FrameworkHooks::Get();
  if (hooks.current_stream.is_none() || !hooks.current_stream) return nullptr;
  py::gil_scoped_acquire gil;
  return reinterpret_cast<void *>(hooks.current_stream().cast<uintptr_t>());
}

namespace {
KernelTensor ToKernelTensor(const py::handle &obj) {
  KernelTensor kt;
  if (obj.is_none()) return kt;
  kt.is_none = false;
  if (py::isinstance<ms::Tensor>(obj)) {
    kt.tensor = obj.cast<ms::Tensor>();
  } else if (py::isinstance<py::bool_>(obj)) {
    kt.value = obj.cast<bool>();
  } else if (py::isinstance<py::int_>(obj)) {
    kt.value = obj.cast<int64_t>();
  } else if (py::isinstance<py::str>(obj)) {
    kt.value = obj.cast<std::string>();
  } else if (py::isinstance<py::list>(obj) || py::isinstance<py::tuple>(obj)) {
    kt.is_sequence = true;
    for (const auto &item : obj) kt.sequence.push_back(item.cast<ms::Tensor>());
  } else {
    MS_EXCEPTION_TYPE << "Unsupported graph-mode input type: " << std::string(py::str(py::type::handle_of(obj)));
  }
  return kt;
}

// What Resize depends on: kind, dtype and shape of every input and the values of the scalar attributes.
std::string InputSignature(const KernelTensorList &inputs) {
  std::ostringstream os;
  auto tensor = [&](const ms::Tensor &t) {
    os << (t.is_contiguous() ? 't' : 's') << static_cast<int>(t.data_type()) << '[';
    for (int64_t d : t.shape()) os << d << ',';
    os << ']';
  };
  for (const auto &in : inputs) {
    if (in.IsNone()) {
      os << "N;";
    } else if (in.IsSequence()) {
      os << 'L';
      for (const auto &t : in.sequence) tensor(t);
      os << ';';
    } else if (in.tensor.is_defined()) {
      tensor(in.tensor);
      os << ';';
    } else if (std::holds_alternative<bool>(in.value)) {
      os << 'b' << std::get<bool>(in.value) << ';';
    } else if (std::holds_alternative<int64_t>(in.value)) {
      os << 'i' << std::get<int64_t>(in.value) << ';';
    } else if (std::holds_alternative<std::string>(in.value)) {
      os << 's' << std::get<std::string>(in.value) << ';';
    } else {
      os << "?;";
    }
  }
  return os.str();
}

// One kernel module per operator, as a graph holds one per node: Init ran once, Resize runs again only when the
// input signature changes (docs/ops_develop_guide.md:193-197).  A module keeps what Resize planned in its members
// and Launch reads them, so a node's Resize, workspace allocation and Launch form one critical section under the
// node's own mutex: a second thread (or a re-entrant call) with another signature waits for the pending Launch
// instead of re-planning the module under it.
struct GraphNode {
  std::mutex mu;   // taken with the GIL released (see LockNode), held across Resize .. Launch
  std::shared_ptr<KernelMod> kernel;
  std::string signature;
  std::vector<size_t> workspace_sizes;
  size_t inits{0}, resizes{0}, launches{0};
};
std::mutex g_nodes_mu;   // guards the map only
std::map<std::string, std::unique_ptr<GraphNode>> &GraphNodes() {
  static auto *nodes = new std::map<std::string, std::unique_ptr<GraphNode>>();   // leaked: kernel modules may hold device state
  return *nodes;
}
GraphNode &NodeOf(const std::string &name) {
  std::lock_guard<std::mutex> lock(g_nodes_mu);
  auto &slot = GraphNodes()[name];
  if (slot == nullptr) slot = std::make_unique<GraphNode>();
  return *slot;
}
// Lock order is node mutex first, interpreter lock second.  The launch below drops the interpreter lock while it
// holds the node mutex, so a thread must never wait for the node mutex while it holds the interpreter lock.
std::unique_lock<std::mutex> LockNode(GraphNode &node) {
  std::unique_lock<std::mutex> lock(node.mu, std::defer_lock);
  py::gil_scoped_release no_gil;
  lock.lock();
  return lock;
}

// Graph-mode execution of one registered op: the reference's compile-time infer plus the kernel
// module life cycle (Init once per instance, Resize on new shapes, Launch).
std::vector<ms::Tensor> GraphRun(const std::string &name, const py::list &args) {
  const OpRegistration *reg = OpRegistry::Instance().Find(name);
  if (reg == nullptr) MS_LOG_EXCEPTION << "Operator '" << name << "' is not registered for graph mode.";
  KernelTensorList inputs;
  for (const auto &a : args) inputs.push_back(ToKernelTensor(a));
  auto func_impl = reg->func_impl();
  const ShapeArray shapes = func_impl->InferShape(inputs);
  const TypeIdList types = func_impl->InferType(inputs);
  if (shapes.size() != types.size()) MS_LOG_EXCEPTION << "For " << name << ", infer returned mismatching outputs.";
  std::vector<ms::Tensor> outputs;
  for (size_t i = 0; i < shapes.size(); ++i) outputs.push_back(AllocateTensor(types[i], shapes[i]));
  GraphNode &node = NodeOf(name);
  std::unique_lock<std::mutex> lock = LockNode(node);
  if (node.kernel == nullptr) {
    node.kernel = reg->kernel_mod();
    if (!node.kernel->Init(inputs, outputs)) {
      node.kernel = nullptr;
      MS_LOG_EXCEPTION << "For " << name << ", KernelMod::Init failed.";
    }
    ++node.inits;
    node.signature.clear();
  }
  const std::string signature = InputSignature(inputs);
  if (node.resizes == 0 || signature != node.signature) {
    node.signature.clear();                       // stays empty if Resize throws: the next call plans again
    node.workspace_sizes = node.kernel->Resize(inputs, outputs);
    node.signature = signature;
    ++node.resizes;
  }
  ++node.launches;
  std::vector<ms::Tensor> workspace;
  for (size_t sz : node.workspace_sizes) workspace.push_back(AllocateTensor(kNumberTypeInt8, ShapeVector{static_cast<int64_t>(sz)}));
  if (!node.kernel->Launch(inputs, workspace, outputs, CurrentStream())) {
    MS_LOG_EXCEPTION << "For " << name << ", KernelMod::Launch failed.";
  }
  return outputs;
}

std::pair<ShapeArray, std::vector<int>> GraphInfer(const std::string &name, const py::list &args) {
  const OpRegistration *reg = OpRegistry::Instance().Find(name);
  if (reg == nullptr) MS_LOG_EXCEPTION << "Operator '" << name << "' is not registered for graph mode.";
  KernelTensorList inputs;
  for (const auto &a : args) inputs.push_back(ToKernelTensor(a));
  auto func_impl = reg->func_impl();
  std::vector<int> types;
  for (TypeId t : func_impl->InferType(inputs)) types.push_back(static_cast<int>(t));
  return {func_impl->InferShape(inputs), types};
}
}  // namespace
}  // namespace ms_custom_ops

PYBIND11_MODULE(MS_EXTENSION_NAME, m) {
  m.doc() = "A custom module for operators";

  py::class_<ms::Tensor>(m, "Tensor")
    .def(py::init<>())
    .def(py::init<uintptr_t, int, ms::ShapeVector, ms::ShapeVector, py::object>(), py::arg("data_ptr"),
         py::arg("type_id"), py::arg("shape"), py::arg("strides"), py::arg("owner") = py::none())
    .def_property_readonly("data_ptr", [](const ms::Tensor &t) { return reinterpret_cast<uintptr_t>(t.GetDataPtr()); })
    .def_property_readonly("type_id", [](const ms::Tensor &t) { return static_cast<int>(t.data_type()); })
    .def_property_readonly("shape", &ms::Tensor::shape)
    .def_property_readonly("strides", &ms::Tensor::strides)
    .def_property_readonly("owner", &ms::Tensor::owner)
    .def("is_defined", &ms::Tensor::is_defined)
    .def("is_contiguous", &ms::Tensor::is_contiguous);

  m.def("_set_framework_hooks", [](py::object allocate, py::object current_stream) {
    auto &hooks = ms_custom_ops::FrameworkHooks::Get();
    hooks.allocate = std::move(allocate);
    hooks.current_stream = std::move(current_stream);
  });
  m.def("_graph_run", &ms_custom_ops::GraphRun, "Run a registered op through the graph-mode kernel module");
  m.def("_graph_infer", &ms_custom_ops::GraphInfer, "InferShape / InferType of a registered op");
  m.def("_registered_graph_ops", []() { return ms_custom_ops::OpRegistry::Instance().Names(); });
  m.def("_plan_cache_stats", []() {
    auto &c = ms_custom_ops::GmmPlanCache::GetInstance();
    return py::make_tuple(c.hits(), c.misses(), c.size());
  });
  m.def("_graph_node_stats", [](const std::string &name) -> py::tuple {
    ms_custom_ops::GraphNode *node = nullptr;
    {
      std::lock_guard<std::mutex> lock(ms_custom_ops::g_nodes_mu);
      auto &nodes = ms_custom_ops::GraphNodes();
      auto it = nodes.find(name);
      if (it == nodes.end()) return py::make_tuple(0, 0, 0);
      node = it->second.get();
    }
    std::unique_lock<std::mutex> lock = ms_custom_ops::LockNode(*node);
    return py::make_tuple(node->inits, node->resizes, node->launches);
  }, "(Init, Resize, Launch) calls of an operator's graph-mode kernel module so far");
  m.def("_plan_cache_clear", []() { ms_custom_ops::GmmPlanCache::GetInstance().Clear(); });
  m.def("_backend_abi_version", []() { return msco_gmm_abi_version(); });

  ModuleRegistry::Instance().RegisterAll(m);
}
