#include "ops/framework/hip_backend/hip_gmm_runner.h"

#include <algorithm>
#include <cstring>
#include <sstream>

namespace ms_custom_ops {

GmmPlan::~GmmPlan() {
  if (handle != nullptr) (void)msco_gmm_destroy(handle);
}

GmmPlanCache &GmmPlanCache::GetInstance() {
  static GmmPlanCache *cache = new GmmPlanCache();  // leaked: device state must not be freed at exit
  return *cache;
}

void GmmPlanCache::Clear() {
  std::lock_guard<std::mutex> lock(mu_);
  items_.clear();
  index_.clear();
}

GmmPlanPtr GmmPlanCache::GetOrCreate(const std::string &op_name, const msco_gmm_desc &desc, const GmmProblem &problem,
                                     void *stream) {
  // key: op name + every descriptor field + shapes + stream (kernel objects are per stream)
  std::string key(op_name);
  key.push_back('\0');
  key.append(reinterpret_cast<const char *>(&desc), sizeof(desc));
  key.append(reinterpret_cast<const char *>(&problem), sizeof(problem));
  key.append(reinterpret_cast<const char *>(&stream), sizeof(stream));

  std::lock_guard<std::mutex> lock(mu_);
  auto it = index_.find(key);
  if (it != index_.end()) {
    ++hits_;
    items_.splice(items_.begin(), items_, it->second);
    return it->second->second;
  }
  ++misses_;
  auto plan = std::make_shared<GmmPlan>();
  int status = msco_gmm_create(&desc, &plan->handle);
  if (status != MSCO_OK) {
    MS_LOG_EXCEPTION << "For " << op_name << ", creating the HIP kernel object failed: " << msco_status_string(status);
  }
  status = msco_gmm_plan(plan->handle, problem.m, problem.k, problem.n, problem.e, &plan->workspace_bytes);
  if (status != MSCO_OK) {
    MS_LOG_EXCEPTION << "For " << op_name << ", planning the HIP kernel failed: " << msco_status_string(status)
                     << " (m=" << problem.m << ", k=" << problem.k << ", n=" << problem.n << ", e=" << problem.e
                     << ")";
  }
  char buf[512];
  (void)msco_gmm_plan_info(plan->handle, buf, sizeof(buf));
  plan->info = buf;
  items_.emplace_front(key, plan);
  index_[key] = items_.begin();
  if (items_.size() > kCapacity) {
    index_.erase(items_.back().first);
    items_.pop_back();
  }
  return plan;
}

msco_dtype ToBackendDtype(TypeId t) {
  switch (t) {
    case kNumberTypeInt8: return MSCO_DT_I8;
    case kNumberTypeInt32: return MSCO_DT_I32;
    case kNumberTypeInt64: return MSCO_DT_I64;
    case kNumberTypeUInt64: return MSCO_DT_U64;
    case kNumberTypeFloat16: return MSCO_DT_F16;
    case kNumberTypeBFloat16: return MSCO_DT_BF16;
    case kNumberTypeFloat32: return MSCO_DT_F32;
    default: return MSCO_DT_NONE;
  }
}

// Non-contiguous tensors are rejected like the reference does
// (ops/framework/ms_kernels_internal/pyboost/internal_pyboost_runner.cc:151-163).
void CheckContiguous(const std::string &op_name, const TensorList &tensors, bool is_input) {
  for (size_t i = 0; i < tensors.size(); ++i) {
    if (!tensors[i].is_defined() || tensors[i].is_contiguous()) continue;
    MS_LOG_EXCEPTION << "For internal op [" << op_name << "], the " << (is_input ? "input" : "output")
                     << " tensorlist[" << i << "] is not contiguous: "
                     << ", please convert it to contiguous tensor using tensor.contiguous().";
  }
}

void LaunchPlan(const std::string &op_name, const GmmPlanPtr &plan, const void *const *inputs, void *out,
                void *workspace, size_t workspace_bytes, void *stream) {
  int status;
  {
    GilReleaseWithCheck no_gil;
    status = msco_gmm_launch(plan->handle, inputs, out, workspace, workspace_bytes, stream);
  }
  if (status != MSCO_OK) {
    MS_LOG_EXCEPTION << "Launch InternalKernel failed, kernel_name: " << op_name << ", status: "
                     << msco_status_string(status);
  }
}

void HipGmmPyboostRunner::GetOrCreateKernel(const TensorList &inputs, const TensorList &outputs) {
  CheckContiguous(op_name_, inputs, true);
  CheckContiguous(op_name_, outputs, false);
  stream_ = CurrentStream();
  const msco_gmm_desc desc = CreateKernel(inputs, outputs);
  const GmmProblem problem = GetProblem(inputs, outputs);
  plan_ = GmmPlanCache::GetInstance().GetOrCreate(op_name_, desc, problem, stream_);
}

void HipGmmPyboostRunner::Run(const TensorList &inputs, const TensorList &outputs) {
  if (plan_ == nullptr) MS_LOG_EXCEPTION << "For " << op_name_ << ", Run called before GetOrCreateKernel.";
  ms::Tensor workspace;
  const size_t ws = CalcWorkspace();
  if (ws > 0) workspace = AllocateTensor(kNumberTypeInt8, ShapeVector{static_cast<int64_t>(ws)});
  LaunchKernel(inputs, outputs, workspace);
}

void HipGmmPyboostRunner::LaunchKernel(const TensorList &inputs, const TensorList &outputs,
                                       const ms::Tensor &workspace) {
  const void *addrs[MSCO_IN_COUNT] = {nullptr};
  for (size_t i = 0; i < inputs.size() && i < MSCO_IN_COUNT; ++i) {
    addrs[i] = inputs[i].is_defined() ? inputs[i].GetDataPtr() : nullptr;
  }
  LaunchPlan(op_name_, plan_, addrs, outputs.at(0).GetDataPtr(), workspace.is_defined() ? workspace.GetDataPtr() : nullptr,
             workspace.is_defined() ? workspace.nbytes() : 0, stream_);
}

std::vector<size_t> HipGmmKernelMod::Resize(const KernelTensorList &inputs, const std::vector<ms::Tensor> &outputs) {
  const TensorList backend_inputs = GetBackendInputs(inputs);
  CheckContiguous(kernel_name_, backend_inputs, true);
  CheckContiguous(kernel_name_, outputs, false);
  desc_ = CreateKernel(inputs, backend_inputs, outputs);
  problem_ = GetProblem(inputs, backend_inputs, outputs);
  plan_stream_ = CurrentStream();
  plan_ = GmmPlanCache::GetInstance().GetOrCreate(kernel_name_, desc_, problem_, plan_stream_);
  std::vector<size_t> sizes;
  if (plan_->workspace_bytes) sizes.push_back(plan_->workspace_bytes);
  if (transpose_x_) sizes.push_back(static_cast<size_t>(std::max<int64_t>(problem_.m * problem_.k, 1)));
  return sizes;
}

bool HipGmmKernelMod::Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &workspace,
                             const std::vector<ms::Tensor> &outputs, void *stream) {
  if (plan_ == nullptr) MS_LOG_EXCEPTION << "For " << kernel_name_ << ", Launch called before Resize.";
  if (stream != plan_stream_) {
    // a kernel object keeps cross-workgroup reduction state and serves one stream: take the one of this stream
    plan_ = GmmPlanCache::GetInstance().GetOrCreate(kernel_name_, desc_, problem_, stream);
    plan_stream_ = stream;
  }
  const TensorList backend_inputs = GetBackendInputs(inputs);
  const void *addrs[MSCO_IN_COUNT] = {nullptr};
  for (size_t i = 0; i < backend_inputs.size() && i < MSCO_IN_COUNT; ++i) {
    addrs[i] = backend_inputs[i].is_defined() ? backend_inputs[i].GetDataPtr() : nullptr;
  }
  const bool has_ws = plan_->workspace_bytes > 0;
  if (workspace.size() != (has_ws ? 1u : 0u) + (transpose_x_ ? 1u : 0u)) {
    MS_LOG_EXCEPTION << "For " << kernel_name_ << ", Launch got " << workspace.size() << " workspace tensors, Resize asked for "
                     << (has_ws ? 1 : 0) + (transpose_x_ ? 1 : 0);
  }
  void *ws = has_ws ? workspace[0].GetDataPtr() : nullptr;
  const size_t ws_bytes = has_ws ? workspace[0].nbytes() : 0;
  if (transpose_x_) {
    void *rows = workspace.back().GetDataPtr();
    if (problem_.m > 0 && problem_.k > 0) {
      const int rc = msco_transpose_2d(addrs[MSCO_IN_X], rows, 1, problem_.k, problem_.m, 1, stream);
      if (rc != MSCO_OK) MS_LOG_EXCEPTION << "For " << kernel_name_ << ", transposing x failed: " << msco_status_string(rc);
    }
    addrs[MSCO_IN_X] = rows;
  }
  const GmmPlanPtr plan = plan_;   // the launch drops the GIL: another thread's Resize may replace plan_ meanwhile
  LaunchPlan(kernel_name_, plan, addrs, outputs.at(0).GetDataPtr(), ws, ws_bytes, stream);
  return true;
}
}  // namespace ms_custom_ops
