// Caller side of the HIP backend's C ABI: the pynative runner, the graph-mode kernel module and the
// plan cache they share.
//
// These take the place of the reference's InternalPyboostRunner
// (ops/framework/ms_kernels_internal/pyboost/internal_pyboost_runner.h:36-106), InternalKernelMod
// (ops/framework/ms_kernels_internal/graphmode/internal_kernel_mod.h:34-112) and the tiling cache
// (ops/framework/ms_kernels_internal/internal_tiling_cache.cc:374-426).  The contract is kept:
// a key over (op, dtypes, layouts, shapes) finds a planned kernel object; the framework allocates
// the workspace the plan asks for; launch receives positional device addresses with nullptr for
// absent optionals; a non-zero backend status becomes an exception.  What is gone is the Ascend
// tiling plumbing: plans depend on shapes only, so there is no host->device tiling copy.
#ifndef MS_CUSTOM_OPS_HIP_GMM_RUNNER_H_
#define MS_CUSTOM_OPS_HIP_GMM_RUNNER_H_

#include <list>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "msco_gmm.h"
#include "ops/framework/module.h"
#include "ops/framework/utils.h"

namespace ms_custom_ops {
using TensorList = std::vector<ms::Tensor>;

struct GmmProblem {
  int64_t m{0}, k{0}, n{0}, e{0};
};

// A planned backend kernel object.  Owned by the cache; never shared between streams.
struct GmmPlan {
  msco_gmm_handle handle{nullptr};
  size_t workspace_bytes{0};
  std::string info;
  ~GmmPlan();
};
using GmmPlanPtr = std::shared_ptr<GmmPlan>;

// LRU cache of planned kernel objects, capacity 64 like the reference's aclnn executor cache
// (ops/framework/aclnn/graphmode/aclnn_kernel_mod.h:47-64,217).
class GmmPlanCache {
 public:
  static GmmPlanCache &GetInstance();
  GmmPlanPtr GetOrCreate(const std::string &op_name, const msco_gmm_desc &desc, const GmmProblem &problem,
                         void *stream);
  size_t hits() const { return hits_; }
  size_t misses() const { return misses_; }
  size_t size() const { return items_.size(); }
  void Clear();

 private:
  using Item = std::pair<std::string, GmmPlanPtr>;
  static constexpr size_t kCapacity = 64;
  std::mutex mu_;
  std::list<Item> items_;
  std::unordered_map<std::string, std::list<Item>::iterator> index_;
  size_t hits_{0}, misses_{0};
};

msco_dtype ToBackendDtype(TypeId t);
void CheckContiguous(const std::string &op_name, const TensorList &tensors, bool is_input);
void LaunchPlan(const std::string &op_name, const GmmPlanPtr &plan, const void *const *inputs, void *out,
                void *workspace, size_t workspace_bytes, void *stream);

// Pynative driver: Setup -> GetOrCreateKernel -> Run, as npu_grouped_matmul uses its runner
// (ops/c_api/grouped_matmul/grouped_matmul.cc:283-314).
class HipGmmPyboostRunner {
 public:
  explicit HipGmmPyboostRunner(std::string op_name) : op_name_(std::move(op_name)) {}
  virtual ~HipGmmPyboostRunner() = default;
  const std::string &op_name() const { return op_name_; }

  // inputs are positional in backend order (MSCO_IN_*); undefined tensors are absent optionals
  void GetOrCreateKernel(const TensorList &inputs, const TensorList &outputs);
  void Run(const TensorList &inputs, const TensorList &outputs);
  const GmmPlanPtr &plan() const { return plan_; }

 protected:
  virtual msco_gmm_desc CreateKernel(const TensorList &inputs, const TensorList &outputs) = 0;
  virtual GmmProblem GetProblem(const TensorList &inputs, const TensorList &outputs) = 0;
  size_t CalcWorkspace() const { return plan_ ? plan_->workspace_bytes : 0; }
  void LaunchKernel(const TensorList &inputs, const TensorList &outputs, const ms::Tensor &workspace);

  std::string op_name_;
  GmmPlanPtr plan_;
  void *stream_{nullptr};
};

// Graph-mode kernel module: Init once, Resize per shape change (planning), Launch per step.
class HipGmmKernelMod : public KernelMod {
 public:
  explicit HipGmmKernelMod(std::string kernel_name) : kernel_name_(std::move(kernel_name)) {}
  std::vector<size_t> Resize(const KernelTensorList &inputs, const std::vector<ms::Tensor> &outputs) override;
  bool Launch(const KernelTensorList &inputs, const std::vector<ms::Tensor> &workspace,
              const std::vector<ms::Tensor> &outputs, void *stream) override;

 protected:
  // maps the op's argument list to backend positional tensors, the descriptor and the problem size
  virtual TensorList GetBackendInputs(const KernelTensorList &inputs) = 0;
  virtual msco_gmm_desc CreateKernel(const KernelTensorList &inputs, const TensorList &backend_inputs,
                                     const std::vector<ms::Tensor> &outputs) = 0;
  virtual GmmProblem GetProblem(const KernelTensorList &inputs, const TensorList &backend_inputs,
                                const std::vector<ms::Tensor> &outputs) = 0;
  std::string kernel_name_;
  // set by GetBackendInputs when x arrives [K, M] and was presented as [M, K]: Resize asks for one more workspace
  // slice of M K bytes (the last one) and Launch transposes x into it first
  bool transpose_x_{false};
  GmmPlanPtr plan_;
  void *plan_stream_{nullptr};   // the stream plan_ belongs to (kernel objects are per stream)
  msco_gmm_desc desc_{};         // what Resize planned for: Launch fetches the plan of its own stream with these
  GmmProblem problem_{};
};
}  // namespace ms_custom_ops
#endif  // MS_CUSTOM_OPS_HIP_GMM_RUNNER_H_
