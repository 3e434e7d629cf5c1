// Thin PyTorch-ROCm binding over the C ABI in optimi_hip.h.
//
// PyTorch owns every buffer and the stream; this file only turns tensors into raw
// pointers, checks that they are what the kernels assume (same device, one supported
// dtype, equal sizes, the parameter's dense layout), picks the calling thread's current
// HIP stream and raises RuntimeError when the library returns a non-zero status.  It
// stands where the reference enters its Triton launchers (optimi/adam.py:278-291,
// lion.py:240-253, stableadamw.py:337-350, adan.py:314-327).

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/csrc/autograd/engine.h>
#include <torch/csrc/autograd/graph_task.h>
#include <torch/csrc/Exceptions.h>
#include <torch/csrc/autograd/python_variable.h>
#include <torch/extension.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "optimi_hip.h"

namespace {

using TensorList = std::vector<at::Tensor>;
using OptTensorList = std::vector<std::optional<at::Tensor>>;

void check_status(int rc, const char* what) {
  TORCH_CHECK(rc == 0, what, " failed: ", optimi_hip_error_string(rc), " (status ", rc, ")");
}

int dtype_code(const at::Tensor& t) {
  switch (t.scalar_type()) {
    case at::kFloat: return OPTIMI_F32;
    case at::kBFloat16: return OPTIMI_BF16;
    case at::kHalf: return OPTIMI_F16;
    default: TORCH_CHECK(false, "optimi_amd: unsupported parameter dtype ", t.scalar_type(), " (float32, bfloat16 and float16 are implemented)");
  }
  return -1;
}

// A buffer may stand in for the parameter element by element only when it has the
// parameter's dtype, device, size and strides.
void check_like(const at::Tensor& ref, const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.device() == ref.device(), "optimi_amd: ", name, " is on ", t.device(), ", parameter on ", ref.device());
  TORCH_CHECK(t.scalar_type() == ref.scalar_type(), "optimi_amd: ", name, " has dtype ", t.scalar_type(), ", parameter ", ref.scalar_type());
  TORCH_CHECK(t.numel() == ref.numel(), "optimi_amd: ", name, " has ", t.numel(), " elements, parameter ", ref.numel());
  TORCH_CHECK(t.strides() == ref.strides(), "optimi_amd: ", name, " strides differ from the parameter's");
}

void check_param(const at::Tensor& p) {
  TORCH_CHECK(p.is_cuda(), "optimi_amd: parameters must live on a HIP device, got ", p.device());
  TORCH_CHECK(p.is_non_overlapping_and_dense(), "optimi_amd: parameter must be dense and non-overlapping in memory");
}

class Group {
 public:
  Group() { check_status(optimi_hip_group_create(&g_), "optimi_hip_group_create"); }
  ~Group() {
    if (g_) (void)optimi_hip_group_destroy(g_);
  }
  Group(const Group&) = delete;
  Group& operator=(const Group&) = delete;
  optimi_group* get() const { return g_; }

 private:
  optimi_group* g_ = nullptr;
};

// Collects the raw pointers of a list that must match `params` tensor by tensor.
struct PtrList {
  std::vector<void*> v;
  void* const* data() const { return v.data(); }
  const void* const* cdata() const { return (const void* const*)v.data(); }
};

PtrList gather(const TensorList& params, const TensorList& list, const char* name) {
  TORCH_CHECK(list.size() == params.size(), "optimi_amd: ", name, " has ", list.size(), " tensors, params has ", params.size());
  PtrList out;
  out.v.reserve(list.size());
  for (size_t i = 0; i < list.size(); ++i) {
    check_like(params[i], list[i], name);
    out.v.push_back(list[i].data_ptr());
  }
  return out;
}

struct Prepared {
  std::vector<int> dtypes;  // every tensor's dtype: fp32 and at most one 16-bit dtype
  bool kahan = false;       // the Kahan branch runs for the 16-bit tensors
  std::vector<int64_t> numel;
  PtrList params;
};

// One launch covers one device; its tensors are fp32 or of one 16-bit dtype, in any mixture.
Prepared prepare(const TensorList& params, uint32_t flags) {
  Prepared pr;
  if (params.empty()) return pr;
  pr.numel.reserve(params.size());
  pr.dtypes.reserve(params.size());
  pr.params.v.reserve(params.size());
  int low = OPTIMI_F32;
  for (const at::Tensor& p : params) {
    check_param(p);
    TORCH_CHECK(p.device() == params[0].device(), "optimi_amd: one launch covers one device");
    const int dtype = dtype_code(p);
    if (dtype != OPTIMI_F32) {
      TORCH_CHECK(low == OPTIMI_F32 || low == dtype, "optimi_amd: one launch covers float32 and one 16-bit dtype, not bfloat16 and float16 together");
      low = dtype;
    }
    pr.dtypes.push_back(dtype);
    pr.numel.push_back(p.numel());
    pr.params.v.push_back(p.data_ptr());
  }
  pr.kahan = low != OPTIMI_F32 && (flags & OPTIMI_KAHAN) && (flags & OPTIMI_UPDATE);
  return pr;
}

// Kahan buffers: taken only when the Kahan branch runs, and only for the 16-bit tensors;
// placeholders and None are ignored.
PtrList gather_kahan(const TensorList& params, const OptTensorList& list, const Prepared& pr) {
  PtrList out;
  if (!pr.kahan) return out;
  TORCH_CHECK(list.size() == params.size(), "optimi_amd: kahan_comps has ", list.size(), " tensors, params has ", params.size());
  out.v.reserve(list.size());
  for (size_t i = 0; i < list.size(); ++i) {
    if (pr.dtypes[i] == OPTIMI_F32) {
      out.v.push_back(nullptr);
      continue;
    }
    TORCH_CHECK(list[i].has_value(), "optimi_amd: kahan_sum is on but a Kahan buffer is missing");
    check_like(params[i], *list[i], "kahan_comp");
    out.v.push_back(list[i]->data_ptr());
  }
  return out;
}

void adam_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                const TensorList& exp_avg_sqs, const OptTensorList& kahan_comps, double lr, double beta1_comp,
                double beta2_hat, double beta2_comp, double weight_decay, double eps, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_adam_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                     pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtypes.data(), lr, beta1_comp, beta2_hat,
                                     beta2_comp, weight_decay, eps, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_adam_multi_mixed");
}

void lion_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                const OptTensorList& kahan_comps, double lr, double beta1_comp, double beta2_comp, double weight_decay,
                uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_lion_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(),
                                     pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtypes.data(), lr, beta1_comp, beta2_comp,
                                     weight_decay, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_lion_multi_mixed");
}

void stableadamw_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                       const TensorList& exp_avg_sqs, const OptTensorList& kahan_comps, double lr, double beta1_comp,
                       double beta2_hat, double beta2_comp, double weight_decay, double eps, double max_lr,
                       uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_stableadamw_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                            pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtypes.data(), lr, beta1_comp,
                                            beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags,
                                            c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_stableadamw_multi_mixed");
}

void adan_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                const TensorList& exp_avg_diffs, const TensorList& exp_avg_sqs, const TensorList& prev_grads,
                const OptTensorList& kahan_comps, double lr, double beta1_comp, double beta2, double beta2_comp,
                double beta3_hat, double beta3_comp, double eps, double weight_decay, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg");
  PtrList df = gather(params, exp_avg_diffs, "exp_avg_diff"), n = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList pg = gather(params, prev_grads, "prev_grad");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_adan_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), df.data(),
                                     n.data(), pg.data(), pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtypes.data(), lr,
                                     beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, flags,
                                     c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_adan_multi_mixed");
}

// Momentum buffers: absent (None or a one-element placeholder) when SGD runs without momentum.
PtrList gather_optional(const TensorList& params, const OptTensorList& list, bool needed, const char* name) {
  PtrList out;
  if (!needed) return out;
  TORCH_CHECK(list.size() == params.size(), "optimi_amd: ", name, " has ", list.size(), " tensors, params has ", params.size());
  out.v.reserve(list.size());
  for (size_t i = 0; i < list.size(); ++i) {
    TORCH_CHECK(list[i].has_value(), "optimi_amd: ", name, " is needed but missing");
    check_like(params[i], *list[i], name);
    out.v.push_back(list[i]->data_ptr());
  }
  return out;
}

void sgd_multi(Group& group, const TensorList& params, const TensorList& grads, const OptTensorList& exp_avgs,
               const OptTensorList& kahan_comps, double lr, double momentum, double weight_decay, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad");
  PtrList m = gather_optional(params, exp_avgs, momentum != 0, "exp_avg");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_sgd_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(),
                                    momentum != 0 ? m.data() : nullptr, pr.kahan ? k.data() : nullptr, pr.numel.data(),
                                    pr.dtypes.data(), lr, momentum, weight_decay, flags,
                                    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_sgd_multi_mixed");
}

void radam_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                 const TensorList& exp_avg_sqs, const OptTensorList& kahan_comps, double lr, double beta1_comp,
                 double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_radam_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                      pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtypes.data(), lr, beta1_comp, beta2_hat,
                                      beta2_comp, weight_decay, eps, rect, flags,
                                      c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_radam_multi_mixed");
}

void ranger_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                  const TensorList& exp_avg_sqs, const TensorList& la_params, const OptTensorList& kahan_comps, double lr,
                  double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect,
                  double alpha, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList la = gather(params, la_params, "la_param");
  PtrList k = gather_kahan(params, kahan_comps, pr);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_ranger_multi_mixed(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                       la.data(), pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtypes.data(), lr, beta1_comp,
                                       beta2_hat, beta2_comp, weight_decay, eps, rect, alpha, flags,
                                       c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_ranger_multi_mixed");
}

// ---- per-tensor entry points (gradient release) --------------------------------------
struct One {
  int dtype;
  bool kahan;
  void* k = nullptr;
};

One prepare_one(const at::Tensor& p, const std::optional<at::Tensor>& kahan_comp, uint32_t flags) {
  check_param(p);
  One o;
  o.dtype = dtype_code(p);
  o.kahan = o.dtype != OPTIMI_F32 && (flags & OPTIMI_KAHAN) && (flags & OPTIMI_UPDATE);
  if (o.kahan) {
    TORCH_CHECK(kahan_comp.has_value(), "optimi_amd: kahan_sum is on but the Kahan buffer is missing");
    check_like(p, *kahan_comp, "kahan_comp");
    o.k = kahan_comp->data_ptr();
  }
  return o;
}

void adam_single(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                 const std::optional<at::Tensor>& kahan_comp, double lr, double beta1_comp, double beta2_hat,
                 double beta2_comp, double weight_decay, double eps, uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  check_like(p, m, "exp_avg");
  check_like(p, v, "exp_avg_sq");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_adam_single(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), o.k, p.numel(), o.dtype, lr,
                                      beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, flags,
                                      c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_adam_single");
}

void lion_single(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const std::optional<at::Tensor>& kahan_comp,
                 double lr, double beta1_comp, double beta2_comp, double weight_decay, uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  check_like(p, m, "exp_avg");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_lion_single(p.data_ptr(), g.data_ptr(), m.data_ptr(), o.k, p.numel(), o.dtype, lr, beta1_comp,
                                      beta2_comp, weight_decay, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_lion_single");
}

void stableadamw_single(Group& group, const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                        const std::optional<at::Tensor>& kahan_comp, double lr, double beta1_comp, double beta2_hat,
                        double beta2_comp, double weight_decay, double eps, double max_lr, uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  check_like(p, m, "exp_avg");
  check_like(p, v, "exp_avg_sq");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_stableadamw_single(group.get(), p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), o.k,
                                             p.numel(), o.dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps,
                                             max_lr, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_stableadamw_single");
}

void adan_single(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& df, const at::Tensor& n,
                 const at::Tensor& pg, const std::optional<at::Tensor>& kahan_comp, double lr, double beta1_comp,
                 double beta2, double beta2_comp, double beta3_hat, double beta3_comp, double eps, double weight_decay,
                 uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  check_like(p, m, "exp_avg");
  check_like(p, df, "exp_avg_diff");
  check_like(p, n, "exp_avg_sq");
  check_like(p, pg, "prev_grad");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_adan_single(p.data_ptr(), g.data_ptr(), m.data_ptr(), df.data_ptr(), n.data_ptr(), pg.data_ptr(),
                                      o.k, p.numel(), o.dtype, lr, beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp,
                                      eps, weight_decay, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_adan_single");
}


void sgd_single(const at::Tensor& p, const at::Tensor& g, const std::optional<at::Tensor>& m,
                const std::optional<at::Tensor>& kahan_comp, double lr, double momentum, double weight_decay, uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  void* mp = nullptr;
  if (momentum != 0) {
    TORCH_CHECK(m.has_value(), "optimi_amd: momentum is on but the momentum buffer is missing");
    check_like(p, *m, "exp_avg");
    mp = m->data_ptr();
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_sgd_single(p.data_ptr(), g.data_ptr(), mp, o.k, p.numel(), o.dtype, lr, momentum, weight_decay,
                                     flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_sgd_single");
}

void radam_single(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                  const std::optional<at::Tensor>& kahan_comp, double lr, double beta1_comp, double beta2_hat,
                  double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  check_like(p, m, "exp_avg");
  check_like(p, v, "exp_avg_sq");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_radam_single(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), o.k, p.numel(), o.dtype, lr,
                                       beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, rect, flags,
                                       c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_radam_single");
}

void ranger_single(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v, const at::Tensor& la,
                   const std::optional<at::Tensor>& kahan_comp, double lr, double beta1_comp, double beta2_hat,
                   double beta2_comp, double weight_decay, double eps, double rect, double alpha, uint32_t flags) {
  One o = prepare_one(p, kahan_comp, flags);
  check_like(p, g, "grad");
  check_like(p, m, "exp_avg");
  check_like(p, v, "exp_avg_sq");
  check_like(p, la, "la_param");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(p.device());
  check_status(optimi_hip_ranger_single(p.data_ptr(), g.data_ptr(), m.data_ptr(), v.data_ptr(), la.data_ptr(), o.k, p.numel(),
                                        o.dtype, lr, beta1_comp, beta2_hat, beta2_comp, weight_decay, eps, rect, alpha, flags,
                                        c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_ranger_single");
}

// ---- gradient-release fast path --------------------------------------------------------
// One call per parameter from the post-accumulate-grad hook: advances the parameter's int32
// CPU step counter, forms the step scalars in double exactly as the functional forms do in
// Python (optimi/adam.py:260-273, lion.py:226-235, stableadamw.py:326-332, adan.py:289-309)
// and either launches the per-tensor kernel or, for a small tensor, parks the step in a
// ReleaseQueue that launches many of them as one list.  std::pow(double, double) is libm's
// pow, the function CPython's float ** int ends in, so the scalars are bit-identical to the
// Python path.

double debias_beta(double beta, int64_t step) {  // optimi/utils.py:31-36
  const double bt = std::pow(beta, (double)step);
  return (bt - beta) / (bt - 1.0);
}

// RAdam's variance rectification term; negative = not yet rectified (optimi/radam.py:269-277).
double rectification(double beta2, int64_t step) {
  const double rho_inf = 2 / (1 - beta2) - 1;
  const double bt = std::pow(beta2, (double)step);
  const double rho = rho_inf - 2 * (double)step * bt / (1 - bt);
  if (rho > 5) return std::sqrt(((rho - 4) * (rho - 2) * rho_inf) / ((rho_inf - 4) * (rho_inf - 2) * rho));
  return -1.0;
}

int64_t tick(const at::Tensor& step) {
  TORCH_CHECK(step.device().is_cpu() && step.scalar_type() == at::kInt && step.numel() == 1,
              "optimi_amd: the step counter must be a one-element int32 CPU tensor");
  int32_t* s = step.data_ptr<int32_t>();
  *s += 1;
  return *s;
}

// The Kahan buffer if it is one: placeholders (one element, maybe another dtype) and None count as absent.
std::optional<at::Tensor> real_kahan(const at::Tensor& p, const std::optional<at::Tensor>& k) {
  if (!k.has_value() || !k->defined() || k->numel() != p.numel() || k->scalar_type() != p.scalar_type()) return std::nullopt;
  return k;
}

at::Tensor grad_like(const at::Tensor& p, const at::Tensor& g) {
  TORCH_CHECK(g.scalar_type() == p.scalar_type(), "optimi_amd: gradient dtype ", g.scalar_type(), " differs from parameter dtype ", p.scalar_type());
  if (g.strides() == p.strides()) return g;
  return at::empty_like(p).copy_(g);
}

uint32_t base_flags(bool kahan_sum, bool update) { return (kahan_sum ? OPTIMI_KAHAN : 0u) | (update ? OPTIMI_UPDATE : 0u); }

// One per-tensor step, ready to launch: the tensors in the order the ABI's entry point for
// `kind` takes them (the parameter first, the Kahan buffer last; absent = nullopt) and the
// scalars in the order it takes them.
enum Kind { ADAM, LION, STABLEADAMW, ADAN, SGD, RADAM, RANGER };
constexpr int kMaxTensors = 7, kMaxScalars = 8;
constexpr int kTensorsOf[] = {5, 4, 5, 7, 4, 5, 6};
constexpr int kScalarsOf[] = {6, 4, 7, 8, 3, 7, 8};

struct StepCall {
  Kind kind;
  uint32_t flags = 0;
  std::optional<at::Tensor> t[kMaxTensors];
  double s[kMaxScalars] = {0, 0, 0, 0, 0, 0, 0, 0};
  const at::Tensor& param() const { return *t[0]; }
  const std::optional<at::Tensor>& kahan() const { return t[kTensorsOf[kind] - 1]; }
};

void launch_now(const StepCall& c, Group* stable_group) {
  const auto& t = c.t;
  const double* s = c.s;
  switch (c.kind) {
    case ADAM: adam_single(*t[0], *t[1], *t[2], *t[3], t[4], s[0], s[1], s[2], s[3], s[4], s[5], c.flags); break;
    case LION: lion_single(*t[0], *t[1], *t[2], t[3], s[0], s[1], s[2], s[3], c.flags); break;
    case STABLEADAMW:
      TORCH_CHECK(stable_group, "optimi_amd: StableAdamW needs a launch workspace");
      stableadamw_single(*stable_group, *t[0], *t[1], *t[2], *t[3], t[4], s[0], s[1], s[2], s[3], s[4], s[5], s[6], c.flags);
      break;
    case ADAN: adan_single(*t[0], *t[1], *t[2], *t[3], *t[4], *t[5], t[6], s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], c.flags); break;
    case SGD: sgd_single(*t[0], *t[1], t[2], t[3], s[0], s[1], s[2], c.flags); break;
    case RADAM: radam_single(*t[0], *t[1], *t[2], *t[3], t[4], s[0], s[1], s[2], s[3], s[4], s[5], s[6], c.flags); break;
    case RANGER: ranger_single(*t[0], *t[1], *t[2], *t[3], *t[4], t[5], s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], c.flags); break;
  }
}

// One whole-list launch of `kind`: ptr[a][i] is tensor i of array a, in the ABI's order for
// that kind, dtypes[i] its dtype; an array without any pointer is passed as absent (Kahan
// buffers when the Kahan branch is off, SGD's momentum buffer without momentum).
void launch_list(Kind kind, optimi_group* g, int n, const std::vector<void*>* ptr, const int64_t* numel, const int* dtypes,
                 const double* s, uint32_t flags, hipStream_t stream) {
  auto arr = [&](int a) { return (void* const*)ptr[a].data(); };
  auto carr = [&](int a) { return (const void* const*)ptr[a].data(); };
  auto opt = [&](int a) -> void* const* {
    for (void* q : ptr[a])
      if (q) return (void* const*)ptr[a].data();
    return nullptr;
  };
  int rc = 0;
  const char* what = "";
  switch (kind) {
    case ADAM:
      rc = optimi_hip_adam_multi_mixed(g, n, arr(0), carr(1), arr(2), arr(3), opt(4), numel, dtypes,
          s[0], s[1], s[2], s[3], s[4], s[5], flags, stream);
      what = "optimi_hip_adam_multi_mixed";
      break;
    case LION:
      rc = optimi_hip_lion_multi_mixed(g, n, arr(0), carr(1), arr(2), opt(3), numel, dtypes, s[0], s[1], s[2], s[3], flags, stream);
      what = "optimi_hip_lion_multi_mixed";
      break;
    case STABLEADAMW:
      rc = optimi_hip_stableadamw_multi_mixed(g, n, arr(0), carr(1), arr(2), arr(3), opt(4), numel, dtypes,
          s[0], s[1], s[2], s[3], s[4], s[5], s[6], flags, stream);
      what = "optimi_hip_stableadamw_multi_mixed";
      break;
    case ADAN:
      rc = optimi_hip_adan_multi_mixed(g, n, arr(0), carr(1), arr(2), arr(3), arr(4), arr(5), opt(6), numel, dtypes,
          s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], flags, stream);
      what = "optimi_hip_adan_multi_mixed";
      break;
    case SGD:
      rc = optimi_hip_sgd_multi_mixed(g, n, arr(0), carr(1), opt(2), opt(3), numel, dtypes, s[0], s[1], s[2], flags, stream);
      what = "optimi_hip_sgd_multi_mixed";
      break;
    case RADAM:
      rc = optimi_hip_radam_multi_mixed(g, n, arr(0), carr(1), arr(2), arr(3), opt(4), numel, dtypes,
          s[0], s[1], s[2], s[3], s[4], s[5], s[6], flags, stream);
      what = "optimi_hip_radam_multi_mixed";
      break;
    case RANGER:
      rc = optimi_hip_ranger_multi_mixed(g, n, arr(0), carr(1), arr(2), arr(3), arr(4), opt(5), numel, dtypes,
          s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], flags, stream);
      what = "optimi_hip_ranger_multi_mixed";
      break;
  }
  check_status(rc, what);
}

// What the per-tensor entry points check before they launch, for a step that may be parked
// instead.  Run before the step counter advances, so that a rejected step leaves no trace.
void validate_call(const StepCall& c) {
  static const char* const names[] = {"param", "grad", "state", "state", "state", "state", "state"};
  const at::Tensor& p = c.param();
  check_param(p);
  (void)dtype_code(p);
  for (int a = 1; a < kTensorsOf[c.kind]; ++a)
    if (c.t[a].has_value()) check_like(p, *c.t[a], names[a]);
}

void check_hip(hipError_t err, const char* what) {
  TORCH_CHECK(err == hipSuccess, "optimi_amd: ", what, " failed: ", hipGetErrorString(err));
}

// Parks the steps of small tensors and launches them together, as one list per run of steps
// that share everything but their tensors (optimizer, device, stream, flags and every scalar -
// which includes the step count through the debiased betas; fp32 tensors and tensors of one
// 16-bit dtype share a list, so a bf16 model with fp32 norms does not break the run at every
// norm).  A tensor of a few thousand elements costs far more to launch than to update, so a
// model with thousands of them is bound by launches; one list launch replaces up to
// `max_tensors` of them.  The queue
// keeps each parked gradient alive until its launch; `max_total` bounds how many bytes of
// gradients that may be.  Results are those of the per-tensor launches, bit for bit.
//
// Steps are parked only while a backward pass runs: the first one parked in a pass registers
// a final callback with the autograd engine, which launches whatever is parked when the pass
// has finished.  That callback may run on another thread than the hooks and without the GIL;
// it touches tensors only.
class ReleaseQueue : public std::enable_shared_from_this<ReleaseQueue> {
 public:
  ReleaseQueue(int64_t max_numel, int64_t max_tensors, int64_t max_total)
      : max_numel_(max_numel), max_tensors_(max_tensors), max_total_(max_total),
        seen_((size_t)(max_tensors > 0 && max_tensors < 4096 ? max_tensors : 4096)) {}
  ~ReleaseQueue() {
    // steps still parked are dropped, never launched from a destructor (the device may be gone);
    // their step counters have advanced, so say so
    if (!batch_.empty())
      std::fprintf(stderr, "optimi_amd: a gradient-release queue was destroyed with %zu parked optimizer steps that "
                           "were never launched (flush it, e.g. through optimizer.step() or state_dict(), first)\n",
                   batch_.size());
  }

  // Parks the step if a backward pass is running and the tensor is small enough, and makes sure
  // the pass ends with a flush; `c` is moved from only when it was parked.
  bool try_park(StepCall&& c) {
    if (c.param().numel() > max_numel_) return false;
    const int task = torch::autograd::get_current_graph_task_id();
    if (task == -1) return false;
    std::lock_guard<std::recursive_mutex> lock(mutex_);
    add(std::move(c));
    schedule(task);
    return true;
  }
  int64_t pending() {
    std::lock_guard<std::recursive_mutex> lock(mutex_);
    return (int64_t)batch_.size();
  }
  // list launches made so far, and the per-tensor steps they carried
  int64_t launches() const { return launches_; }
  int64_t launched_steps() const { return launched_steps_; }

  // Makes sure the running backward pass `task` ends with a flush.
  void schedule(int task) {
    std::lock_guard<std::recursive_mutex> lock(mutex_);
    if (task == -1 || task == scheduled_task_) return;
    std::weak_ptr<ReleaseQueue> weak = weak_from_this();
    torch::autograd::Engine::get_default_engine().queue_callback([weak] {
      if (std::shared_ptr<ReleaseQueue> q = weak.lock()) {
        {
          std::lock_guard<std::recursive_mutex> inner(q->mutex_);
          q->scheduled_task_ = -1;
        }
        q->flush(/*end_of_backward=*/true);
      }
    });
    scheduled_task_ = task;
  }

  void add(StepCall&& c) {
    std::lock_guard<std::recursive_mutex> lock(mutex_);
    const hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(c.param().device().index()).stream();
    if (!batch_.empty() && (!same_run(c, stream) || seen_.contains(c.param().data_ptr()))) flush();
    if (batch_.empty()) {
      stream_ = stream;
      low_dtype_ = at::kFloat;
      batch_.reserve((size_t)(max_tensors_ > 0 && max_tensors_ < 4096 ? max_tensors_ : 4096));  // flush() took the old storage along
    }
    if (c.param().scalar_type() != at::kFloat) low_dtype_ = c.param().scalar_type();
    total_ += c.param().numel() * (int64_t)c.param().element_size();
    seen_.insert(c.param().data_ptr());
    batch_.push_back(std::move(c));
    if ((int64_t)batch_.size() >= max_tensors_ || total_ >= max_total_) flush();
  }

  // `end_of_backward`: called from the autograd engine's final callback.  The engine runs those
  // under the streams that were current when backward() was called, after making them wait for
  // the streams the gradients were accumulated on - so there the launch goes to the device's
  // current stream, which is where the caller's next work (the next forward, step(),
  // state_dict()) is ordered.  Everywhere else the launch goes to the stream the steps were
  // parked on (the stream their gradients are ready on), and when that is not the current
  // stream, the current stream is made to wait for the launch.
  void flush(bool end_of_backward = false) {
    // The parked steps leave the queue under its lock and are launched, and their tensors let
    // go, outside it: dropping the last reference to a tensor that Python knows takes the GIL,
    // and a hook that holds the GIL may be waiting for the queue's lock at that moment.
    std::vector<StepCall> batch;
    hipStream_t stream = nullptr;
    {
      std::lock_guard<std::recursive_mutex> lock(mutex_);
      if (batch_.empty()) return;
      batch.swap(batch_);
      stream = stream_;
      seen_.clear();
      total_ = 0;
    }
    const StepCall& c0 = batch[0];
    const int n = (int)batch.size(), nt = kTensorsOf[c0.kind];
    std::vector<void*> ptr[kMaxTensors];
    std::vector<int64_t> numel((size_t)n);
    std::vector<int> dtypes((size_t)n);
    for (int a = 0; a < nt; ++a) ptr[a].resize((size_t)n, nullptr);
    for (int i = 0; i < n; ++i) {
      numel[(size_t)i] = batch[(size_t)i].param().numel();
      dtypes[(size_t)i] = dtype_code(batch[(size_t)i].param());
      for (int a = 0; a < nt; ++a)
        if (batch[(size_t)i].t[a].has_value()) ptr[a][(size_t)i] = batch[(size_t)i].t[a]->data_ptr();
    }
    c10::hip::HIPGuardMasqueradingAsCUDA guard(c0.param().device());
    std::lock_guard<std::mutex> launching(launch_mutex_);  // the workspaces serve one launch at a time
    std::unique_ptr<Group>& slot = groups_[c0.param().device().index()];  // a workspace lives on one device
    if (!slot) slot = std::make_unique<Group>();  // made on first use: a queue may exist before any device work
    const auto current_stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(c0.param().device().index());
    const hipStream_t current = current_stream.stream();
    const hipStream_t launch = end_of_backward ? current : stream;
    if (launch != stream) {
      // The parked gradients were allocated on the stream they were parked on and are let go as
      // soon as this function returns: tell the caching allocator that another stream reads them.
      for (const StepCall& c : batch) c.t[1]->record_stream(current_stream);
    }
    // never OPTIMI_RESIDENT: these tensors are a slice of a model whose backward pass has just
    // gone through the caches
    launch_list(c0.kind, slot->get(), n, ptr, numel.data(), dtypes.data(), c0.s, c0.flags, launch);
    ++launches_;
    launched_steps_ += n;
    if (launch != current) {
      hipEvent_t done = nullptr;
      check_hip(hipEventCreateWithFlags(&done, hipEventDisableTiming), "hipEventCreateWithFlags");
      hipError_t err = hipEventRecord(done, launch);
      if (err == hipSuccess) err = hipStreamWaitEvent(current, done, 0);
      (void)hipEventDestroy(done);  // the runtime keeps a recorded event alive until it has completed
      check_hip(err, "ordering the current stream after the gradient-release launch");
    }
  }

 private:

  bool same_run(const StepCall& c, hipStream_t stream) const {
    const StepCall& c0 = batch_[0];
    if (c.kind != c0.kind || c.flags != c0.flags || stream != stream_) return false;
    if (c.param().device() != c0.param().device()) return false;
    const at::ScalarType dtype = c.param().scalar_type();
    if (dtype != at::kFloat && low_dtype_ != at::kFloat && dtype != low_dtype_) return false;  // bf16 and fp16 do not share a list
    if (std::memcmp(c.s, c0.s, sizeof(c.s)) != 0) return false;
    // the same arrays present, except the Kahan buffer (the last one), which fp32 tensors never have
    for (int a = 0; a < kTensorsOf[c.kind] - 1; ++a)
      if (c.t[a].has_value() != c0.t[a].has_value()) return false;
    return true;
  }

  int64_t max_numel_, max_tensors_, max_total_;
  std::recursive_mutex mutex_;
  std::mutex launch_mutex_;
  int scheduled_task_ = -1;  // the backward pass that already carries the flush callback
  std::unordered_map<int, std::unique_ptr<Group>> groups_;
  std::vector<StepCall> batch_;
  // The parameters parked so far (two steps of one parameter must not share a launch): a flat
  // open-addressing table, because a node-based set pays an allocation for every parked step.
  class PointerSet {
   public:
    explicit PointerSet(size_t expected) {
      size_t cap = 64;
      while (cap < 2 * expected) cap *= 2;
      slots_.assign(cap, nullptr);
    }
    bool contains(const void* p) const {
      for (size_t i = hash(p);; i = (i + 1) & (slots_.size() - 1)) {
        if (slots_[i] == p) return true;
        if (!slots_[i]) return false;
      }
    }
    void insert(const void* p) {
      if (2 * (count_ + 1) > slots_.size()) grow();
      for (size_t i = hash(p);; i = (i + 1) & (slots_.size() - 1)) {
        if (slots_[i] == p) return;
        if (!slots_[i]) {
          slots_[i] = p;
          ++count_;
          return;
        }
      }
    }
    void clear() {
      if (count_) std::fill(slots_.begin(), slots_.end(), nullptr);
      count_ = 0;
    }

   private:
    size_t hash(const void* p) const { return (size_t)(((uintptr_t)p >> 4) * 0x9e3779b97f4a7c15ull >> 20) & (slots_.size() - 1); }
    void grow() {
      std::vector<const void*> old(2 * slots_.size(), nullptr);
      old.swap(slots_);
      count_ = 0;
      for (const void* p : old)
        if (p) insert(p);
    }
    std::vector<const void*> slots_;
    size_t count_ = 0;
  };
  PointerSet seen_;
  int64_t total_ = 0;
  hipStream_t stream_ = nullptr;
  at::ScalarType low_dtype_ = at::kFloat;  // the 16-bit dtype among the parked tensors, float while there is none
  std::atomic<int64_t> launches_{0}, launched_steps_{0};
};

// Parks the step when there is a queue, a backward pass is running and the tensor is small
// enough, otherwise launches it.  Returns whether the step was parked.
bool submit(StepCall&& c, ReleaseQueue* queue, Group* stable_group = nullptr) {
  if (queue && queue->try_park(std::move(c))) return true;
  launch_now(c, stable_group);
  return false;
}

// The scalar prologue of each functional form: flags and scalars as the ABI takes them, from
// the raw hyper-parameters and the step count `t` (1-based, already advanced).
struct Hyper {
  uint32_t flags = 0;
  double s[kMaxScalars] = {0, 0, 0, 0, 0, 0, 0, 0};
};

double decayed(double weight_decay, double lr, bool decouple_wd, bool decouple_lr, const std::optional<double>& max_lr) {
  if (weight_decay == 0) return 0;
  if (decouple_lr) return 1 - (lr / max_lr.value()) * weight_decay;
  if (decouple_wd) return 1 - lr * weight_decay;
  return weight_decay;  // L2: the raw coefficient
}

Hyper adam_hyper(int64_t t, double lr, double beta1, double beta2, double weight_decay, double eps, bool decouple_wd,
                 bool decouple_lr, const std::optional<double>& max_lr, bool kahan_sum, bool update) {  // optimi/adam.py:260-273
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t);
  return {base_flags(kahan_sum, update) | ((decouple_wd || decouple_lr) ? OPTIMI_DECOUPLE_WD : 0u),
          {lr, 1 - b1h, b2h, 1 - b2h, decayed(weight_decay, lr, decouple_wd, decouple_lr, max_lr), eps}};
}

Hyper lion_hyper(double lr, double beta1, double beta2, double weight_decay, bool decouple_lr,
                 const std::optional<double>& max_lr, bool kahan_sum, bool update) {  // optimi/lion.py:226-235
  return {base_flags(kahan_sum, update), {lr, 1 - beta1, 1 - beta2, decayed(weight_decay, lr, true, decouple_lr, max_lr)}};
}

Hyper stableadamw_hyper(int64_t t, double lr, double beta1, double beta2, double weight_decay, double eps, bool decouple_lr,
                        const std::optional<double>& max_lr, bool kahan_sum, bool update) {  // optimi/stableadamw.py:326-332
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t);
  return {base_flags(kahan_sum, update) | (decouple_lr ? OPTIMI_DECOUPLE_LR : 0u),
          {lr, 1 - b1h, b2h, 1 - b2h, weight_decay, eps, (decouple_lr && max_lr.has_value()) ? *max_lr : 0.0}};
}

Hyper adan_hyper(int64_t t, double lr, double beta1, double beta2, double beta3, double weight_decay, double eps,
                 bool decouple_lr, const std::optional<double>& max_lr, bool adam_wd, bool kahan_sum, bool update) {  // optimi/adan.py:289-309
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t), b3h = debias_beta(beta3, t);
  if (weight_decay != 0) {
    weight_decay = decouple_lr ? (lr / max_lr.value()) * weight_decay : lr * weight_decay;
    weight_decay = adam_wd ? 1 - weight_decay : 1 + weight_decay;
  }
  return {base_flags(kahan_sum, update) | (adam_wd ? OPTIMI_ADAM_WD : 0u),
          {lr, 1 - b1h, beta2, 1 - b2h, b3h, 1 - b3h, eps, weight_decay}};
}

Hyper sgd_hyper(double lr, double momentum, double weight_decay, bool dampening, bool decouple_wd, bool decouple_lr,
                const std::optional<double>& max_lr, bool kahan_sum, bool update) {  // optimi/sgd.py:213-240
  return {base_flags(kahan_sum, update) | ((decouple_wd || decouple_lr) ? OPTIMI_DECOUPLE_WD : 0u) | (dampening ? OPTIMI_DAMPENING : 0u),
          {lr, momentum, decayed(weight_decay, lr, decouple_wd, decouple_lr, max_lr)}};
}

// RAdam (optimi/radam.py:214-322) and, with lookahead, Ranger (optimi/ranger.py:230-344)
Hyper ranger_hyper(int64_t t, bool lookahead, double lr, double beta1, double beta2, double weight_decay, double eps,
                   int64_t sync_every, double alpha, bool decouple_wd, bool decouple_lr, const std::optional<double>& max_lr,
                   bool kahan_sum, bool update) {
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t);
  const double rect = rectification(beta2, t);
  uint32_t flags = base_flags(kahan_sum, update) | ((decouple_wd || decouple_lr) ? OPTIMI_DECOUPLE_WD : 0u) |
                   (rect >= 0 ? OPTIMI_RECTIFY : 0u);
  if (lookahead && t % sync_every == 0) flags |= OPTIMI_LOOKAHEAD;
  return {flags, {lr, 1 - b1h, b2h, 1 - b2h, decayed(weight_decay, lr, decouple_wd, decouple_lr, max_lr), eps,
                  rect >= 0 ? rect : 0.0, alpha}};
}

// The tensors of one step, validated; the scalars follow through set_hyper once the step
// counter has been advanced - nothing is mutated for a step that is rejected here.
StepCall make_call(Kind kind, std::initializer_list<std::optional<at::Tensor>> tensors) {
  StepCall c;
  c.kind = kind;
  int a = 0;
  for (const auto& t : tensors) c.t[a++] = t;
  validate_call(c);
  return c;
}

StepCall&& set_hyper(StepCall&& c, const Hyper& h) {
  c.flags = h.flags;
  std::memcpy(c.s, h.s, sizeof(c.s));
  return std::move(c);
}

bool adam_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                  const std::optional<at::Tensor>& k, const at::Tensor& step, double lr, double beta1, double beta2,
                  double weight_decay, double eps, bool decouple_wd, bool decouple_lr, std::optional<double> max_lr,
                  bool kahan_sum, bool update, ReleaseQueue* queue) {
  StepCall c = make_call(ADAM, {p, grad_like(p, g), m, v, real_kahan(p, k)});
  const Hyper h = adam_hyper(tick(step), lr, beta1, beta2, weight_decay, eps, decouple_wd, decouple_lr, max_lr, kahan_sum, update);
  return submit(set_hyper(std::move(c), h), queue);
}

bool lion_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const std::optional<at::Tensor>& k,
                  double lr, double beta1, double beta2, double weight_decay, bool decouple_lr,
                  std::optional<double> max_lr, bool kahan_sum, bool update, ReleaseQueue* queue) {
  const Hyper h = lion_hyper(lr, beta1, beta2, weight_decay, decouple_lr, max_lr, kahan_sum, update);
  return submit(set_hyper(make_call(LION, {p, grad_like(p, g), m, real_kahan(p, k)}), h), queue);
}

bool stableadamw_release(Group& group, const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                         const std::optional<at::Tensor>& k, const at::Tensor& step, double lr, double beta1, double beta2,
                         double weight_decay, double eps, bool decouple_lr, std::optional<double> max_lr, bool kahan_sum,
                         bool update, ReleaseQueue* queue) {
  StepCall c = make_call(STABLEADAMW, {p, grad_like(p, g), m, v, real_kahan(p, k)});
  const Hyper h = stableadamw_hyper(tick(step), lr, beta1, beta2, weight_decay, eps, decouple_lr, max_lr, kahan_sum, update);
  return submit(set_hyper(std::move(c), h), queue, &group);
}

bool adan_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& df, const at::Tensor& n,
                  const at::Tensor& pg, const std::optional<at::Tensor>& k, const at::Tensor& step, double lr, double beta1,
                  double beta2, double beta3, double weight_decay, double eps, bool decouple_lr, std::optional<double> max_lr,
                  bool adam_wd, bool kahan_sum, bool update, ReleaseQueue* queue) {
  StepCall c = make_call(ADAN, {p, grad_like(p, g), m, df, n, pg, real_kahan(p, k)});
  const Hyper h = adan_hyper(tick(step), lr, beta1, beta2, beta3, weight_decay, eps, decouple_lr, max_lr, adam_wd, kahan_sum, update);
  return submit(set_hyper(std::move(c), h), queue);
}

bool sgd_release(const at::Tensor& p, const at::Tensor& g, const std::optional<at::Tensor>& m,
                 const std::optional<at::Tensor>& k, double lr, double momentum, double weight_decay, bool dampening,
                 bool decouple_wd, bool decouple_lr, std::optional<double> max_lr, bool kahan_sum, bool update,
                 ReleaseQueue* queue) {
  const Hyper h = sgd_hyper(lr, momentum, weight_decay, dampening, decouple_wd, decouple_lr, max_lr, kahan_sum, update);
  return submit(set_hyper(make_call(SGD, {p, grad_like(p, g), momentum != 0 ? real_kahan(p, m) : std::nullopt, real_kahan(p, k)}), h), queue);
}

bool ranger_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                    const std::optional<at::Tensor>& la, const std::optional<at::Tensor>& k, const at::Tensor& step, double lr,
                    double beta1, double beta2, double weight_decay, double eps, int64_t sync_every, double alpha,
                    bool decouple_wd, bool decouple_lr, std::optional<double> max_lr, bool kahan_sum, bool update,
                    ReleaseQueue* queue) {
  // la = None makes this RAdam; with la it is Ranger
  StepCall c = la.has_value() ? make_call(RANGER, {p, grad_like(p, g), m, v, *la, real_kahan(p, k)})
                              : make_call(RADAM, {p, grad_like(p, g), m, v, real_kahan(p, k)});
  const Hyper h = ranger_hyper(tick(step), la.has_value(), lr, beta1, beta2, weight_decay, eps, sync_every, alpha, decouple_wd,
                               decouple_lr, max_lr, kahan_sum, update);
  return submit(set_hyper(std::move(c), h), queue);
}


// ---- the post-accumulate-grad hook itself ------------------------------------------------
// What optimi's hook does in Python for every parameter of every backward pass - look the
// parameter's state and group up, read the hyper-parameters, step, free the gradient
// (optimi/gradientrelease.py:13-15, adam.py:183-208, optimizer.py:96-114) - done here without a
// Python frame.  Hyper-parameters are read from the group dict on every call, so schedulers
// that rewrite them are seen.  State tensors are cached per parameter and re-validated by
// identity against the state dict on every call; a parameter seen for the first time, or whose
// state changed, goes through the optimizer's Python method `_release_entry`, which creates
// the state exactly as step(param=...) would.  When step hooks are registered on the optimizer
// the Python path runs instead, so they fire.
class ReleaseHookCore {
 public:
  ReleaseHookCore(const py::object& optimizer, int kind, std::shared_ptr<ReleaseQueue> queue)
      : optimizer_(py::weakref(optimizer)), kind_((Kind)kind), queue_(std::move(queue)) {
    TORCH_CHECK(kind >= ADAM && kind <= RANGER, "optimi_amd: unknown optimizer kind ", kind);
    static const char* const keys[][5] = {
        {"exp_avg", "exp_avg_sq", "kahan_comp", nullptr, nullptr},               // ADAM
        {"exp_avg", "kahan_comp", nullptr, nullptr, nullptr},                    // LION
        {"exp_avg", "exp_avg_sq", "kahan_comp", nullptr, nullptr},               // STABLEADAMW
        {"exp_avg", "exp_avg_diff", "exp_avg_sq", "prev_grad", "kahan_comp"},    // ADAN
        {"exp_avg", "kahan_comp", nullptr, nullptr, nullptr},                    // SGD
        {"exp_avg", "exp_avg_sq", "kahan_comp", nullptr, nullptr},               // RADAM
        {"exp_avg", "exp_avg_sq", "la_param", "kahan_comp", nullptr},            // RANGER
    };
    for (int i = 0; i < 5 && keys[kind][i]; ++i) state_keys_.emplace_back(keys[kind][i]);
    has_step_ = kind_ != LION && kind_ != SGD;
    rebind();
  }

  // Forgets every cached parameter and re-reads the optimizer's hook tables; the optimizer
  // calls this whenever its state or groups are replaced wholesale (load_state_dict).
  void invalidate() {
    entries_.clear();
    workspaces_.clear();  // keyed by group dicts that may be gone now
    hyper_cache_.clear();
    rebind();
  }


  void call(const py::handle& param_h) {
    TORCH_CHECK(THPVariable_Check(param_h.ptr()), "optimi_amd: the gradient release hook takes the parameter");
    PyObject* opt_ptr = PyWeakref_GetObject(optimizer_.ptr());  // borrowed
    TORCH_CHECK(opt_ptr && opt_ptr != Py_None, "optimi_amd: the optimizer of this gradient release hook no longer exists");
    py::object optimizer = py::reinterpret_borrow<py::object>(opt_ptr);
    // What is the same for every parameter of a backward pass - whether step hooks are registered,
    // whether the pass only accumulates - is looked up once per pass (outside a pass: every call).
    const int task = torch::autograd::get_current_graph_task_id();
    if (task == -1 || task != pass_task_) {
      pass_hooks_ = any_step_hooks();
      pass_update_ = !truthy(py::reinterpret_steal<py::object>(attr(opt_ptr, k_.accumulation)).ptr());
      pass_task_ = task;
    }
    if (pass_hooks_) {
      optimizer.attr(k_.release)(param_h);
      return;
    }
    const at::Tensor& p = THPVariable_Unpack(param_h.ptr());
    Entry* e = find(p);
    if (!e || !valid(*e)) e = refresh(optimizer, k_.entry, param_h, p, true);
    const at::Tensor g = p.grad();
    TORCH_CHECK(g.defined(), "optimi_amd: the gradient release hook ran on a parameter without a gradient");
    at::NoGradGuard no_grad;
    PyObject* grp = e->group.ptr();
    StepCall c = pack(*e, Hyper{}, p, grad_like(p, g), momentum_of(grp));
    validate_call(c);  // before the counter moves: a rejected step leaves the state as it was
    submit(set_hyper(std::move(c), hyper_for(grp, has_step_ ? tick(e->step) : 0, pass_update_)), queue_.get(), e->workspace);
    p.mutable_grad().reset();  // param.grad = None
  }

  // One whole-group step (optimi/adam.py:158-182 and the functional form behind it) without the
  // per-parameter Python walk: collects the parameters of `group` that have a gradient, advances
  // the group's step counter, forms the scalars and launches one list per device.
  // Returns false, having done nothing, when the group has not been set up yet (the first step
  // goes through Python, which resolves the backend) - the caller then takes the Python path.
  // `resident`: the caller steps back to back, with nothing in between that would sweep the
  // last-level cache, and everything the optimizer touches fits that cache - the list is then
  // read with cached loads (OPTIMI_RESIDENT).  The size test is the caller's, over all groups: the
  // few norm weights of a no-decay group beside 100 GB of matrices are not resident.
  bool step_group(const py::dict& group, bool resident) {
    PyObject* grp = group.ptr();
    if (!flag(grp, k_.setup) || item(grp, k_.triton) != Py_True) return false;
    py::object optimizer = optimizer_();
    TORCH_CHECK(!optimizer.is_none(), "optimi_amd: the optimizer no longer exists");
    PyObject* plist = item(grp, k_.params);
    TORCH_CHECK(PyList_Check(plist), "optimi_amd: group['params'] must be a list");
    at::NoGradGuard no_grad;

    // pass 1: the parameters that step, their cached states (created on first sight); no side effects on steps
    struct Item {
      const at::Tensor* p;  // lives in the parameter list
      at::Tensor g;         // the gradient, or a copy of it with the parameter's strides
      Entry* e;
    };
    std::vector<Item> items;
    const double momentum = momentum_of(grp);
    const Py_ssize_t n_params = PyList_GET_SIZE(plist);
    items.reserve((size_t)n_params);
    for (Py_ssize_t i = 0; i < n_params; ++i) {
      PyObject* obj = PyList_GET_ITEM(plist, i);
      TORCH_CHECK(THPVariable_Check(obj), "optimi_amd: group['params'] holds something that is not a tensor");
      const at::Tensor& p = THPVariable_Unpack(obj);
      const at::Tensor& g = p.grad();
      if (!g.defined()) continue;
      TORCH_CHECK(!g.is_sparse(), "optimi_amd does not support sparse gradients");
      Entry* e = find(p);
      if (!e || !valid(*e, false)) e = refresh(optimizer, k_.group_entry, py::handle(obj), p, false, group);
      at::Tensor g_like = grad_like(p, g);
      validate_view(view(*e, p, g_like, momentum));  // everything that can reject the step, before the counter moves
      items.push_back({&p, std::move(g_like), e});
    }

    // the group's counter advances even when nothing has a gradient, as in the reference
    int64_t t = 0;
    if (has_step_) {
      PyObject* step = item(grp, k_.step);
      TORCH_CHECK(THPVariable_Check(step), "optimi_amd: group['step'] must be a tensor");
      t = tick(THPVariable_Unpack(step));
    }
    if (items.empty()) return true;
    const Hyper h = hyper_for(grp, t, true);

    // pass 2: one launch per device, in order of first appearance.  fp32 parameters and the
    // parameters of one 16-bit dtype go together; a group that holds bf16 and fp16 gets a launch for each.
    const int nt = kTensorsOf[kind_];
    std::vector<char> done(items.size(), 0);
    for (size_t first = 0; first < items.size(); ++first) {
      if (done[first]) continue;
      const at::Tensor& p0 = *items[first].p;
      at::ScalarType low = at::kFloat;
      std::vector<void*> ptr[kMaxTensors];
      std::vector<char> has[kMaxTensors];  // the array exists for the tensor (a tensor without elements has no address)
      std::vector<int64_t> numel;
      std::vector<int> dtypes;
      const size_t room = items.size() - first;
      for (int a = 0; a < nt; ++a) {
        ptr[a].reserve(room);
        has[a].reserve(room);
      }
      numel.reserve(room);
      dtypes.reserve(room);
      for (size_t i = first; i < items.size(); ++i) {
        const at::Tensor& p = *items[i].p;
        if (done[i] || p.device() != p0.device()) continue;
        if (p.scalar_type() != at::kFloat) {
          if (low != at::kFloat && p.scalar_type() != low) continue;
          low = p.scalar_type();
        }
        done[i] = 1;
        const CallView c = view(*items[i].e, p, items[i].g, momentum);
        for (int a = 0; a < nt; ++a) {
          ptr[a].push_back(c.t[a] ? c.t[a]->data_ptr() : nullptr);
          has[a].push_back(c.t[a] != nullptr);
        }
        if (p.scalar_type() == at::kFloat) ptr[nt - 1].back() = nullptr;  // no Kahan buffer for fp32
        numel.push_back(p.numel());
        dtypes.push_back(dtype_code(p));
      }
      // an absent array must be absent for every tensor of the launch (the Kahan buffer: for every 16-bit one)
      for (int a = 2; a < nt; ++a) {
        int present = -1;
        for (size_t i = 0; i < ptr[a].size(); ++i) {
          if (a == nt - 1 && dtypes[i] == OPTIMI_F32) continue;
          const int here = has[a][i];
          TORCH_CHECK(present < 0 || present == here, "optimi_amd: a state buffer is missing for some parameters of a group");
          present = here;
        }
      }
      c10::hip::HIPGuardMasqueradingAsCUDA guard(p0.device());
      // one workspace per parameter group (and device, and 16-bit dtype): its device tables then hold
      // this group's list from one step to the next and are uploaded once, however many groups
      // the optimizer steps in between
      std::unique_ptr<Group>& slot = workspaces_[{grp, (int)p0.device().index(), (int)low}];
      if (!slot) slot = std::make_unique<Group>();
      launch_list(kind_, slot->get(), (int)numel.size(), ptr, numel.data(), dtypes.data(), h.s,
                  h.flags | (resident ? (uint32_t)OPTIMI_RESIDENT : 0u),
                  c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(p0.device().index()).stream());
    }
    return true;
  }

 private:
  struct Entry {
    c10::weak_intrusive_ptr<c10::TensorImpl> param;  // weak: a hook must not keep its parameter alive
    py::object state, group, workspace_obj;
    Group* workspace = nullptr;
    PyObject* ids[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    PyObject* step_id = nullptr;
    bool release = false;  // made for the gradient-release hook (group and step counter cached too)
    uint64_t state_version = 0;    // the state dict's version tag when the cached tensors were last checked against it
    bool checked_release = false;  // that check covered the group and the step counter too
    std::optional<at::Tensor> t[5];
    at::Tensor step;
    explicit Entry(const at::Tensor& p) : param(p.getIntrusivePtr()) {}
  };

  struct Names {
    py::str release{"_release"}, entry{"_release_entry"}, accumulation{"_optimizer_accumulation"}, group{"group"}, step{"step"};
    py::str lr{"lr"}, beta1{"beta1"}, beta2{"beta2"}, beta3{"beta3"}, weight_decay{"weight_decay"}, eps{"eps"};
    py::str decouple_wd{"decouple_wd"}, decouple_lr{"decouple_lr"}, max_lr{"max_lr"}, kahan_sum{"kahan_sum"};
    py::str momentum{"momentum"}, dampening{"dampening"}, k{"k"}, alpha{"alpha"};
    py::str setup{"setup"}, triton{"triton"}, params{"params"}, group_entry{"_group_entry"};
  };

  static PyObject* attr(PyObject* obj, const py::str& name) {
    PyObject* v = PyObject_GetAttr(obj, name.ptr());
    if (!v) throw py::error_already_set();
    return v;  // new reference
  }
  static PyObject* item(PyObject* dict, const py::str& key) {
    PyObject* v = PyDict_GetItemWithError(dict, key.ptr());  // borrowed
    if (!v) {
      if (PyErr_Occurred()) throw py::error_already_set();
      TORCH_CHECK(false, "optimi_amd: '", std::string(key), "' is missing from the parameter group");
    }
    return v;
  }
  // Values that can change without the dict that holds them changing (a tensor learning rate
  // filled in place, a user's own number type) must be read afresh on every call.
  static inline thread_local bool read_only_immutables_ = true;
  static double as_double(PyObject* v) {
    if (!PyFloat_CheckExact(v) && !PyLong_CheckExact(v)) read_only_immutables_ = false;
    const double d = PyFloat_AsDouble(v);
    if (d == -1.0 && PyErr_Occurred()) throw py::error_already_set();
    return d;
  }
  static bool truthy(PyObject* v) {
    if (v != Py_True && v != Py_False && v != Py_None) read_only_immutables_ = false;
    const int r = PyObject_IsTrue(v);
    if (r < 0) throw py::error_already_set();
    return r == 1;
  }
  static double num(PyObject* dict, const py::str& key) { return as_double(item(dict, key)); }
  static bool flag(PyObject* dict, const py::str& key) { return truthy(item(dict, key)); }
  static std::optional<double> opt_num(PyObject* dict, const py::str& key) {
    PyObject* v = item(dict, key);
    if (v == Py_None) return std::nullopt;
    return as_double(v);
  }

  // SGD keeps a momentum buffer in its state even when momentum is 0; it is not passed then
  double momentum_of(PyObject* grp) const { return kind_ == SGD ? num(grp, k_.momentum) : 1.0; }

  // A dict's version tag changes whenever the dict is modified (a key added or removed, a value
  // replaced by another object), so an unchanged tag means that everything read from the dict
  // before still holds.  0 = not available on this interpreter: nothing is cached then.
  static uint64_t dict_version(PyObject* dict) {
#if PY_VERSION_HEX < 0x030C0000
    return ((PyDictObject*)dict)->ma_version_tag;
#else
    (void)dict;
    return 0;
#endif
  }

  // The step scalars of a group at step count `t`.  Every parameter of a group shares them, so
  // they are formed once (a dozen dict reads and two or three pow() calls) and reused for as long as
  // the group dict is unmodified and the step count and the kind of step are the same - a
  // scheduler that rewrites group["lr"] changes the dict's version tag and is seen at once.
  const Hyper& hyper_for(PyObject* grp, int64_t t, bool update) {
    const uint64_t version = dict_version(grp);
    HyperSlot* slot = nullptr;
    for (HyperSlot& s : hyper_cache_)
      if (s.group == grp) slot = &s;
    if (!slot) {
      hyper_cache_.emplace_back();
      slot = &hyper_cache_.back();
      slot->group = grp;
      slot->version = 0;
    }
    if (version == 0 || slot->version != version || slot->t != t || slot->update != update) {
      slot->version = 0;  // void while it is being rebuilt (read_hyper may throw)
      read_only_immutables_ = true;
      slot->h = read_hyper(grp, t, update);
      slot->t = t;
      slot->update = update;
      slot->version = read_only_immutables_ ? version : 0;  // 0: read again next time
    }
    return slot->h;
  }

  Hyper read_hyper(PyObject* grp, int64_t t, bool update) const {
    switch (kind_) {
      case ADAM:
        return adam_hyper(t, num(grp, k_.lr), num(grp, k_.beta1), num(grp, k_.beta2), num(grp, k_.weight_decay), num(grp, k_.eps),
                          flag(grp, k_.decouple_wd), flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr), flag(grp, k_.kahan_sum), update);
      case LION:
        return lion_hyper(num(grp, k_.lr), num(grp, k_.beta1), num(grp, k_.beta2), num(grp, k_.weight_decay),
                          flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr), flag(grp, k_.kahan_sum), update);
      case STABLEADAMW:
        return stableadamw_hyper(t, num(grp, k_.lr), num(grp, k_.beta1), num(grp, k_.beta2), num(grp, k_.weight_decay),
                                 num(grp, k_.eps), flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr), flag(grp, k_.kahan_sum), update);
      case ADAN:  // adam_wd is not forwarded by the reference's class either (optimi/adan.py:186-208)
        return adan_hyper(t, num(grp, k_.lr), num(grp, k_.beta1), num(grp, k_.beta2), num(grp, k_.beta3), num(grp, k_.weight_decay),
                          num(grp, k_.eps), flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr), false, flag(grp, k_.kahan_sum), update);
      case SGD:
        return sgd_hyper(num(grp, k_.lr), num(grp, k_.momentum), num(grp, k_.weight_decay), flag(grp, k_.dampening),
                         flag(grp, k_.decouple_wd), flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr), flag(grp, k_.kahan_sum), update);
      case RADAM:
        return ranger_hyper(t, false, num(grp, k_.lr), num(grp, k_.beta1), num(grp, k_.beta2), num(grp, k_.weight_decay),
                            num(grp, k_.eps), 1, 0.0, flag(grp, k_.decouple_wd), flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr),
                            flag(grp, k_.kahan_sum), update);
      case RANGER:
        return ranger_hyper(t, true, num(grp, k_.lr), num(grp, k_.beta1), num(grp, k_.beta2), num(grp, k_.weight_decay),
                            num(grp, k_.eps), (int64_t)num(grp, k_.k), num(grp, k_.alpha), flag(grp, k_.decouple_wd),
                            flag(grp, k_.decouple_lr), opt_num(grp, k_.max_lr), flag(grp, k_.kahan_sum), update);
    }
    TORCH_CHECK(false, "optimi_amd: unknown optimizer kind");
  }

  // The step of one parameter in the ABI's tensor order: param, grad, the states, the Kahan buffer last.
  StepCall pack(const Entry& e, const Hyper& h, const at::Tensor& p, const at::Tensor& g, double momentum) const {
    StepCall c;
    c.kind = kind_;
    c.flags = h.flags;
    std::memcpy(c.s, h.s, sizeof(c.s));
    c.t[0] = p;
    c.t[1] = g;
    const size_t n = state_keys_.size();
    for (size_t i = 0; i < n; ++i) {
      const bool placeholder_possible = i + 1 == n || kind_ == SGD;  // Kahan buffer; SGD's momentum buffer
      c.t[2 + i] = placeholder_possible ? real_kahan(p, e.t[i]) : e.t[i];
    }
    if (kind_ == SGD && momentum == 0) c.t[2] = std::nullopt;
    return c;
  }

  // The same without owning anything, for the whole-group walk: the tensors stay where they are (the
  // parameter list, the entries' cached states, the gradients the parameters hold) for the
  // length of the call, so pointers to them do; null = absent.
  struct CallView {
    const at::Tensor* t[kMaxTensors] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
  };
  CallView view(const Entry& e, const at::Tensor& p, const at::Tensor& g, double momentum) const {
    CallView c;
    c.t[0] = &p;
    c.t[1] = &g;
    const size_t n = state_keys_.size();
    for (size_t i = 0; i < n; ++i) {
      const std::optional<at::Tensor>& s = e.t[i];
      if (!s.has_value()) continue;
      const bool placeholder_possible = i + 1 == n || kind_ == SGD;  // Kahan buffer; SGD's momentum buffer
      if (placeholder_possible && (!s->defined() || s->numel() != p.numel() || s->scalar_type() != p.scalar_type())) continue;
      c.t[2 + i] = &*s;
    }
    if (kind_ == SGD && momentum == 0) c.t[2] = nullptr;
    return c;
  }
  // what validate_call checks
  void validate_view(const CallView& c) const {
    static const char* const names[] = {"param", "grad", "state", "state", "state", "state", "state"};
    const at::Tensor& p = *c.t[0];
    check_param(p);
    (void)dtype_code(p);
    for (int a = 1; a < kTensorsOf[kind_]; ++a)
      if (c.t[a]) check_like(p, *c.t[a], names[a]);
  }

  void rebind() {
    hook_tables_.clear();
    py::object optimizer = optimizer_();
    if (optimizer.is_none()) return;
    py::module_ mod = py::module_::import("torch.optim.optimizer");
    hook_tables_.push_back(optimizer.attr("_optimizer_step_pre_hooks"));
    hook_tables_.push_back(optimizer.attr("_optimizer_step_post_hooks"));
    hook_tables_.push_back(mod.attr("_global_optimizer_pre_hooks"));
    hook_tables_.push_back(mod.attr("_global_optimizer_post_hooks"));
  }

  bool any_step_hooks() const {
    for (const py::object& table : hook_tables_) {
      const Py_ssize_t n = PyObject_Length(table.ptr());
      if (n < 0) throw py::error_already_set();
      if (n > 0) return true;
    }
    return false;
  }

  Entry* find(const at::Tensor& p) {
    auto it = entries_.find(p.unsafeGetTensorImpl());
    if (it == entries_.end()) return nullptr;
    if (it->second.param.expired()) {  // another tensor lives at that address now
      entries_.erase(it);
      return nullptr;
    }
    return &it->second;
  }

  // every cached tensor is still the object the state dict holds
  // (`release`: also the group and the per-parameter step counter that gradient release keeps there)
  // (an unmodified state dict - same version tag as when it was last checked - needs no look-ups)
  bool valid(Entry& e, bool release = true) const {
    PyObject* st = e.state.ptr();
    if (release && !e.release) return false;
    const uint64_t version = dict_version(st);
    if (version != 0 && version == e.state_version && e.checked_release >= release) return true;
    for (size_t i = 0; i < state_keys_.size(); ++i)
      if (PyDict_GetItemWithError(st, state_keys_[i].ptr()) != e.ids[i]) return false;
    if (release) {
      if (PyDict_GetItemWithError(st, k_.group.ptr()) != e.group.ptr()) return false;
      if (has_step_ && PyDict_GetItemWithError(st, k_.step.ptr()) != e.step_id) return false;
    }
    e.state_version = version;
    e.checked_release = release;
    return true;
  }

  Entry* refresh(const py::object& optimizer, const py::str& method, const py::handle& param_h, const at::Tensor& p,
                 bool release, const py::handle& group = py::handle()) {
    PyErr_Clear();
    // (state dict, group dict, launch workspace or None), state created and the backend checked
    py::tuple made = group ? optimizer.attr(method)(param_h, group) : optimizer.attr(method)(param_h);
    Entry e(p);
    e.release = release;
    e.state = made[0];
    e.group = made[1];
    e.workspace_obj = made[2];
    TORCH_CHECK(PyDict_Check(e.state.ptr()) && PyDict_Check(e.group.ptr()), "optimi_amd: state and group must be dicts");
    if (!e.workspace_obj.is_none()) e.workspace = &e.workspace_obj.cast<Group&>();
    TORCH_CHECK(kind_ != STABLEADAMW || e.workspace || !release, "optimi_amd: StableAdamW needs a launch workspace");
    for (size_t i = 0; i < state_keys_.size(); ++i) {
      PyObject* v = PyDict_GetItemWithError(e.state.ptr(), state_keys_[i].ptr());
      TORCH_CHECK(v, "optimi_amd: optimizer state has no '", std::string(state_keys_[i]), "'");
      e.ids[i] = v;
      if (v != Py_None) {
        TORCH_CHECK(THPVariable_Check(v), "optimi_amd: state '", std::string(state_keys_[i]), "' is not a tensor");
        e.t[i] = THPVariable_Unpack(v);
      }
    }
    // all but the last key (the Kahan buffer) and SGD's momentum buffer must be tensors
    for (size_t i = 0; i + 1 < state_keys_.size(); ++i)
      TORCH_CHECK(e.t[i].has_value() || kind_ == SGD, "optimi_amd: state '", std::string(state_keys_[i]), "' is None");
    if (has_step_ && release) {
      PyObject* v = PyDict_GetItemWithError(e.state.ptr(), k_.step.ptr());
      TORCH_CHECK(v && THPVariable_Check(v), "optimi_amd: the per-parameter step counter is missing");
      e.step_id = v;
      e.step = THPVariable_Unpack(v);
    }
    auto placed = entries_.insert_or_assign(p.unsafeGetTensorImpl(), std::move(e));
    return &placed.first->second;
  }

  py::weakref optimizer_;
  Kind kind_;
  std::shared_ptr<ReleaseQueue> queue_;
  bool has_step_ = true;
  Names k_;
  std::vector<py::str> state_keys_;
  std::vector<py::object> hook_tables_;
  std::unordered_map<c10::TensorImpl*, Entry> entries_;
  struct HyperSlot {
    PyObject* group = nullptr;
    uint64_t version = 0;
    int64_t t = 0;
    bool update = false;
    Hyper h;
  };
  std::vector<HyperSlot> hyper_cache_;  // one slot per parameter group seen
  int pass_task_ = -1;                  // the backward pass pass_hooks_ and pass_update_ were read in
  bool pass_hooks_ = false, pass_update_ = true;
  struct WorkspaceKey {
    PyObject* group;  // the parameter group's dict (an address only, never dereferenced)
    int device, low;  // the list's device and its 16-bit dtype (float for an all-fp32 list)
    bool operator==(const WorkspaceKey& o) const { return group == o.group && device == o.device && low == o.low; }
  };
  struct WorkspaceHash {
    size_t operator()(const WorkspaceKey& k) const {
      return std::hash<const void*>()(k.group) ^ (std::hash<int64_t>()(((int64_t)k.device << 32) ^ (int64_t)k.low) * 0x9e3779b97f4a7c15ull);
    }
  };
  std::unordered_map<WorkspaceKey, std::unique_ptr<Group>, WorkspaceHash> workspaces_;  // the launch tables of each list
};

// What is registered on the parameters: a handle that does not own the hook, so that
// parameter -> hook -> cached state -> group -> parameter is not a cycle the garbage
// collector cannot see.  The optimizer owns the ReleaseHookCore.
// The handle is a bare CPython type whose tp_call goes straight to ReleaseHookCore::call: the
// autograd engine calls it once per parameter per backward pass, and a pybind11 method call
// (overload resolution, argument casters) costs several hundred nanoseconds that a model with
// thousands of small tensors pays thousands of times.
struct ReleaseHookObject {
  PyObject_HEAD
  std::weak_ptr<ReleaseHookCore>* core;
};

PyObject* release_hook_call(PyObject* self, PyObject* args, PyObject* kwargs) {
  HANDLE_TH_ERRORS
  TORCH_CHECK(PyTuple_GET_SIZE(args) == 1 && (!kwargs || PyDict_GET_SIZE(kwargs) == 0),
              "optimi_amd: the gradient release hook takes the parameter and nothing else");
  std::shared_ptr<ReleaseHookCore> core = ((ReleaseHookObject*)self)->core->lock();
  TORCH_CHECK(core, "optimi_amd: the optimizer of this gradient release hook no longer exists");
  core->call(py::handle(PyTuple_GET_ITEM(args, 0)));
  Py_RETURN_NONE;
  END_HANDLE_TH_ERRORS
}

void release_hook_dealloc(PyObject* self) {
  delete ((ReleaseHookObject*)self)->core;
  Py_TYPE(self)->tp_free(self);
}

PyTypeObject ReleaseHookType = {PyVarObject_HEAD_INIT(nullptr, 0)};

bool init_release_hook_type() {
  ReleaseHookType.tp_name = "optimi_amd._C.ReleaseHook";
  ReleaseHookType.tp_basicsize = sizeof(ReleaseHookObject);
  ReleaseHookType.tp_flags = Py_TPFLAGS_DEFAULT;
  ReleaseHookType.tp_doc = "post-accumulate-grad hook of one optimizer (callable with the parameter)";
  ReleaseHookType.tp_call = release_hook_call;
  ReleaseHookType.tp_dealloc = release_hook_dealloc;
  return PyType_Ready(&ReleaseHookType) == 0;
}

py::object make_release_hook(const std::shared_ptr<ReleaseHookCore>& core) {
  PyObject* obj = ReleaseHookType.tp_alloc(&ReleaseHookType, 0);
  if (!obj) throw py::error_already_set();
  ((ReleaseHookObject*)obj)->core = new std::weak_ptr<ReleaseHookCore>(core);
  return py::reinterpret_steal<py::object>(obj);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
  mod.doc() = "PyTorch-ROCm binding of the optimi_hip C ABI";
  mod.attr("KAHAN") = (uint32_t)OPTIMI_KAHAN;
  mod.attr("UPDATE") = (uint32_t)OPTIMI_UPDATE;
  mod.attr("DECOUPLE_WD") = (uint32_t)OPTIMI_DECOUPLE_WD;
  mod.attr("ADAM_WD") = (uint32_t)OPTIMI_ADAM_WD;
  mod.attr("DECOUPLE_LR") = (uint32_t)OPTIMI_DECOUPLE_LR;
  mod.attr("DAMPENING") = (uint32_t)OPTIMI_DAMPENING;
  mod.attr("RECTIFY") = (uint32_t)OPTIMI_RECTIFY;
  mod.attr("LOOKAHEAD") = (uint32_t)OPTIMI_LOOKAHEAD;
  mod.attr("RESIDENT") = (uint32_t)OPTIMI_RESIDENT;
  mod.def("resident_bytes", &optimi_hip_resident_bytes);
  mod.def("abi_version", &optimi_hip_version);
  py::class_<Group>(mod, "Group").def(py::init<>());
  py::class_<ReleaseHookCore, std::shared_ptr<ReleaseHookCore>>(mod, "ReleaseHookCore")
      .def(py::init<const py::object&, int, std::shared_ptr<ReleaseQueue>>(), py::arg("optimizer"), py::arg("kind"), py::arg("queue"))
      .def("invalidate", &ReleaseHookCore::invalidate)
      .def("step_group", &ReleaseHookCore::step_group, py::arg("group"), py::arg("resident") = false)
      .def("__call__", &ReleaseHookCore::call);
  if (!init_release_hook_type()) throw py::error_already_set();
  mod.def("ReleaseHook", &make_release_hook, py::arg("core"));
  mod.attr("KIND_ADAM") = (int)ADAM;
  mod.attr("KIND_LION") = (int)LION;
  mod.attr("KIND_STABLEADAMW") = (int)STABLEADAMW;
  mod.attr("KIND_ADAN") = (int)ADAN;
  mod.attr("KIND_SGD") = (int)SGD;
  mod.attr("KIND_RADAM") = (int)RADAM;
  mod.attr("KIND_RANGER") = (int)RANGER;
  py::class_<ReleaseQueue, std::shared_ptr<ReleaseQueue>>(mod, "ReleaseQueue")
      .def(py::init<int64_t, int64_t, int64_t>(), py::arg("max_numel"), py::arg("max_tensors"), py::arg("max_total_bytes"))
      .def("flush", [](ReleaseQueue& q) { q.flush(); })
      .def("pending", &ReleaseQueue::pending)
      .def("launches", &ReleaseQueue::launches)
      .def("launched_steps", &ReleaseQueue::launched_steps);
  mod.def("adam_multi", &adam_multi);
  mod.def("lion_multi", &lion_multi);
  mod.def("stableadamw_multi", &stableadamw_multi);
  mod.def("adan_multi", &adan_multi);
  mod.def("adam_single", &adam_single);
  mod.def("lion_single", &lion_single);
  mod.def("stableadamw_single", &stableadamw_single);
  mod.def("adan_single", &adan_single);
  mod.def("adam_release", &adam_release);
  mod.def("lion_release", &lion_release);
  mod.def("stableadamw_release", &stableadamw_release);
  mod.def("adan_release", &adan_release);
  mod.def("debias_beta", &debias_beta);
  mod.def("rectification", &rectification);
  mod.def("sgd_multi", &sgd_multi);
  mod.def("radam_multi", &radam_multi);
  mod.def("ranger_multi", &ranger_multi);
  mod.def("sgd_single", &sgd_single);
  mod.def("radam_single", &radam_single);
  mod.def("ranger_single", &ranger_single);
  mod.def("sgd_release", &sgd_release);
  mod.def("ranger_release", &ranger_release);
}
