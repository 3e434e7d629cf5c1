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
#include <torch/extension.h>

#include <cmath>
#include <optional>
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

// Kahan buffers: taken only when the Kahan branch runs; placeholders and None are ignored.
PtrList gather_kahan(const TensorList& params, const OptTensorList& list, bool needed) {
  PtrList out;
  if (!needed) return out;
  TORCH_CHECK(list.size() == params.size(), "optimi_amd: kahan_comps has ", list.size(), " tensors, params has ", params.size());
  out.v.reserve(list.size());
  for (size_t i = 0; i < list.size(); ++i) {
    TORCH_CHECK(list[i].has_value(), "optimi_amd: kahan_sum is on but a Kahan buffer is missing");
    check_like(params[i], *list[i], "kahan_comp");
    out.v.push_back(list[i]->data_ptr());
  }
  return out;
}

struct Prepared {
  int dtype = OPTIMI_F32;
  bool kahan = false;
  std::vector<int64_t> numel;
  PtrList params;
};

Prepared prepare(const TensorList& params, uint32_t flags) {
  Prepared pr;
  if (params.empty()) return pr;
  pr.dtype = dtype_code(params[0]);
  pr.kahan = pr.dtype != OPTIMI_F32 && (flags & OPTIMI_KAHAN) && (flags & OPTIMI_UPDATE);
  pr.numel.reserve(params.size());
  pr.params.v.reserve(params.size());
  for (const at::Tensor& p : params) {
    check_param(p);
    TORCH_CHECK(p.device() == params[0].device(), "optimi_amd: one launch covers one device");
    TORCH_CHECK(p.scalar_type() == params[0].scalar_type(), "optimi_amd: one launch covers one dtype");
    pr.numel.push_back(p.numel());
    pr.params.v.push_back(p.data_ptr());
  }
  return pr;
}

void adam_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                const TensorList& exp_avg_sqs, const OptTensorList& kahan_comps, double lr, double beta1_comp,
                double beta2_hat, double beta2_comp, double weight_decay, double eps, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_adam_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                     pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtype, lr, beta1_comp, beta2_hat,
                                     beta2_comp, weight_decay, eps, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_adam_multi");
}

void lion_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                const OptTensorList& kahan_comps, double lr, double beta1_comp, double beta2_comp, double weight_decay,
                uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg");
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_lion_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(),
                                     pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtype, lr, beta1_comp, beta2_comp,
                                     weight_decay, flags, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_lion_multi");
}

void stableadamw_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                       const TensorList& exp_avg_sqs, const OptTensorList& kahan_comps, double lr, double beta1_comp,
                       double beta2_hat, double beta2_comp, double weight_decay, double eps, double max_lr,
                       uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_stableadamw_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                            pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtype, lr, beta1_comp,
                                            beta2_hat, beta2_comp, weight_decay, eps, max_lr, flags,
                                            c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_stableadamw_multi");
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
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_adan_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), df.data(),
                                     n.data(), pg.data(), pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtype, lr,
                                     beta1_comp, beta2, beta2_comp, beta3_hat, beta3_comp, eps, weight_decay, flags,
                                     c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_adan_multi");
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
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_sgd_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(),
                                    momentum != 0 ? m.data() : nullptr, pr.kahan ? k.data() : nullptr, pr.numel.data(),
                                    pr.dtype, lr, momentum, weight_decay, flags,
                                    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_sgd_multi");
}

void radam_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                 const TensorList& exp_avg_sqs, const OptTensorList& kahan_comps, double lr, double beta1_comp,
                 double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_radam_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                      pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtype, lr, beta1_comp, beta2_hat,
                                      beta2_comp, weight_decay, eps, rect, flags,
                                      c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_radam_multi");
}

void ranger_multi(Group& group, const TensorList& params, const TensorList& grads, const TensorList& exp_avgs,
                  const TensorList& exp_avg_sqs, const TensorList& la_params, const OptTensorList& kahan_comps, double lr,
                  double beta1_comp, double beta2_hat, double beta2_comp, double weight_decay, double eps, double rect,
                  double alpha, uint32_t flags) {
  if (params.empty()) return;
  Prepared pr = prepare(params, flags);
  PtrList g = gather(params, grads, "grad"), m = gather(params, exp_avgs, "exp_avg"), v = gather(params, exp_avg_sqs, "exp_avg_sq");
  PtrList la = gather(params, la_params, "la_param");
  PtrList k = gather_kahan(params, kahan_comps, pr.kahan);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(params[0].device());
  check_status(optimi_hip_ranger_multi(group.get(), (int)params.size(), pr.params.data(), g.cdata(), m.data(), v.data(),
                                       la.data(), pr.kahan ? k.data() : nullptr, pr.numel.data(), pr.dtype, lr, beta1_comp,
                                       beta2_hat, beta2_comp, weight_decay, eps, rect, alpha, flags,
                                       c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream()),
               "optimi_hip_ranger_multi");
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


// ---- gradient-release fast path --------------------------------------------------------
// One call per parameter from the post-accumulate-grad hook: advances the parameter's int32
// CPU step counter, forms the step scalars in double exactly as the functional forms do in
// Python (optimi/adam.py:260-273, lion.py:226-235, stableadamw.py:326-332, adan.py:289-309)
// and launches the per-tensor kernel.  std::pow(double, double) is libm's pow, the function
// CPython's float ** int ends in, so the scalars are bit-identical to the Python path.

double debias_beta(double beta, int64_t step) {  // optimi/utils.py:31-36
  const double bt = std::pow(beta, (double)step);
  return (bt - beta) / (bt - 1.0);
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

void adam_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                  const std::optional<at::Tensor>& k, const at::Tensor& step, double lr, double beta1, double beta2,
                  double weight_decay, double eps, bool decouple_wd, bool decouple_lr, std::optional<double> max_lr,
                  bool kahan_sum, bool update) {
  const int64_t t = tick(step);
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t);
  if (weight_decay != 0) {
    if (decouple_lr) weight_decay = 1 - (lr / max_lr.value()) * weight_decay;
    else if (decouple_wd) weight_decay = 1 - lr * weight_decay;
  }
  const uint32_t flags = base_flags(kahan_sum, update) | ((decouple_wd || decouple_lr) ? OPTIMI_DECOUPLE_WD : 0u);
  adam_single(p, grad_like(p, g), m, v, real_kahan(p, k), lr, 1 - b1h, b2h, 1 - b2h, weight_decay, eps, flags);
}

void lion_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const std::optional<at::Tensor>& k,
                  double lr, double beta1, double beta2, double weight_decay, bool decouple_lr,
                  std::optional<double> max_lr, bool kahan_sum, bool update) {
  if (weight_decay != 0) weight_decay = decouple_lr ? 1 - (lr / max_lr.value()) * weight_decay : 1 - lr * weight_decay;
  lion_single(p, grad_like(p, g), m, real_kahan(p, k), lr, 1 - beta1, 1 - beta2, weight_decay, base_flags(kahan_sum, update));
}

void stableadamw_release(Group& group, const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                         const std::optional<at::Tensor>& k, const at::Tensor& step, double lr, double beta1, double beta2,
                         double weight_decay, double eps, bool decouple_lr, std::optional<double> max_lr, bool kahan_sum,
                         bool update) {
  const int64_t t = tick(step);
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t);
  const uint32_t flags = base_flags(kahan_sum, update) | (decouple_lr ? OPTIMI_DECOUPLE_LR : 0u);
  stableadamw_single(group, p, grad_like(p, g), m, v, real_kahan(p, k), lr, 1 - b1h, b2h, 1 - b2h, weight_decay, eps,
                     (decouple_lr && max_lr.has_value()) ? *max_lr : 0.0, flags);
}

void adan_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& df, const at::Tensor& n,
                  const at::Tensor& pg, const std::optional<at::Tensor>& k, const at::Tensor& step, double lr, double beta1,
                  double beta2, double beta3, double weight_decay, double eps, bool decouple_lr, std::optional<double> max_lr,
                  bool adam_wd, bool kahan_sum, bool update) {
  const int64_t t = tick(step);
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t), b3h = debias_beta(beta3, t);
  if (weight_decay != 0) {
    weight_decay = decouple_lr ? (lr / max_lr.value()) * weight_decay : lr * weight_decay;
    weight_decay = adam_wd ? 1 - weight_decay : 1 + weight_decay;
  }
  const uint32_t flags = base_flags(kahan_sum, update) | (adam_wd ? OPTIMI_ADAM_WD : 0u);
  adan_single(p, grad_like(p, g), m, df, n, pg, real_kahan(p, k), lr, 1 - b1h, beta2, 1 - b2h, b3h, 1 - b3h, eps, weight_decay,
              flags);
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

// RAdam's variance rectification term; negative = not yet rectified (optimi/radam.py:269-277).
double rectification(double beta2, int64_t step) {
  const double rho_inf = 2 / (1 - beta2) - 1;
  const double bt = std::pow(beta2, (double)step);
  const double rho = rho_inf - 2 * (double)step * bt / (1 - bt);
  if (rho > 5) return std::sqrt(((rho - 4) * (rho - 2) * rho_inf) / ((rho_inf - 4) * (rho_inf - 2) * rho));
  return -1.0;
}

void sgd_release(const at::Tensor& p, const at::Tensor& g, const std::optional<at::Tensor>& m,
                 const std::optional<at::Tensor>& k, double lr, double momentum, double weight_decay, bool dampening,
                 bool decouple_wd, bool decouple_lr, std::optional<double> max_lr, bool kahan_sum, bool update) {
  if (weight_decay != 0) {
    if (decouple_lr) weight_decay = 1 - (lr / max_lr.value()) * weight_decay;
    else if (decouple_wd) weight_decay = 1 - lr * weight_decay;
  }
  const uint32_t flags = base_flags(kahan_sum, update) | ((decouple_wd || decouple_lr) ? OPTIMI_DECOUPLE_WD : 0u) |
                         (dampening ? OPTIMI_DAMPENING : 0u);
  sgd_single(p, grad_like(p, g), momentum != 0 ? real_kahan(p, m) : std::nullopt, real_kahan(p, k), lr, momentum, weight_decay, flags);
}

void ranger_release(const at::Tensor& p, const at::Tensor& g, const at::Tensor& m, const at::Tensor& v,
                    const std::optional<at::Tensor>& la, const std::optional<at::Tensor>& k, const at::Tensor& step, double lr,
                    double beta1, double beta2, double weight_decay, double eps, int64_t sync_every, double alpha,
                    bool decouple_wd, bool decouple_lr, std::optional<double> max_lr, bool kahan_sum, bool update) {
  // la = None makes this RAdam (optimi/radam.py:214-322); with la it is Ranger (optimi/ranger.py:230-344)
  const int64_t t = tick(step);
  const double b1h = debias_beta(beta1, t), b2h = debias_beta(beta2, t);
  const double rect = rectification(beta2, t);
  if (weight_decay != 0) {
    if (decouple_lr) weight_decay = 1 - (lr / max_lr.value()) * weight_decay;
    else if (decouple_wd) weight_decay = 1 - lr * weight_decay;
  }
  uint32_t flags = base_flags(kahan_sum, update) | ((decouple_wd || decouple_lr) ? OPTIMI_DECOUPLE_WD : 0u) |
                   (rect >= 0 ? OPTIMI_RECTIFY : 0u);
  if (la.has_value()) {
    if (t % sync_every == 0) flags |= OPTIMI_LOOKAHEAD;
    ranger_single(p, grad_like(p, g), m, v, *la, real_kahan(p, k), lr, 1 - b1h, b2h, 1 - b2h, weight_decay, eps,
                  rect >= 0 ? rect : 0.0, alpha, flags);
  } else {
    radam_single(p, grad_like(p, g), m, v, real_kahan(p, k), lr, 1 - b1h, b2h, 1 - b2h, weight_decay, eps,
                 rect >= 0 ? rect : 0.0, flags);
  }
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
  mod.def("abi_version", &optimi_hip_version);
  py::class_<Group>(mod, "Group").def(py::init<>());
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
