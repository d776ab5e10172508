#include "optim.h"

#include <cmath>
#include <cstdint>

#include "../../include/deers_rocm.h"

namespace deers_host {

AdamW AdamWConfig::build(std::vector<Tensor> parameters) const {
  AdamW opt;
  opt.parameters_ = std::move(parameters);
  opt.lr_ = lr;
  opt.beta1_ = betas_.first;
  opt.beta2_ = betas_.second;
  opt.eps_ = eps_;
  opt.weight_decay_ = weight_decay_;
  return opt;
}

std::optional<std::pair<Tensor, Tensor>> AdamW::state_for(const Tensor& parameter) const {
  auto m = m_.find(parameter.id());
  auto v = v_.find(parameter.id());
  if (m == m_.end() || v == v_.end()) return std::nullopt;
  return std::make_pair(m->second, v->second);
}

void AdamW::load_state_for(const Tensor& parameter, Tensor m, Tensor v) {
  m_[parameter.id()] = m.detach();
  v_[parameter.id()] = v.detach();
}

void AdamW::backward_step(const Tensor& loss) {
  GradientStore grads = loss.backward();
  step_with_grads(grads);
}

void AdamW::step_with_grads(const GradientStore& grads, double grad_scale) {
  step_ += 1;  // src/optim.rs:215
  // every parameter that has a gradient, gathered per type for the multi-tensor launch
  // (the compacted gradients are kept alive in `held` until the launches are enqueued)
  struct Group {
    std::vector<void*> w, m, v;
    std::vector<const void*> g;
    std::vector<int64_t> n;
  };
  Group groups[2];
  std::vector<Tensor> held;
  for (const Tensor& param : parameters_) {
    const Tensor* found = grads.get(param.id());
    if (!found) continue;
    if (!param.is_compact()) throw std::logic_error("AdamW: parameters must be compact");
    if (found->shape() != param.shape() || found->dtype() != param.dtype())
      throw std::logic_error("AdamW: gradient does not match its parameter");
    if (param.dtype() != DType::F16 && param.dtype() != DType::F32)
      throw std::logic_error("AdamW: parameters are f16 or f32");
    held.push_back(found->compact());
    auto m = m_.find(param.id());
    if (m == m_.end()) m = m_.emplace(param.id(), param.zeros_like()).first;
    auto v = v_.find(param.id());
    if (v == v_.end()) v = v_.emplace(param.id(), param.zeros_like()).first;
    Group& grp = groups[param.dtype() == DType::F16 ? 0 : 1];
    grp.w.push_back(param.data());
    grp.g.push_back(held.back().data());
    grp.m.push_back(m->second.data());
    grp.v.push_back(v->second.data());
    grp.n.push_back((int64_t)param.layout().size());
  }
  for (int t = 0; t < 2; ++t) {
    const Group& grp = groups[t];
    if (grp.w.empty()) continue;
    check(deers_rocm_adamw_step_multi(t == 0 ? DEERS_ROCM_F16 : DEERS_ROCM_F32, (int)grp.w.size(),
                                      grp.w.data(), grp.g.data(), grp.m.data(), grp.v.data(), grp.n.data(),
                                      lr_, beta1_, beta2_, eps_, weight_decay_, (int64_t)step_, grad_scale));
  }
}

float clip_grad_scale(const std::vector<Tensor>& parameters, const GradientStore& grads,
                      double max_norm, double* scale) {
  if (!(max_norm > 0.0)) throw std::logic_error("max_norm must be positive");
  if (scale) *scale = 1.0;
  if (parameters.empty()) return 0.0f;
  Tensor total = Tensor::zeros({1}, DType::F32);
  // all gradients of a type in one reduction; one that is not 16-byte aligned (a view
  // into a larger buffer) goes through the single-tensor call
  std::vector<Tensor> held;
  std::vector<const void*> ptrs[2];
  std::vector<int64_t> sizes[2];
  for (const Tensor& p : parameters) {
    const Tensor* g = grads.get(p.id());
    if (!g) continue;
    held.push_back(g->compact());
    const Tensor& gc = held.back();
    const int64_t n = (int64_t)gc.layout().size();
    if (n == 0) continue;
    if ((uintptr_t)gc.data() & 15) {
      check(deers_rocm_sum_squares((int)gc.dtype(), gc.data(), n, (float*)total.data(), 1));
      continue;
    }
    const int t = gc.dtype() == DType::F16 ? 0 : 1;
    ptrs[t].push_back(gc.data());
    sizes[t].push_back(n);
  }
  for (int t = 0; t < 2; ++t)
    if (!ptrs[t].empty())
      check(deers_rocm_sum_squares_multi(t == 0 ? DEERS_ROCM_F16 : DEERS_ROCM_F32, (int)ptrs[t].size(),
                                         ptrs[t].data(), sizes[t].data(), (float*)total.data(), 1));
  float sum = 0.0f;
  total.to_host(&sum);  // the one synchronisation, as to_vec is in the reference
  const float norm = std::sqrt(sum);
  if (!std::isfinite(norm) || norm <= (float)max_norm) return norm;
  if (scale) *scale = max_norm / ((double)norm + 1e-6);
  return norm;
}

float clip_grad_norm(const std::vector<Tensor>& parameters, GradientStore& grads, double max_norm) {
  double scale = 1.0;
  const float norm = clip_grad_scale(parameters, grads, max_norm, &scale);
  if (scale == 1.0) return norm;
  for (const Tensor& p : parameters) {
    const Tensor* g = grads.get(p.id());
    if (!g) continue;
    // a fresh tensor, as `grad * scale` is in the reference: the stored gradient may be
    // shared with the graph that produced it
    Tensor scaled = g->zeros_like();
    const Tensor gc = g->compact();
    const int64_t n = (int64_t)gc.layout().size(), one = 1;
    check(deers_rocm_copy_compact((int)gc.dtype(), gc.data(), &n, &one, 1, scaled.data()));
    check(deers_rocm_scale((int)scaled.dtype(), scaled.data(), (int64_t)scaled.layout().size(), scale));
    grads.insert(p.id(), scaled.detach());
  }
  return norm;
}

}  // namespace deers_host
