#include "optim.h"

#include <cmath>

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
  for (const Tensor& param : parameters_) {
    const Tensor* found = grads.get(param.id());
    if (!found) continue;
    if (!param.is_compact()) throw std::logic_error("AdamW: parameters must be compact");
    if (found->shape() != param.shape() || found->dtype() != param.dtype())
      throw std::logic_error("AdamW: gradient does not match its parameter");
    const Tensor grad = found->compact();
    auto m = m_.find(param.id());
    if (m == m_.end()) m = m_.emplace(param.id(), param.zeros_like()).first;
    auto v = v_.find(param.id());
    if (v == v_.end()) v = v_.emplace(param.id(), param.zeros_like()).first;
    check(deers_rocm_adamw_step((int)param.dtype(), param.data(), grad.data(), m->second.data(),
                                v->second.data(), (int64_t)param.layout().size(), lr_, beta1_,
                                beta2_, eps_, weight_decay_, (int64_t)step_, grad_scale));
  }
}

float clip_grad_scale(const std::vector<Tensor>& parameters, const GradientStore& grads,
                      double max_norm, double* scale) {
  if (!(max_norm > 0.0)) throw std::logic_error("max_norm must be positive");
  if (scale) *scale = 1.0;
  if (parameters.empty()) return 0.0f;
  Tensor total = Tensor::zeros({1}, DType::F32);
  for (const Tensor& p : parameters) {
    const Tensor* g = grads.get(p.id());
    if (!g) continue;
    const Tensor gc = g->compact();
    check(deers_rocm_sum_squares((int)gc.dtype(), gc.data(), (int64_t)gc.layout().size(),
                                 (float*)total.data(), 1));
  }
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
