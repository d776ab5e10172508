// Optimizer side of the C++ host: AdamW and clip_grad_norm with the reference's names
// and contracts (src/optim.rs:44-296), on the fused device step of
// include/deers_rocm.h.  A parameter is an attached leaf Tensor (the role of
// nn::Parameter, src/nn/parameter.rs:15-28); the step rewrites its storage in place, so
// the tensor keeps its id and its requires_grad flag as Parameter::set does.
#ifndef DEERS_HOST_OPTIM_H
#define DEERS_HOST_OPTIM_H

#include <optional>
#include <unordered_map>
#include <utility>
#include <vector>

#include "tensor.h"

namespace deers_host {

class AdamW;

// src/optim.rs:44-96
struct AdamWConfig {
  double lr;
  std::pair<double, double> betas_{0.9, 0.999};
  double eps_ = 1e-8;
  double weight_decay_ = 0.0;

  explicit AdamWConfig(double lr_) : lr(lr_) {}
  AdamWConfig& betas(double b1, double b2) { betas_ = {b1, b2}; return *this; }
  AdamWConfig& eps(double e) { eps_ = e; return *this; }
  AdamWConfig& weight_decay(double wd) { weight_decay_ = wd; return *this; }
  AdamW build(std::vector<Tensor> parameters) const;
};

// src/optim.rs:98-251
class AdamW {
 public:
  void set_lr(double lr) { lr_ = lr; }
  double lr() const { return lr_; }
  size_t step_count() const { return step_; }
  void set_step_count(size_t step) { step_ = step; }
  // The moments tracked for `parameter`, if it has been stepped or loaded.
  std::optional<std::pair<Tensor, Tensor>> state_for(const Tensor& parameter) const;
  void load_state_for(const Tensor& parameter, Tensor m, Tensor v);

  // loss.backward() then one step.
  void backward_step(const Tensor& loss);
  // One step from a gradient store; parameters without a gradient are skipped.
  // grad_scale != 1 applies clip_grad_norm's rescaling inside the same kernel
  // (see clip_grad_scale below) instead of rewriting the gradients first.
  void step_with_grads(const GradientStore& grads, double grad_scale = 1.0);

 private:
  friend struct AdamWConfig;
  std::vector<Tensor> parameters_;
  double lr_ = 0, beta1_ = 0.9, beta2_ = 0.999, eps_ = 1e-8, weight_decay_ = 0;
  std::unordered_map<TensorId, Tensor> m_, v_;
  size_t step_ = 0;
};

// src/optim.rs:258-296: the global gradient norm over `parameters`; when it exceeds
// max_norm every gradient in the store is replaced by a rescaled copy.  Returns the norm
// before clipping.  max_norm <= 0 is a programmer error (std::logic_error).
float clip_grad_norm(const std::vector<Tensor>& parameters, GradientStore& grads, double max_norm);

// The same decision without touching the gradients: returns the norm and sets *scale to
// the factor clip_grad_norm would apply (1.0 when it would not clip), for
// AdamW::step_with_grads(grads, scale).
float clip_grad_scale(const std::vector<Tensor>& parameters, const GradientStore& grads,
                      double max_norm, double* scale);

}  // namespace deers_host
#endif
