// Operators of the C++ host side; see ops.h for the reference ops each follows.
#include "ops.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/deers_rocm.h"

namespace deers_host {

namespace {

bool backed(const Tensor& t) { return t.storage()->ptr() != nullptr; }

// Fresh compact storage shaped like `shape`.
Tensor empty(const std::vector<int64_t>& shape, DType dtype, bool is_backed) {
  Layout l(shape);
  auto st = std::make_shared<RocmStorage>(l.size(), dtype, is_backed);
  return Tensor(std::move(st), std::move(l), false, nullptr);
}

}  // namespace

// IEEE binary16 bits of a float, round to nearest even (what f16::from_f32 does).
uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to infinity
  if (x < 0x38800000u) {                                    // subnormal or zero
    if (x < 0x33000000u) return (uint16_t)sign;
    const int shift = 126 - (int)(x >> 23);                 // 14..24
    const uint32_t mant = (x & 0x7fffffu) | 0x800000u;
    const uint32_t q = mant >> shift, rem = mant & ((1u << shift) - 1), half = 1u << (shift - 1);
    return (uint16_t)(sign | (q + ((rem > half) || (rem == half && (q & 1)))));
  }
  const uint32_t q = (x - 0x38000000u) >> 13, rem = x & 0x1fffu;
  return (uint16_t)(sign | (q + ((rem > 0x1000u) || (rem == 0x1000u && (q & 1)))));
}

namespace {

// A [B,H,T,D] view the kernels take as is: unit D stride (alignment is the
// library's check).  Anything else is compacted.
Tensor kernel_ready(const Tensor& t) {
  const Layout& l = t.layout();
  const int64_t per16 = 16 / (int64_t)size_in_bytes(t.dtype());
  bool ok = l.strides.back() == 1 && l.offset % per16 == 0;
  for (size_t d = 0; d + 1 < l.ndim(); ++d) ok = ok && l.strides[d] >= 0 && l.strides[d] % per16 == 0;
  return ok ? t : t.compact();
}

}  // namespace

// ---- Neg ----
Tensor Neg::forward(std::unique_ptr<Neg> self) {
  const Tensor a = self->arg_.compact();
  Tensor out = empty(a.shape(), a.dtype(), backed(a));
  if (backed(a)) check(deers_rocm_neg((int)a.dtype(), a.data(), out.data(), a.layout().size()));
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}
void Neg::backward(GradientStore& grads, const Tensor& out_grad) const {
  grads.accumulate(arg_, out_grad.neg());
}

// ---- EWiseAdd ----
EWiseAdd::EWiseAdd(Tensor a, Tensor b) : a_(std::move(a)), b_(std::move(b)) {
  if (a_.shape() != b_.shape()) throw std::logic_error("EWiseAdd: shapes differ");
  if (a_.dtype() != b_.dtype()) throw std::logic_error("EWiseAdd: dtypes differ");
}
Tensor EWiseAdd::forward(std::unique_ptr<EWiseAdd> self) {
  const Tensor a = self->a_.compact(), b = self->b_.compact();
  Tensor out = empty(a.shape(), a.dtype(), backed(a));
  if (backed(a))
    check(deers_rocm_add((int)a.dtype(), a.data(), b.data(), out.data(), a.layout().size()));
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}
void EWiseAdd::backward(GradientStore& grads, const Tensor& out_grad) const {
  grads.accumulate(a_, out_grad);
  grads.accumulate(b_, out_grad);
}

// ---- Permute ----
Permute::Permute(Tensor arg, std::vector<size_t> axes) : arg_(std::move(arg)), axes_(std::move(axes)) {
  if (arg_.layout().ndim() != axes_.size())
    throw std::logic_error("permute: tensor has " + std::to_string(arg_.layout().ndim()) +
                           " dims but got " + std::to_string(axes_.size()) + " axes");
}
Tensor Permute::forward(std::unique_ptr<Permute> self) {
  auto storage = self->arg_.storage();
  Layout layout = self->arg_.layout().permute(self->axes_);
  return Tensor(std::move(storage), std::move(layout), false, std::move(self));
}
void Permute::backward(GradientStore& grads, const Tensor& out_grad) const {
  std::vector<size_t> inverse(axes_.size());
  for (size_t new_axis = 0; new_axis < axes_.size(); ++new_axis) inverse[axes_[new_axis]] = new_axis;
  grads.accumulate(arg_, out_grad.permute(inverse));
}

// ---- Compact ----
Tensor Compact::forward(std::unique_ptr<Compact> self) {
  const Tensor& a = self->arg_;
  Tensor out = empty(a.shape(), a.dtype(), backed(a));
  if (backed(a) && a.layout().size())
    check(deers_rocm_copy_compact((int)a.dtype(), a.data(), a.layout().shape.data(),
                                  a.layout().strides.data(), (int)a.layout().ndim(), out.data()));
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}
void Compact::backward(GradientStore& grads, const Tensor& out_grad) const {
  grads.accumulate(arg_, out_grad);
}

// ---- Reshape ----
Reshape::Reshape(Tensor arg, std::vector<int64_t> new_shape)
    : arg_(arg.compact()), new_shape_(std::move(new_shape)) {
  if (arg_.layout().size() != Layout(new_shape_).size())
    throw std::logic_error("reshape: size " + std::to_string(arg_.layout().size()) +
                           " cannot be reshaped to size " + std::to_string(Layout(new_shape_).size()));
}
Tensor Reshape::forward(std::unique_ptr<Reshape> self) {
  auto storage = self->arg_.storage();
  Layout layout(self->new_shape_);
  return Tensor(std::move(storage), std::move(layout), false, std::move(self));
}
void Reshape::backward(GradientStore& grads, const Tensor& out_grad) const {
  grads.accumulate(arg_, out_grad.reshape(arg_.shape()));
}

// ---- MatMul ----
MatMul::MatMul(Tensor a, Tensor b) : a_(std::move(a)), b_(std::move(b)) {
  const size_t nd = a_.layout().ndim();
  if (nd < 2 || b_.layout().ndim() < 2)
    throw std::logic_error("matmul requires ndim >= 2");
  if (nd != b_.layout().ndim()) throw std::logic_error("matmul requires same number of dimensions");
  if (a_.shape()[nd - 1] != b_.shape()[nd - 2]) throw std::logic_error("matmul inner dimensions must match");
  for (size_t i = 0; i + 2 < nd; ++i)
    if (a_.shape()[i] != b_.shape()[i]) throw std::logic_error("matmul batch dimension mismatch");
  if (a_.dtype() != b_.dtype()) throw std::logic_error("matmul: dtypes differ");
}

namespace {
// Describes the last two axes and the (collapsed) batch axes of `t` for the library:
// returns false when the batch axes cannot be expressed by one stride or no matrix
// stride is 1, in which case the caller compacts.
bool gemm_view(const Tensor& t, int64_t* rs, int64_t* cs, int64_t* bs) {
  const Layout& l = t.layout();
  const size_t nd = l.ndim();
  *rs = l.strides[nd - 2];
  *cs = l.strides[nd - 1];
  const int64_t rows = l.shape[nd - 2], cols = l.shape[nd - 1];
  if (!((*cs == 1 && *rs >= cols) || (*rs == 1 && *cs >= rows) || rows == 1 || cols == 1)) return false;
  // batch axes must walk memory like one axis: stride[i] == stride[i+1] * shape[i+1]
  *bs = 0;
  int64_t expect = -1;
  for (int i = (int)nd - 3; i >= 0; --i) {
    if (l.shape[i] == 1) continue;
    if (expect >= 0 && l.strides[i] != expect) return false;
    if (expect < 0) *bs = l.strides[i];
    expect = l.strides[i] * l.shape[i];
  }
  return *bs >= 0;
}
}  // namespace

namespace {
// a @ b, plus `addend` (compact, the product's shape and type) where one is given, into
// fresh storage
Tensor run_product(Tensor a, Tensor b, const Tensor* addend) {
  int64_t ars, acs, abs_, brs, bcs, bbs;
  if (!gemm_view(a, &ars, &acs, &abs_)) { a = a.detach().compact(); gemm_view(a, &ars, &acs, &abs_); }
  if (!gemm_view(b, &brs, &bcs, &bbs)) { b = b.detach().compact(); gemm_view(b, &brs, &bcs, &bbs); }
  const size_t nd = a.layout().ndim();
  const int64_t m = a.shape()[nd - 2], k = a.shape()[nd - 1], n = b.shape()[nd - 1];
  std::vector<int64_t> out_shape(a.shape().begin(), a.shape().end() - 2);
  int64_t batch = 1;
  for (int64_t d : out_shape) batch *= d;
  out_shape.push_back(m);
  out_shape.push_back(n);
  Tensor out = empty(out_shape, a.dtype(), backed(a));
  if (addend && (!addend->is_compact() || addend->shape() != out_shape || addend->dtype() != a.dtype()))
    throw std::logic_error("matmul_add: the addend must be a compact tensor of the product's shape and type");
  if (backed(a) && addend)
    check(deers_rocm_matmul_add((int)a.dtype(), a.data(), ars, acs, abs_, b.data(), brs, bcs, bbs,
                                addend->data(), out.data(), batch, m, n, k));
  else if (backed(a))
    check(deers_rocm_matmul((int)a.dtype(), a.data(), ars, acs, abs_, b.data(), brs, bcs, bbs,
                            out.data(), batch, m, n, k));
  return out;
}

// GradientStore::accumulate of the product a @ b (src/backprop.rs:101-112 after
// src/ops.rs:1089-1101): where `target` already holds a gradient the sum rides on the
// product, into fresh storage, since another entry may share the held tensor.
void accumulate_product(GradientStore& grads, const Tensor& target, const Tensor& a, const Tensor& b) {
  const Tensor* held = grads.get(target.id());
  if (held && held->is_compact() && held->dtype() == a.dtype() && held->shape().size() == a.shape().size() &&
      std::equal(held->shape().begin(), held->shape().end() - 2, a.shape().begin()) &&
      held->shape()[held->shape().size() - 2] == a.shape()[a.shape().size() - 2] &&
      held->shape().back() == b.shape().back()) {
    const Tensor addend = *held;
    grads.insert(target.id(), matmul_add(a, b, addend));
  } else {
    grads.accumulate(target, a.matmul(b));
  }
}
}  // namespace

Tensor MatMul::forward(std::unique_ptr<MatMul> self) {
  const Tensor out = run_product(self->a_, self->b_, nullptr);
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}

void MatMul::backward(GradientStore& grads, const Tensor& out_grad) const {
  accumulate_product(grads, a_, out_grad, b_.transpose());
  accumulate_product(grads, b_, a_.transpose(), out_grad);
}

// ---- MatMulAdd ----
MatMulAdd::MatMulAdd(Tensor a, Tensor b, Tensor c) : a_(std::move(a)), b_(std::move(b)), c_(c.compact()) {
  const size_t nd = a_.layout().ndim();
  if (nd < 2 || nd != b_.layout().ndim() || a_.shape()[nd - 1] != b_.shape()[nd - 2])
    throw std::logic_error("matmul_add: a [..,M,K] and b [..,K,N] of equal rank");
  for (size_t i = 0; i + 2 < nd; ++i)
    if (a_.shape()[i] != b_.shape()[i]) throw std::logic_error("matmul_add: batch dimension mismatch");
  if (a_.dtype() != b_.dtype() || a_.dtype() != c_.dtype()) throw std::logic_error("matmul_add: dtypes differ");
}
Tensor MatMulAdd::forward(std::unique_ptr<MatMulAdd> self) {
  const Tensor out = run_product(self->a_, self->b_, &self->c_);
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}
void MatMulAdd::backward(GradientStore& grads, const Tensor& out_grad) const {
  grads.accumulate(c_, out_grad);
  accumulate_product(grads, a_, out_grad, b_.transpose());
  accumulate_product(grads, b_, a_.transpose(), out_grad);
}
Tensor matmul_add(const Tensor& a, const Tensor& b, const Tensor& c) {
  return MatMulAdd::forward(std::make_unique<MatMulAdd>(a, b, c));
}

// ---- Tensor conveniences that build ops ----
Tensor Tensor::transpose() const {
  const size_t nd = layout().ndim();
  std::vector<size_t> dims(nd);
  for (size_t i = 0; i < nd; ++i) dims[i] = i;
  std::swap(dims[nd - 1], dims[nd - 2]);
  return permute(dims);
}
Tensor Tensor::reshape(const std::vector<int64_t>& shape) const {
  return Reshape::forward(std::make_unique<Reshape>(*this, shape));
}
Tensor Tensor::matmul(const Tensor& other) const {
  return MatMul::forward(std::make_unique<MatMul>(*this, other));
}
Tensor Tensor::permute(const std::vector<size_t>& dims) const {
  return Permute::forward(std::make_unique<Permute>(*this, dims));
}
Tensor Tensor::compact() const {
  if (is_compact()) return *this;
  return Compact::forward(std::make_unique<Compact>(*this));
}
Tensor Tensor::neg() const { return Neg::forward(std::make_unique<Neg>(*this)); }
Tensor Tensor::add(const Tensor& other) const {
  return EWiseAdd::forward(std::make_unique<EWiseAdd>(*this, other));
}

// ---- FusedLogSoftmax ----
FusedLogSoftmax::FusedLogSoftmax(Tensor arg, size_t axis) : arg_(std::move(arg)), axis_(axis) {
  if (arg_.layout().ndim() == 0 || axis_ != arg_.layout().ndim() - 1)
    throw std::logic_error("FusedLogSoftmax: the axis must be the last one");
}
Tensor FusedLogSoftmax::forward(std::unique_ptr<FusedLogSoftmax> self) {
  const Tensor x = self->arg_.compact();
  const int64_t inner = x.shape()[self->axis_];
  const int64_t outer = inner ? (int64_t)x.layout().size() / inner : 0;
  Tensor out = empty(x.shape(), x.dtype(), backed(x));
  if (backed(x)) check(deers_rocm_log_softmax_fwd((int)x.dtype(), x.data(), out.data(), outer, inner));
  self->lsm_output_ = out;
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}
void FusedLogSoftmax::backward(GradientStore& grads, const Tensor& out_grad) const {
  if (!lsm_output_.defined()) throw std::logic_error("forward must run before backward");
  const Tensor g = out_grad.compact();
  const int64_t inner = g.shape()[axis_];
  const int64_t outer = inner ? (int64_t)g.layout().size() / inner : 0;
  Tensor dx = empty(g.shape(), g.dtype(), backed(g));
  if (backed(g))
    check(deers_rocm_log_softmax_bwd((int)g.dtype(), g.data(), lsm_output_.data(), dx.data(), outer,
                                     inner));
  grads.accumulate(arg_, dx);
}
Tensor Tensor::log_softmax(size_t axis) const {
  return FusedLogSoftmax::forward(std::make_unique<FusedLogSoftmax>(*this, axis));
}

// ---- IndexSelect ----
IndexSelect::IndexSelect(Tensor arg, size_t dim, Tensor indices)
    : arg_(std::move(arg)), indices_(std::move(indices)) {
  if (dim >= arg_.layout().ndim())
    throw std::logic_error("index_select: dim " + std::to_string(dim) + " out of bounds for " +
                           std::to_string(arg_.layout().ndim()) + " dims");
  if (dim != 0 || arg_.layout().ndim() != 2)
    throw std::logic_error("index_select: only dim 0 of a 2-D tensor is built on this device");
  if (indices_.layout().ndim() != 1) throw std::logic_error("index_select requires 1D indices");
  if (indices_.dtype() != DType::I64) throw std::logic_error("index_select indices must be i64");
  arg_ = arg_.compact();  // src/ops.rs:1405
  indices_ = indices_.compact();
}
Tensor IndexSelect::forward(std::unique_ptr<IndexSelect> self) {
  const Tensor& w = self->arg_;
  const int64_t n = self->indices_.shape()[0], rows = w.shape()[0], width = w.shape()[1];
  Tensor out = empty({n, width}, w.dtype(), backed(w));
  if (backed(w))
    check(deers_rocm_index_select((int)w.dtype(), w.data(), (const int64_t*)self->indices_.data(),
                                  out.data(), rows, n, width));
  return Tensor(out.storage(), out.layout(), false, std::move(self));
}
void IndexSelect::backward(GradientStore& grads, const Tensor& out_grad) const {
  const Tensor g = out_grad.compact();
  Tensor dw = arg_.zeros_like();
  if (backed(g))
    check(deers_rocm_index_add((int)g.dtype(), g.data(), (const int64_t*)indices_.data(), dw.data(),
                               arg_.shape()[0], indices_.shape()[0], arg_.shape()[1]));
  grads.accumulate(arg_, dw);
}
Tensor Tensor::index_select(size_t dim, const Tensor& indices) const {
  return IndexSelect::forward(std::make_unique<IndexSelect>(*this, dim, indices));
}

// ---- RmsNorm ----
static void rows_of(const Tensor& t, int64_t* outer, int64_t* inner) {
  if (t.layout().ndim() == 0) throw std::logic_error("a row-wise op needs at least one axis");
  *inner = t.shape().back();
  *outer = *inner ? (int64_t)t.layout().size() / *inner : 0;
}
Tensor RmsNorm::forward(std::unique_ptr<RmsNorm> self) {
  self->arg_ = self->arg_.compact();
  const Tensor& x = self->arg_;
  int64_t outer, inner;
  rows_of(x, &outer, &inner);
  Tensor y = empty(x.shape(), x.dtype(), backed(x));
  if (backed(x)) check(deers_rocm_rms_norm_fwd((int)x.dtype(), x.data(), y.data(), outer, inner, self->eps_));
  return Tensor(y.storage(), y.layout(), false, std::move(self));
}
void RmsNorm::backward(GradientStore& grads, const Tensor& out_grad) const {
  const Tensor g = out_grad.compact();
  int64_t outer, inner;
  rows_of(arg_, &outer, &inner);
  Tensor dx = empty(arg_.shape(), arg_.dtype(), backed(arg_));
  // a gradient the input already holds (the residual branch's) is added in the same pass
  const Tensor* held = grads.get(arg_.id());
  if (held && held->is_compact() && held->shape() == arg_.shape() && held->dtype() == arg_.dtype()) {
    if (backed(arg_))
      check(deers_rocm_rms_norm_bwd_add((int)arg_.dtype(), arg_.data(), g.data(), held->data(), dx.data(), outer,
                                        inner, eps_));
    grads.insert(arg_.id(), dx);
    return;
  }
  if (backed(arg_))
    check(deers_rocm_rms_norm_bwd((int)arg_.dtype(), arg_.data(), g.data(), dx.data(), outer, inner, eps_));
  grads.accumulate(arg_, dx);
}
Tensor rms_norm(const Tensor& x, double eps) {
  return RmsNorm::forward(std::make_unique<RmsNorm>(x, eps));
}

// ---- ReluSq ----
Tensor ReluSq::forward(std::unique_ptr<ReluSq> self) {
  self->arg_ = self->arg_.compact();
  const Tensor& x = self->arg_;
  Tensor y = empty(x.shape(), x.dtype(), backed(x));
  if (backed(x)) check(deers_rocm_relu_sq_fwd((int)x.dtype(), x.data(), y.data(), (int64_t)x.layout().size()));
  return Tensor(y.storage(), y.layout(), false, std::move(self));
}
void ReluSq::backward(GradientStore& grads, const Tensor& out_grad) const {
  const Tensor g = out_grad.compact();
  Tensor dx = empty(arg_.shape(), arg_.dtype(), backed(arg_));
  if (backed(arg_))
    check(deers_rocm_relu_sq_bwd((int)arg_.dtype(), arg_.data(), g.data(), dx.data(),
                                 (int64_t)arg_.layout().size()));
  grads.accumulate(arg_, dx);
}
Tensor relu_sq(const Tensor& x) { return ReluSq::forward(std::make_unique<ReluSq>(x)); }

// ---- CrossEntropy ----
CrossEntropy::CrossEntropy(Tensor logits, Tensor targets)
    : logits_(std::move(logits)), targets_(std::move(targets)) {
  if (logits_.layout().ndim() != 2) throw std::logic_error("cross_entropy: logits must be [N, classes]");
  if (targets_.layout().ndim() != 1 || targets_.shape()[0] != logits_.shape()[0])
    throw std::logic_error("cross_entropy: targets must be [N]");
  if (targets_.dtype() != DType::I64) throw std::logic_error("cross_entropy: targets must be i64");
  if (logits_.shape()[0] < 1) throw std::logic_error("cross_entropy: empty batch");
  logits_ = logits_.compact();
  targets_ = targets_.compact();
}
Tensor CrossEntropy::forward(std::unique_ptr<CrossEntropy> self) {
  const Tensor& x = self->logits_;
  const int64_t n = x.shape()[0], v = x.shape()[1];
  Tensor loss = empty({1}, DType::F32, backed(x));
  self->row_lse_ = empty({n}, DType::F32, backed(x));
  if (backed(x) && x.requires_grad()) {
    // A loss that will be differentiated: the forward also writes the gradient for an upstream
    // gradient of one (what Tensor::backward seeds, src/backprop.rs:52-66) while each row is
    // still in the caches; the backward then only applies the upstream factor.
    self->grad_for_one_ = empty(x.shape(), x.dtype(), true);
    check(deers_rocm_cross_entropy_fwd_grad((int)x.dtype(), x.data(), (const int64_t*)self->targets_.data(),
                                            (float*)self->row_lse_.data(), (float*)loss.data(),
                                            self->grad_for_one_.data(), n, v));
  } else if (backed(x)) {
    check(deers_rocm_cross_entropy_fwd((int)x.dtype(), x.data(), (const int64_t*)self->targets_.data(),
                                       (float*)self->row_lse_.data(), (float*)loss.data(), n, v));
  }
  return Tensor(loss.storage(), loss.layout(), false, std::move(self));
}
void CrossEntropy::backward(GradientStore& grads, const Tensor& out_grad) const {
  if (!row_lse_.defined()) throw std::logic_error("forward must run before backward");
  if (out_grad.dtype() != DType::F32 || out_grad.layout().size() != 1)
    throw std::logic_error("cross_entropy: the upstream gradient is one f32 value");
  const Tensor up = out_grad.compact();
  const Tensor& x = logits_;
  if (grad_for_one_.defined()) {
    // the first backward takes the gradient the forward wrote; a second one (the graph kept and
    // differentiated again) recomputes, since the first may have scaled the buffer
    Tensor dx = std::move(grad_for_one_);
    grad_for_one_ = Tensor();
    check(deers_rocm_scale_by_scalar((int)x.dtype(), const_cast<void*>(dx.data()), (int64_t)dx.layout().size(),
                                     (const float*)up.data()));
    grads.accumulate(logits_, dx);
    return;
  }
  Tensor dx = empty(x.shape(), x.dtype(), backed(x));
  if (backed(x))
    check(deers_rocm_cross_entropy_bwd((int)x.dtype(), x.data(), (const int64_t*)targets_.data(),
                                       (const float*)row_lse_.data(), (const float*)up.data(), dx.data(),
                                       x.shape()[0], x.shape()[1]));
  grads.accumulate(logits_, dx);
}
Tensor cross_entropy(const Tensor& logits, const Tensor& targets) {
  return CrossEntropy::forward(std::make_unique<CrossEntropy>(logits, targets));
}

// ---- FusedCausalAttention ----
FusedCausalAttention::FusedCausalAttention(Tensor q, Tensor k, Tensor v, double scale)
    : q_(std::move(q)), k_(std::move(k)), v_(std::move(v)), scale_(scale) {
  if (q_.layout().ndim() != 4) throw std::logic_error("FusedCausalAttention: q must be [B,H,T,D]");
  if (q_.shape() != k_.shape() || q_.shape() != v_.shape())
    throw std::logic_error("FusedCausalAttention: q, k, v shapes differ");
  if (q_.dtype() != k_.dtype() || q_.dtype() != v_.dtype())
    throw std::logic_error("FusedCausalAttention: dtypes differ");
}

namespace {
// Logical [B,H,T,D] over fresh [B,T,H,D] memory.
Tensor heads_interleaved(int64_t B, int64_t H, int64_t T, int64_t D, DType dtype) {
  const Tensor bthd = empty({B, T, H, D}, dtype, true);
  return Tensor(bthd.storage(), bthd.layout().permute({0, 2, 1, 3}), false, nullptr);
}
}  // namespace

Tensor FusedCausalAttention::forward(std::unique_ptr<FusedCausalAttention> self) {
  if (!fused_kernels_take(self->q_.shape()[3])) return forward_composed(std::move(self));
  const Tensor q = kernel_ready(self->q_), k = kernel_ready(self->k_), v = kernel_ready(self->v_);
  const auto& s = q.shape();
  const int64_t B = s[0], H = s[1], T = s[2], D = s[3];
  // The heads are written interleaved, [B,T,H,D] in memory under the logical [B,H,T,D]: the
  // module's `y.permute([0,2,1,3]).reshape([B*T, C])` (src/models/gpt.rs:145) is then a view
  // of compact memory and costs no copy.
  const Tensor o = heads_interleaved(B, H, T, D, q.dtype());
  Tensor lse = empty({B, H, T}, DType::F32, true);
  check(deers_rocm_attn_fwd((int)q.dtype(), q.data(), q.layout().strides.data(), k.data(),
                            k.layout().strides.data(), v.data(), v.layout().strides.data(), o.data(),
                            o.layout().strides.data(), (float*)lse.data(), B, H, T, D, (float)self->scale_));
  self->saved_o_ = o;
  self->saved_lse_ = lse;
  return Tensor(o.storage(), o.layout(), false, std::move(self));
}

namespace {

// Additive causal mask [T,T] in the tensor's dtype: -inf where the key lies after the
// query, else 0 (causal_mask with seqlen_offset 0, src/nn/functional.rs:12-55; the
// reference builds [B,1,T,T] on the host per call, here one [T,T] block is broadcast over
// batch and heads by stride 0).
Tensor causal_mask_tt(int64_t T, DType dtype) {
  if (dtype == DType::F32) {
    std::vector<float> m((size_t)(T * T), 0.f);
    for (int64_t i = 0; i < T; ++i)
      for (int64_t j = i + 1; j < T; ++j) m[(size_t)(i * T + j)] = -INFINITY;
    return Tensor::from_host(m.data(), {T, T}, dtype);
  }
  std::vector<uint16_t> m((size_t)(T * T), 0);
  for (int64_t i = 0; i < T; ++i)
    for (int64_t j = i + 1; j < T; ++j) m[(size_t)(i * T + j)] = 0xFC00;  // -inf
  return Tensor::from_host(m.data(), {T, T}, dtype);
}

// c[batch,m,n] = a @ b with explicit (row, col, batch) element strides per operand
void gemm(DType dt, const Tensor& a, int64_t ars, int64_t acs, int64_t abs_, const Tensor& b,
          int64_t brs, int64_t bcs, int64_t bbs, Tensor& c, int64_t batch, int64_t m, int64_t n,
          int64_t k) {
  check(deers_rocm_matmul((int)dt, a.data(), ars, acs, abs_, b.data(), brs, bcs, bbs, c.data(), batch,
                          m, n, k));
}

}  // namespace

Tensor FusedCausalAttention::forward_composed(std::unique_ptr<FusedCausalAttention> self) {
  const Tensor q = self->q_.compact(), k = self->k_.compact(), v = self->v_.compact();
  const auto& s = q.shape();
  const int64_t B = s[0], H = s[1], T = s[2], D = s[3], BH = B * H;
  const DType dt = q.dtype();
  if (BH * T * T >= ((int64_t)1 << 31))
    throw std::logic_error("attention: head width " + std::to_string(D) +
                           " takes the unfused path, whose [B,H,T,T] tensors would be too large here");
  const std::vector<int64_t> sc_shape{B, H, T, T};
  Tensor scores = empty(sc_shape, dt, true), scaled = empty(sc_shape, dt, true);
  // q @ k^T: k read as [D,T] through its strides (MatMul on a transposed view)
  gemm(dt, q, D, 1, T * D, k, 1, D, T * D, scores, BH, T, T, D);
  check(deers_rocm_unary((int)dt, DEERS_ROCM_UNARY_SCALAR_MUL, scores.data(), 4, sc_shape.data(), nullptr,
                         self->scale_, scaled.data()));
  const Tensor mask = causal_mask_tt(T, dt);
  const int64_t mask_strides[4] = {0, 0, T, 1};
  check(deers_rocm_binary((int)dt, DEERS_ROCM_BINARY_ADD, scaled.data(), nullptr, mask.data(), mask_strides,
                          4, sc_shape.data(), scores.data()));
  // softmax = exp(log_softmax) (src/tensor.rs:456-458), log_softmax as the fused row kernel
  Tensor lsm = empty(sc_shape, dt, true), p = empty(sc_shape, dt, true);
  check(deers_rocm_log_softmax_fwd((int)dt, scores.data(), lsm.data(), BH * T, T));
  check(deers_rocm_unary((int)dt, DEERS_ROCM_UNARY_EXP, lsm.data(), 4, sc_shape.data(), nullptr, 0.0,
                         p.data()));
  Tensor o = empty(s, dt, true);
  gemm(dt, p, T, 1, T * T, v, D, 1, T * D, o, BH, T, D, T);
  self->saved_p_ = p;
  self->saved_lsm_ = lsm;
  return Tensor(o.storage(), o.layout(), false, std::move(self));
}

void FusedCausalAttention::backward_composed(GradientStore& grads, const Tensor& out_grad) const {
  const Tensor q = q_.compact(), k = k_.compact(), v = v_.compact(), g = out_grad.compact();
  const auto& s = q.shape();
  const int64_t B = s[0], H = s[1], T = s[2], D = s[3], BH = B * H;
  const DType dt = q.dtype();
  const std::vector<int64_t> sc_shape{B, H, T, T};
  // MatMul::backward of attn @ v: dAttn = dY @ v^T, dV = attn^T @ dY (src/ops.rs:1089-1101)
  Tensor dv = empty(s, dt, true), dp = empty(sc_shape, dt, true);
  gemm(dt, saved_p_, 1, T, T * T, g, D, 1, T * D, dv, BH, T, D, T);
  gemm(dt, g, D, 1, T * D, v, 1, D, T * D, dp, BH, T, T, D);
  // EWiseExp::backward: dLsm = dAttn * exp(lsm) (src/ops.rs:422-425)
  Tensor dlsm = empty(sc_shape, dt, true), dx = empty(sc_shape, dt, true);
  check(deers_rocm_binary((int)dt, DEERS_ROCM_BINARY_MUL, dp.data(), nullptr, saved_p_.data(), nullptr, 4,
                          sc_shape.data(), dlsm.data()));
  // FusedLogSoftmax::backward: dX = dLsm - exp(lsm) * rowsum(dLsm) (src/ops.rs:1223-1246)
  check(deers_rocm_log_softmax_bwd((int)dt, dlsm.data(), saved_lsm_.data(), dx.data(), BH * T, T));
  // the mask has no gradient; ScalarMul::backward: dS = dX * scale (src/ops.rs:638-643)
  check(deers_rocm_unary((int)dt, DEERS_ROCM_UNARY_SCALAR_MUL, dx.data(), 4, sc_shape.data(), nullptr, scale_,
                         dlsm.data()));
  // MatMul::backward of q @ k^T: dQ = dS @ k, d(k^T) = q^T @ dS, i.e. dK = dS^T @ q
  Tensor dq = empty(s, dt, true), dk = empty(s, dt, true);
  gemm(dt, dlsm, T, 1, T * T, k, D, 1, T * D, dq, BH, T, D, T);
  gemm(dt, dlsm, 1, T, T * T, q, D, 1, T * D, dk, BH, T, D, T);
  grads.accumulate(q_, dq);
  grads.accumulate(k_, dk);
  grads.accumulate(v_, dv);
}

void FusedCausalAttention::backward(GradientStore& grads, const Tensor& out_grad) const {
  if (saved_p_.defined()) return backward_composed(grads, out_grad);
  if (!saved_o_.defined()) throw std::logic_error("forward must run before backward");
  // out_grad usually arrives as the inverse-permuted view of the reshape gradient:
  // logical [B,H,T,D] over [B,T,H,D] memory, which the kernels read directly.
  const Tensor q = kernel_ready(q_), k = kernel_ready(k_), v = kernel_ready(v_);
  const Tensor g = kernel_ready(out_grad);
  const auto& s = q.shape();
  const int64_t B = s[0], H = s[1], T = s[2], D = s[3];
  Tensor dq = empty(s, q.dtype(), true), dk = empty(s, q.dtype(), true);
  // v usually is the permuted view of a [B,T,H,D] projection: its gradient is written in the
  // same memory order, so that the permute's and the reshape's backward are views too
  const bool v_interleaved = v.layout().strides[1] == D && v.layout().strides[2] == H * D;
  const Tensor dv = v_interleaved ? heads_interleaved(B, H, T, D, q.dtype()) : empty(s, q.dtype(), true);
  check(deers_rocm_attn_bwd((int)q.dtype(), q.data(), q.layout().strides.data(), k.data(),
                            k.layout().strides.data(), v.data(), v.layout().strides.data(),
                            saved_o_.data(), saved_o_.layout().strides.data(), (const float*)saved_lse_.data(),
                            g.data(), g.layout().strides.data(), dq.data(), nullptr, dk.data(), nullptr,
                            const_cast<void*>(dv.data()), dv.layout().strides.data(), B, H, T, D, (float)scale_));
  grads.accumulate(q_, dq);
  grads.accumulate(k_, dk);
  grads.accumulate(v_, dv);
}

// ---- RotaryHeads ----
RotaryHeads::RotaryHeads(Tensor x, Tensor cos, Tensor sin)
    : x_(std::move(x)), cos_(std::move(cos)), sin_(std::move(sin)) {
  if (x_.layout().ndim() != 4) throw std::logic_error("RoPE expects a 4D attention tensor");
  if (cos_.shape() != sin_.shape()) throw std::logic_error("RoPE cos/sin shapes must match");
  const int64_t D = x_.shape()[3];
  if (D % 2) throw std::logic_error("RoPE requires an even head dimension");
  if (cos_.layout().ndim() != 4 || cos_.shape()[3] != D / 2)
    throw std::logic_error("RoPE cache last dimension must equal head_dim / 2");
  if (cos_.shape()[1] != x_.shape()[1]) throw std::logic_error("RoPE cache must match sequence length");
  if (cos_.dtype() != x_.dtype() || sin_.dtype() != x_.dtype())
    throw std::logic_error("RoPE cache dtype must match the tensor");
}

Tensor RotaryHeads::forward(std::unique_ptr<RotaryHeads> self) {
  const Tensor x = kernel_ready(self->x_);
  const Tensor cos = self->cos_.compact(), sin = self->sin_.compact();
  const int64_t B = x.shape()[0], T = x.shape()[1], H = x.shape()[2], D = x.shape()[3];
  Tensor y = empty({B, H, T, D}, x.dtype(), true);
  check(deers_rocm_rope_fwd((int)x.dtype(), x.data(), x.layout().strides.data(), cos.data(),
                            sin.data(), y.data(), nullptr, B, T, H, D));
  return Tensor(y.storage(), y.layout(), false, std::move(self));
}

void RotaryHeads::backward(GradientStore& grads, const Tensor& out_grad) const {
  const Tensor g = kernel_ready(out_grad);  // logical [B,H,T,D]
  const Tensor cos = cos_.compact(), sin = sin_.compact();
  const int64_t B = g.shape()[0], H = g.shape()[1], T = g.shape()[2], D = g.shape()[3];
  Tensor dx = empty({B, T, H, D}, g.dtype(), true);
  check(deers_rocm_rope_bwd((int)g.dtype(), g.data(), g.layout().strides.data(), cos.data(),
                            sin.data(), dx.data(), B, T, H, D));
  grads.accumulate(x_, dx);
}

std::pair<Tensor, Tensor> precompute_rotary_embeddings(int64_t seq_len, int64_t head_dim,
                                                       float base, DType dtype) {
  if (head_dim % 2) throw std::logic_error("RoPE requires an even head dimension");
  const int64_t half = head_dim / 2;
  std::vector<float> inv_freq(half);
  for (int64_t i = 0; i < half; ++i)
    inv_freq[i] = 1.0f / std::pow(base, (float)(2 * i) / (float)head_dim);
  std::vector<float> c(seq_len * half), s(seq_len * half);
  for (int64_t t = 0; t < seq_len; ++t)
    for (int64_t i = 0; i < half; ++i) {
      const float a = (float)t * inv_freq[i];
      c[t * half + i] = std::cos(a);
      s[t * half + i] = std::sin(a);
    }
  const std::vector<int64_t> shape{1, seq_len, 1, half};
  if (dtype == DType::F32)
    return {Tensor::from_host(c.data(), shape, dtype), Tensor::from_host(s.data(), shape, dtype)};
  std::vector<uint16_t> ch(c.size()), sh(s.size());
  for (size_t i = 0; i < c.size(); ++i) {
    ch[i] = f32_to_f16_bits(c[i]);
    sh[i] = f32_to_f16_bits(s[i]);
  }
  return {Tensor::from_host(ch.data(), shape, dtype), Tensor::from_host(sh.data(), shape, dtype)};
}

Tensor rotary_heads(const Tensor& x, const Tensor& cos, const Tensor& sin) {
  return RotaryHeads::forward(std::make_unique<RotaryHeads>(x, cos, sin));
}

Tensor causal_self_attention(const Tensor& q, const Tensor& k, const Tensor& v) {
  const double scale = 1.0 / std::sqrt((double)q.shape().at(3));
  return FusedCausalAttention::forward(std::make_unique<FusedCausalAttention>(q, k, v, scale));
}

// ---- CausalSelfAttention module ----
CausalSelfAttention::CausalSelfAttention(int64_t n_embd, int64_t n_head, Tensor wq, Tensor wk,
                                         Tensor wv, Tensor wo)
    : n_head_(n_head), head_dim_(n_embd / n_head), wq_(std::move(wq)), wk_(std::move(wk)),
      wv_(std::move(wv)), wo_(std::move(wo)) {
  if (n_embd % n_head) throw std::logic_error("n_embd must be divisible by n_head");
  for (const Tensor* w : {&wq_, &wk_, &wv_, &wo_})
    if (w->shape() != std::vector<int64_t>{n_embd, n_embd})
      throw std::logic_error("projection weights must be [n_embd, n_embd]");
}

Tensor CausalSelfAttention::forward(const Tensor& x, const Tensor& cos, const Tensor& sin,
                                    const Tensor* residual) const {
  if (x.layout().ndim() != 3) throw std::logic_error("attention expects input shape [B, T, C]");
  const int64_t B = x.shape()[0], T = x.shape()[1], C = x.shape()[2];
  if (C != n_head_ * head_dim_) throw std::logic_error("input channel size must match attention width");
  const Tensor x_flat = x.reshape({B * T, C});
  const std::vector<int64_t> bthd{B, T, n_head_, head_dim_};
  const Tensor q = x_flat.matmul(wq_).reshape(bthd);  // [B,T,H,D]
  const Tensor k = x_flat.matmul(wk_).reshape(bthd);
  const Tensor v = x_flat.matmul(wv_).reshape(bthd);
  const Tensor qh = rotary_heads(q, cos, sin);         // [B,H,T,D], compact
  const Tensor kh = rotary_heads(k, cos, sin);
  const Tensor vh = v.permute({0, 2, 1, 3});           // a view; the kernels read it by stride
  const Tensor y = causal_self_attention(qh, kh, vh).permute({0, 2, 1, 3}).reshape({B * T, C});
  // the block's `x + attn(..)` (src/models/gpt.rs:237-239) rides on the output projection
  if (residual) return matmul_add(y, wo_, residual->reshape({B * T, C})).reshape({B, T, C});
  return y.matmul(wo_).reshape({B, T, C});
}

KvCache KvCache::create(int64_t B, int64_t H, int64_t capacity, int64_t D, DType dtype) {
  // said here, once, rather than by the first decode_step deep inside a generation loop
  if (dtype != DType::F16)
    throw std::logic_error("KvCache: the decode kernels read f16 caches only; an f32 model "
                           "generates through GPT::forward on the whole window, as the reference "
                           "does (examples/tinystories_train.rs:250-276)");
  if (D != 32 && D != 64 && D != 128)
    throw std::logic_error("KvCache: the decode kernels take head widths 32, 64 and 128 (got " +
                           std::to_string(D) + ")");
  KvCache c;
  c.k = Tensor::zeros({B, H, capacity, D}, dtype);
  c.v = Tensor::zeros({B, H, capacity, D}, dtype);
  c.capacity = capacity;
  return c;
}

const Tensor& CausalSelfAttention::packed_qkv(KvCache& cache) const {
  if (!cache.wqkv.defined()) {
    const int64_t C = n_head_ * head_dim_;
    const size_t el = size_in_bytes(wq_.dtype());
    cache.wqkv = empty({C, 3 * C}, wq_.dtype(), true);
    const Tensor* w[3] = {&wq_, &wk_, &wv_};
    for (int i = 0; i < 3; ++i) {
      const Tensor wc = w[i]->compact();
      const int64_t wshape[2] = {C, C}, src[2] = {C, 1}, dst[2] = {3 * C, 1};
      check(deers_rocm_copy_view((int)wq_.dtype(), wc.data(), src, (char*)cache.wqkv.data() + i * C * el, dst,
                                 wshape, 2));
    }
  }
  return cache.wqkv;
}

Tensor CausalSelfAttention::prefill(const Tensor& x, KvCache& cache, const Tensor& cos,
                                    const Tensor& sin, const Tensor* residual) const {
  NoGradGuard no_grad;
  if (x.layout().ndim() != 3) throw std::logic_error("prefill expects input shape [B, T, C]");
  if (cache.len != 0) throw std::logic_error("prefill: the KV cache must be empty");
  const int64_t B = x.shape()[0], T = x.shape()[1], C = x.shape()[2], H = n_head_, D = head_dim_;
  const int64_t cap = cache.capacity;
  if (C != H * D) throw std::logic_error("input channel size must match attention width");
  if (T < 1 || T > cap) throw std::logic_error("prefill: the prompt does not fit the KV cache");
  if (T > cos.shape()[1]) throw std::logic_error("prefill: prompt longer than the RoPE tables");
  const int dt = (int)x.dtype();
  const size_t el = size_in_bytes(x.dtype());
  const Tensor qkv = x.reshape({B * T, C}).matmul(packed_qkv(cache));  // [B*T, 3C]
  const char* q_data = (const char*)qkv.data();
  const char* k_data = q_data + C * el;
  const char* v_data = q_data + 2 * C * el;
  const Tensor cc = cos.compact(), sc = sin.compact();  // rows [0,T) of the tables are used
  // q, k, v as [B,T,H,D] views of the fused projection rows
  const int64_t bthd[4] = {T * 3 * C, 3 * C, D, 1};
  const int64_t cache_bhtd[4] = {H * cap * D, cap * D, D, 1};
  Tensor qh = empty({B, H, T, D}, x.dtype(), true);
  check(deers_rocm_rope_fwd(dt, q_data, bthd, cc.data(), sc.data(), qh.data(), nullptr, B, T, H, D));
  // rotated keys straight into rows [0,T) of the cache, values beside them
  check(deers_rocm_rope_fwd(dt, k_data, bthd, cc.data(), sc.data(), cache.k.data(), cache_bhtd, B, T, H, D));
  const int64_t shape_bhtd[4] = {B, H, T, D}, v_bhtd[4] = {T * 3 * C, D, 3 * C, 1};
  check(deers_rocm_copy_view(dt, v_data, v_bhtd, cache.v.data(), cache_bhtd, shape_bhtd, 4));
  cache.len = T;
  // the fused causal forward reads keys and values from the cache and writes the merged
  // heads [B,T,H*D] directly (its output taken as a [B,H,T,D] view of that buffer)
  Tensor y = empty({B * T, C}, x.dtype(), true);
  Tensor lse = empty({B, H, T}, DType::F32, true);
  const int64_t y_bhtd[4] = {T * C, D, C, 1};
  const double scale = 1.0 / std::sqrt((double)D);
  check(deers_rocm_attn_fwd(dt, qh.data(), nullptr, cache.k.data(), cache_bhtd, cache.v.data(), cache_bhtd,
                            y.data(), y_bhtd, (float*)lse.data(), B, H, T, D, (float)scale));
  if (residual) {
    matmul_add_into(y, wo_, residual->reshape({B * T, C}));
    return *residual;
  }
  return y.matmul(wo_).reshape({B, T, C});
}

Tensor CausalSelfAttention::decode_step(const Tensor& x_t, KvCache& cache, const Tensor& cos,
                                        const Tensor& sin, const Tensor* residual,
                                        const double* norm_eps) const {
  NoGradGuard no_grad;
  if (x_t.layout().ndim() != 3 || x_t.shape()[1] != 1)
    throw std::logic_error("decode_step expects input shape [B, 1, C]");
  if (cache.len >= cache.capacity) throw std::logic_error("decode_step: KV cache is full");
  const int64_t B = x_t.shape()[0], C = x_t.shape()[2], H = n_head_, D = head_dim_;
  const int64_t pos = cache.len, cap = cache.capacity;
  if (pos >= cos.shape()[1]) throw std::logic_error("decode_step: position beyond the RoPE tables");
  const int dt = (int)x_t.dtype();
  const size_t el = size_in_bytes(x_t.dtype());
  const Tensor x_flat = x_t.reshape({B, C});
  // [B, 3C]: q | k | v, each [B, H*D]
  if (!cache.step_qkv.w.defined()) {
    cache.step_qkv = LinearWeight::pack(packed_qkv(cache));
    cache.step_out = LinearWeight::pack(wo_);
  }
  const Tensor qkv = fused_linear(x_flat, cache.step_qkv,
                                  norm_eps ? LinearPrologue::RmsNorm : LinearPrologue::Plain,
                                  norm_eps ? *norm_eps : 0.0, nullptr, &cache.step_out);
  const char* q_data = (const char*)qkv.data();
  const char* k_data = q_data + C * el;
  const char* v_data = q_data + 2 * C * el;
  // row `pos` of the compact [1,T,1,D/2] tables
  const Tensor cc = cos.compact(), sc = sin.compact();
  const char* cos_t = (const char*)cc.data() + pos * (D / 2) * el;
  const char* sin_t = (const char*)sc.data() + pos * (D / 2) * el;
  const int64_t in_strides[2] = {3 * C, D};                          // [B,H,D] inside a [B, 3C] row
  const int64_t kv_strides[3] = {H * cap * D, cap * D, D};
  // rotate q and k at this position, append k and v to the caches, attend over the
  // cache.len + 1 rows: one launch
  Tensor o = empty({B, H * D}, x_t.dtype(), true);
  const double scale = 1.0 / std::sqrt((double)D);
  check(deers_rocm_attn_decode_append(dt, q_data, k_data, v_data, in_strides, cos_t, sin_t, cache.k.data(),
                                      cache.v.data(), kv_strides, o.data(), pos, cap, B, H, D, (float)scale));
  cache.len = pos + 1;
  if (residual) {
    const Tensor res = residual->reshape({B, C});
    fused_linear(o, cache.step_out, LinearPrologue::Plain, 0.0, &res, &cache.step_up);
    return *residual;
  }
  return fused_linear(o, cache.step_out, LinearPrologue::Plain, 0.0, nullptr).reshape({B, 1, C});
}

LinearWeight LinearWeight::pack(const Tensor& w) {
  NoGradGuard no_grad;
  if (w.layout().ndim() != 2) throw std::logic_error("LinearWeight: w [K,N]");
  LinearWeight out;
  out.w = w.detach().compact();
  const int64_t K = w.shape()[0], N = w.shape()[1];
  if (w.dtype() == DType::F16 && N % 32 == 0 && K % 256 == 0 && backed(out.w)) {
    out.tiles = empty({N / 32, K, 32}, w.dtype(), true);
    const int64_t shape[3] = {N / 32, K, 32}, src[3] = {32, N, 1}, dst[3] = {32 * K, 32, 1};
    check(deers_rocm_copy_view((int)w.dtype(), out.w.data(), src, out.tiles.data(), dst, shape, 3));
  }
  return out;
}

Tensor fused_linear(const Tensor& x, const Tensor& w, LinearPrologue f, double eps, const Tensor* acc) {
  LinearWeight lw;
  lw.w = w;
  return fused_linear(x, lw, f, eps, acc);
}

Tensor fused_linear(const Tensor& x, const LinearWeight& lw, LinearPrologue f, double eps, const Tensor* acc,
                    const LinearWeight* next) {
  NoGradGuard no_grad;
  const Tensor& w = lw.w;
  if (x.layout().ndim() != 2 || w.layout().ndim() != 2 || x.shape()[1] != w.shape()[0])
    throw std::logic_error("fused_linear: x [M,K] and w [K,N]");
  const int64_t M = x.shape()[0], K = x.shape()[1], N = w.shape()[1];
  if (acc && (!acc->is_compact() || (int64_t)acc->layout().size() != M * N || acc->dtype() != x.dtype()))
    throw std::logic_error("fused_linear: the accumulator must be a compact [M,N] tensor of x's type");
  if (x.dtype() == DType::F16 && w.dtype() == DType::F16 && M >= 1 && M <= 32 && N % 8 == 0 && K % 256 == 0 &&
      x.is_compact() && w.is_compact() && backed(x)) {
    Tensor y = acc ? *acc : empty({M, N}, x.dtype(), true);
    const bool tiled = lw.tiles.defined();
    if (next && next->tiles.defined())
      check(deers_rocm_decode_linear_hint(next->tiles.data(), next->w.shape()[1], next->w.shape()[0]));
    check(deers_rocm_decode_linear((int)x.dtype(), (int)f, (float)eps, x.data(), K,
                                   tiled ? lw.tiles.data() : w.data(), tiled ? DEERS_ROCM_LINEAR_W_PACKED : N,
                                   const_cast<void*>(y.data()), acc ? 1 : 0, M, N, K));
    return acc ? acc->reshape({M, N}) : y;
  }
  const Tensor fx = f == LinearPrologue::RmsNorm ? rms_norm(x, eps) : f == LinearPrologue::ReluSq ? relu_sq(x) : x;
  if (!acc) return fx.matmul(w);
  matmul_add_into(fx, w, acc->reshape({M, N}));
  return acc->reshape({M, N});
}

void matmul_add_into(const Tensor& a, const Tensor& b, const Tensor& acc) {
  NoGradGuard no_grad;
  Tensor ac = a, bc = b;
  int64_t ars, acs, abs_, brs, bcs, bbs;
  if (!gemm_view(ac, &ars, &acs, &abs_)) { ac = ac.detach().compact(); gemm_view(ac, &ars, &acs, &abs_); }
  if (!gemm_view(bc, &brs, &bcs, &bbs)) { bc = bc.detach().compact(); gemm_view(bc, &brs, &bcs, &bbs); }
  const size_t nd = ac.layout().ndim();
  const int64_t m = ac.shape()[nd - 2], k = ac.shape()[nd - 1], n = bc.shape()[nd - 1];
  int64_t batch = 1;
  for (size_t d = 0; d + 2 < nd; ++d) batch *= ac.shape()[d];
  if (!acc.is_compact() || (int64_t)acc.layout().size() != batch * m * n || acc.dtype() != ac.dtype())
    throw std::logic_error("matmul_add_into: the accumulator must be a compact tensor of the product's shape and type");
  if (backed(ac))
    check(deers_rocm_matmul_acc((int)ac.dtype(), ac.data(), ars, acs, abs_, bc.data(), brs, bcs, bbs,
                                const_cast<void*>(acc.data()), batch, m, n, k));
}

Tensor attention_decode(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache) {
  if (q.layout().ndim() != 3 || k_cache.layout().ndim() != 4 || k_cache.shape() != v_cache.shape())
    throw std::logic_error("attention_decode: q [B,H,D], caches [B,H,L,D]");
  const Tensor qc = q.compact(), kc = k_cache.compact(), vc = v_cache.compact();
  const int64_t B = kc.shape()[0], H = kc.shape()[1], L = kc.shape()[2], D = kc.shape()[3];
  Tensor o = empty({B, H, D}, q.dtype(), true);
  const double scale = 1.0 / std::sqrt((double)D);
  check(deers_rocm_attn_decode((int)q.dtype(), qc.data(), kc.data(), vc.data(), nullptr, o.data(), B, H,
                               L, D, (float)scale));
  return o;
}

}  // namespace deers_host
