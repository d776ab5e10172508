// Tensor, Layout, storage and reverse-mode sweep of the C++ host side; see tensor.h
// for the reference types each class follows.
#include "tensor.h"

#include <algorithm>
#include <atomic>
#include <unordered_set>

#include "../../include/deers_rocm.h"

namespace deers_host {

void check(int rc) {
  if (rc != DEERS_ROCM_OK) throw RocmError(deers_rocm_last_error());
}

// ---- Layout ----------------------------------------------------------------

Layout::Layout(std::vector<int64_t> shape_) : shape(std::move(shape_)) {
  strides.assign(shape.size(), 1);
  for (int d = (int)shape.size() - 2; d >= 0; --d) strides[d] = strides[d + 1] * shape[d + 1];
}

size_t Layout::size() const {
  size_t n = 1;
  for (int64_t s : shape) n *= (size_t)s;
  return n;
}

bool Layout::is_compact() const {
  if (offset != 0) return false;
  int64_t expect = 1;
  for (int d = (int)shape.size() - 1; d >= 0; --d) {
    if (shape[d] != 1 && strides[d] != expect) return false;
    expect *= shape[d];
  }
  return true;
}

Layout Layout::permute(const std::vector<size_t>& dims) const {
  if (dims.size() != shape.size())
    throw std::logic_error("permute: tensor has " + std::to_string(shape.size()) +
                           " dims but got " + std::to_string(dims.size()) + " axes");
  Layout out;
  out.offset = offset;
  for (size_t d : dims) {
    out.shape.push_back(shape.at(d));
    out.strides.push_back(strides.at(d));
  }
  return out;
}

Layout Layout::transpose(size_t a, size_t b) const {
  std::vector<size_t> dims(shape.size());
  for (size_t i = 0; i < dims.size(); ++i) dims[i] = i;
  std::swap(dims.at(a), dims.at(b));
  return permute(dims);
}

// ---- storage -----------------------------------------------------------------

RocmStorage::RocmStorage(size_t len, DType dtype, bool backed) : len_(len), dtype_(dtype) {
  if (backed && len > 0) check(deers_rocm_alloc(len * size_in_bytes(dtype), &ptr_));
}

RocmStorage::~RocmStorage() {
  if (ptr_) (void)deers_rocm_free(ptr_);
}

// ---- NO_GRAD -----------------------------------------------------------------

namespace {
thread_local bool t_no_grad = false;
std::atomic<size_t> g_next_id{0};
}  // namespace

NoGradGuard::NoGradGuard() : prev_(t_no_grad) { t_no_grad = true; }
NoGradGuard::~NoGradGuard() { t_no_grad = prev_; }

// ---- Tensor ------------------------------------------------------------------

Tensor::Tensor(std::shared_ptr<RocmStorage> storage, Layout layout, bool requires_grad,
               std::unique_ptr<TensorOp> op) {
  if (t_no_grad) {
    requires_grad = false;
    op.reset();
  } else {
    if (op && !requires_grad)
      for (const Tensor* dep : op->dependencies()) requires_grad = requires_grad || dep->requires_grad();
    if (!requires_grad) op.reset();
  }
  p_ = std::make_shared<Internal>();
  p_->id = g_next_id.fetch_add(1);
  p_->storage = std::move(storage);
  p_->layout = std::move(layout);
  p_->op = std::move(op);
  p_->requires_grad = requires_grad;
}

Tensor Tensor::full(std::vector<int64_t> shape, DType dtype, float value) {
  Layout l(std::move(shape));
  auto st = std::make_shared<RocmStorage>(l.size(), dtype, true);
  check(deers_rocm_fill((int)dtype, st->ptr(), l.size(), value));
  return Tensor(std::move(st), std::move(l), false, nullptr);
}
Tensor Tensor::zeros(std::vector<int64_t> shape, DType dtype) { return full(std::move(shape), dtype, 0.f); }
Tensor Tensor::ones(std::vector<int64_t> shape, DType dtype) { return full(std::move(shape), dtype, 1.f); }

Tensor Tensor::from_host(const void* data, std::vector<int64_t> shape, DType dtype) {
  Layout l(std::move(shape));
  auto st = std::make_shared<RocmStorage>(l.size(), dtype, true);
  if (l.size()) check(deers_rocm_htod(st->ptr(), data, l.size() * size_in_bytes(dtype)));
  return Tensor(std::move(st), std::move(l), false, nullptr);
}

Tensor Tensor::unbacked(std::vector<int64_t> shape, DType dtype) {
  Layout l(std::move(shape));
  auto st = std::make_shared<RocmStorage>(l.size(), dtype, false);
  return Tensor(std::move(st), std::move(l), false, nullptr);
}

void* Tensor::data() const {
  char* base = static_cast<char*>(p_->storage->ptr());
  return base ? base + p_->layout.offset * (int64_t)size_in_bytes(dtype()) : nullptr;
}

Tensor Tensor::attach() const { return Tensor(p_->storage, p_->layout, true, nullptr); }
Tensor Tensor::detach() const {
  NoGradGuard g;
  return Tensor(p_->storage, p_->layout, false, nullptr);
}

Tensor Tensor::ones_like() const {
  if (!p_->storage->ptr()) return unbacked(shape(), dtype());
  return ones(shape(), dtype());
}
Tensor Tensor::zeros_like() const {
  if (!p_->storage->ptr()) return unbacked(shape(), dtype());
  return zeros(shape(), dtype());
}

void Tensor::to_host(void* dst) const {
  Tensor c = is_compact() ? *this : detach().compact();
  check(deers_rocm_dtoh(dst, c.data(), c.layout().size() * size_in_bytes(dtype())));
}

std::vector<const Tensor*> Tensor::sorted_nodes() const {
  std::vector<const Tensor*> post;
  if (!requires_grad()) return post;
  std::unordered_set<TensorId> visited;
  // iterative DFS post-order
  struct Frame { const Tensor* node; std::vector<const Tensor*> deps; size_t next; };
  std::vector<Frame> stack;
  auto push = [&](const Tensor* t) {
    if (!visited.insert(t->id()).second) return;
    Frame f{t, {}, 0};
    if (t->op())
      for (const Tensor* d : t->op()->dependencies())
        if (d->requires_grad()) f.deps.push_back(d);
    stack.push_back(std::move(f));
  };
  push(this);
  while (!stack.empty()) {
    Frame& f = stack.back();
    if (f.next < f.deps.size()) {
      const Tensor* d = f.deps[f.next++];
      push(d);
    } else {
      post.push_back(f.node);
      stack.pop_back();
    }
  }
  std::reverse(post.begin(), post.end());
  return post;
}

GradientStore Tensor::backward_from(const Tensor& seed) const {
  if (seed.shape() != shape()) throw std::logic_error("backward_from: seed shape differs");
  NoGradGuard no_grad;
  GradientStore grads;
  grads.insert(id(), seed);
  for (const Tensor* node : sorted_nodes()) {
    const Tensor* g = grads.get(node->id());
    if (!g) throw std::logic_error("Gradient must exist");
    const Tensor out_grad = *g;  // keep alive while the op mutates the store
    if (node->op()) node->op()->backward(grads, out_grad);
  }
  return grads;
}

GradientStore Tensor::backward() const {
  NoGradGuard no_grad;
  return backward_from(ones_like());
}

// ---- GradientStore -------------------------------------------------------------

const Tensor* GradientStore::get(TensorId id) const {
  auto it = store_.find(id);
  return it == store_.end() ? nullptr : &it->second;
}

Tensor GradientStore::get_or_insert_with_ones(const Tensor& t) {
  auto it = store_.find(t.id());
  if (it == store_.end()) it = store_.emplace(t.id(), t.ones_like()).first;
  return it->second;
}

void GradientStore::accumulate(const Tensor& tensor, Tensor grad) {
  auto it = store_.find(tensor.id());
  if (it == store_.end())
    store_.emplace(tensor.id(), std::move(grad));
  else
    it->second = it->second.add(grad);
}

}  // namespace deers_host
