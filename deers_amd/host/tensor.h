// Host side of the ROCm attention path, in C++ above the C ABI of
// include/deers_rocm.h: the slice of deers' tensor / autograd machinery that the
// fused attention op lives in, with the reference's names and contracts.
//
//   Layout        src/layout.rs        (shape, element strides, offset; views)
//   RocmStorage   src/storage/cuda.rs  (device buffer owned by the storage value)
//   Tensor        src/tensor.rs:50-130 (Arc-shared, id, op, requires_grad, NO_GRAD)
//   TensorOp      src/ops.rs:82-97     (forward / backward / dependencies / name)
//   GradientStore src/backprop.rs:79-135
//   Tensor::backward / sorted_nodes    src/backprop.rs:13-66
//
// Only the ROCm device exists here; every tensor's storage lives in HBM.  A tensor
// may be created "unbacked" (no allocation) for tests of graph logic alone.
#ifndef DEERS_HOST_TENSOR_H
#define DEERS_HOST_TENSOR_H

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace deers_host {

// Backend failures carry the library's message, the role of Error::Cuda(String)
// (src/error.rs:40-41); programmer errors are std::logic_error (the reference
// panics, AGENTS.md:13-18).
struct RocmError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
void check(int rc);  // throws RocmError with deers_rocm_last_error() if rc != 0

// F16 / F32 carry the library's dtype codes; I64 exists for index tensors only (token
// ids, class targets: DType::I64 in the reference) and no arithmetic kernel takes it.
enum class DType { F16 = 0, F32 = 1, I64 = 2 };
inline size_t size_in_bytes(DType d) { return d == DType::F16 ? 2 : (d == DType::F32 ? 4 : 8); }

// src/layout.rs: shape, strides in elements, offset in elements.
struct Layout {
  std::vector<int64_t> shape;
  std::vector<int64_t> strides;
  int64_t offset = 0;

  Layout() = default;
  explicit Layout(std::vector<int64_t> shape_);  // compact row-major
  size_t ndim() const { return shape.size(); }
  size_t size() const;       // number of elements
  bool is_compact() const;   // row-major with no gaps (src/layout.rs:103-117)
  Layout permute(const std::vector<size_t>& dims) const;  // src/layout.rs:160-175
  Layout transpose(size_t a, size_t b) const;
};

// Device buffer; freed when the last tensor sharing it goes away.
class RocmStorage {
 public:
  RocmStorage(size_t len, DType dtype, bool backed);
  ~RocmStorage();
  RocmStorage(const RocmStorage&) = delete;
  RocmStorage& operator=(const RocmStorage&) = delete;
  void* ptr() const { return ptr_; }
  size_t len() const { return len_; }
  DType dtype() const { return dtype_; }

 private:
  void* ptr_ = nullptr;
  size_t len_;
  DType dtype_;
};

class Tensor;
class GradientStore;
using TensorId = size_t;

// src/ops.rs:82-97.  `forward` consumes the op in the reference; here each op has a
// static `forward(std::unique_ptr<Op>)` that hands the op to the tensor it returns.
class TensorOp {
 public:
  virtual ~TensorOp() = default;
  virtual void backward(GradientStore& grads, const Tensor& out_grad) const = 0;
  virtual std::vector<const Tensor*> dependencies() const = 0;
  virtual const char* name() const = 0;
};

// Thread-local switch that drops autograd tracking (src/tensor.rs:12-14, 29-47).
class NoGradGuard {
 public:
  NoGradGuard();
  ~NoGradGuard();

 private:
  bool prev_;
};

class Tensor {
 public:
  Tensor() = default;
  // src/tensor.rs:85-108: requires_grad is derived from the op's dependencies, and
  // the op is dropped when nothing requires grad or NO_GRAD is set.
  Tensor(std::shared_ptr<RocmStorage> storage, Layout layout, bool requires_grad,
         std::unique_ptr<TensorOp> op);

  static Tensor zeros(std::vector<int64_t> shape, DType dtype);
  static Tensor ones(std::vector<int64_t> shape, DType dtype);
  static Tensor full(std::vector<int64_t> shape, DType dtype, float value);
  static Tensor from_host(const void* data, std::vector<int64_t> shape, DType dtype);
  static Tensor unbacked(std::vector<int64_t> shape, DType dtype);  // graph tests only

  bool defined() const { return static_cast<bool>(p_); }
  TensorId id() const { return p_->id; }
  const Layout& layout() const { return p_->layout; }
  const std::vector<int64_t>& shape() const { return p_->layout.shape; }
  DType dtype() const { return p_->storage->dtype(); }
  bool requires_grad() const { return p_->requires_grad; }
  const TensorOp* op() const { return p_->op.get(); }
  const std::shared_ptr<RocmStorage>& storage() const { return p_->storage; }
  // first element of the view
  void* data() const;

  // Marks a leaf as requiring gradients (src/tensor.rs attach()).
  Tensor attach() const;
  // A leaf sharing this storage and layout with no history (src/tensor.rs detach()).
  Tensor detach() const;

  Tensor ones_like() const;
  Tensor zeros_like() const;
  bool is_compact() const { return p_->layout.is_compact(); }
  // Differentiable views and copies (src/ops.rs:687-727, 1254-1287).
  Tensor permute(const std::vector<size_t>& dims) const;
  Tensor compact() const;  // returns *this when already compact
  Tensor transpose() const;  // swaps the last two axes (a Permute)
  Tensor reshape(const std::vector<int64_t>& shape) const;  // compacts first (src/ops.rs:913)
  Tensor matmul(const Tensor& other) const;
  // Rows of a 2-D tensor picked by a 1-D I64 index tensor (src/ops.rs:1383-1447, dim 0).
  Tensor index_select(size_t dim, const Tensor& indices) const;
  // Log-softmax over the last axis through the fused op (src/tensor.rs:408-427).
  Tensor log_softmax(size_t axis) const;
  // Differentiable element-wise ops used by the contract tests.
  Tensor neg() const;
  Tensor add(const Tensor& other) const;

  // Copies the logical contents to the host in row-major order (a sync point, as
  // to_vec is in the reference).
  void to_host(void* dst) const;

  // Reverse sweep (src/backprop.rs:48-66).  `backward()` seeds ones_like(self);
  // `backward_from` seeds a caller-provided output gradient of the same shape.
  GradientStore backward() const;
  GradientStore backward_from(const Tensor& seed) const;
  // Reverse topological order, output first (src/backprop.rs:13-43).
  std::vector<const Tensor*> sorted_nodes() const;

  bool operator==(const Tensor& o) const { return p_ == o.p_; }

 private:
  struct Internal {
    TensorId id;
    std::shared_ptr<RocmStorage> storage;
    Layout layout;
    std::unique_ptr<TensorOp> op;
    bool requires_grad;
  };
  std::shared_ptr<Internal> p_;
};

// src/backprop.rs:79-135.
class GradientStore {
 public:
  const Tensor* get(TensorId id) const;
  Tensor get_or_insert_with_ones(const Tensor& t);
  // First gradient is stored as is, later ones are summed element-wise.
  void accumulate(const Tensor& tensor, Tensor grad);
  void insert(TensorId id, Tensor t) { store_[id] = std::move(t); }
  size_t len() const { return store_.size(); }
  bool is_empty() const { return store_.empty(); }

 private:
  std::unordered_map<TensorId, Tensor> store_;
};

}  // namespace deers_host
#endif
