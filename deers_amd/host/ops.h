// Operators of the C++ host side.  Neg, EWiseAdd, Permute and Compact follow the
// reference ops of the same names (src/ops.rs:100-127, 130-173, 687-727,
// 1254-1287); FusedCausalAttention is the new op that replaces the composed
// attention core of src/models/gpt.rs:139-144 on the ROCm device, shaped after
// FusedLogSoftmax (src/ops.rs:1186-1251).
#ifndef DEERS_HOST_OPS_H
#define DEERS_HOST_OPS_H

#include <utility>

#include "tensor.h"

namespace deers_host {

// IEEE binary16 bits of a float, round to nearest even (what f16::from_f32 does); the
// host compiler has no half type.
uint16_t f32_to_f16_bits(float f);

class Neg : public TensorOp {
 public:
  explicit Neg(Tensor arg) : arg_(std::move(arg)) {}
  static Tensor forward(std::unique_ptr<Neg> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "Neg"; }

 private:
  Tensor arg_;
};

class EWiseAdd : public TensorOp {
 public:
  EWiseAdd(Tensor a, Tensor b);  // shapes must match (std::logic_error otherwise)
  static Tensor forward(std::unique_ptr<EWiseAdd> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&a_, &b_}; }
  const char* name() const override { return "EWiseAdd"; }

 private:
  Tensor a_, b_;
};

class Permute : public TensorOp {
 public:
  Permute(Tensor arg, std::vector<size_t> axes);
  static Tensor forward(std::unique_ptr<Permute> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "Permute"; }

 private:
  Tensor arg_;
  std::vector<size_t> axes_;
};

class Compact : public TensorOp {
 public:
  explicit Compact(Tensor arg) : arg_(std::move(arg)) {}
  static Tensor forward(std::unique_ptr<Compact> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "Compact"; }

 private:
  Tensor arg_;
};

// Same storage under a new compact shape; the argument is compacted first, which is
// where the reference's head merge copy happens (src/ops.rs:899-934).
class Reshape : public TensorOp {
 public:
  Reshape(Tensor arg, std::vector<int64_t> new_shape);
  static Tensor forward(std::unique_ptr<Reshape> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "Reshape"; }

 private:
  Tensor arg_;
  std::vector<int64_t> new_shape_;
};

// Batched a[..,m,k] @ b[..,k,n] with equal batch dimensions (src/ops.rs:1012-1106);
// operands go to the library by stride, so the transposed views of the backward
// (dA = dC @ B^T, dB = A^T @ dC) cost no copy.
class MatMul : public TensorOp {
 public:
  MatMul(Tensor a, Tensor b);
  static Tensor forward(std::unique_ptr<MatMul> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&a_, &b_}; }
  const char* name() const override { return "MatMul"; }

 private:
  Tensor a_, b_;
};

// a @ b + c in one launch: a MatMul followed by an EWiseAdd in the reference (the residual
// connections of a block, src/models/gpt.rs:237-239); backward as those two ops
// (src/ops.rs:1089-1101 and the binary add's pass-through).
class MatMulAdd : public TensorOp {
 public:
  MatMulAdd(Tensor a, Tensor b, Tensor c);
  static Tensor forward(std::unique_ptr<MatMulAdd> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&a_, &b_, &c_}; }
  const char* name() const override { return "MatMulAdd"; }

 private:
  Tensor a_, b_, c_;  // c_ compacted by the constructor
};
Tensor matmul_add(const Tensor& a, const Tensor& b, const Tensor& c);

// y = softmax(q k^T * scale + causal mask) v for q, k, v logical [B,H,T,D] (views
// welcome: any strides with a unit D stride go to the kernels as they are, other
// views are compacted first, as FusedLogSoftmax::forward compacts its argument,
// src/ops.rs:1205).  Returns a [B,H,T,D] tensor whose memory is [B,T,H,D], so that the
// module's permute + reshape (src/models/gpt.rs:145) is a view, and keeps (O, LSE) for the
// backward, which overwrites fresh dq/dk/dv buffers (dv in v's memory order) and hands
// them to GradientStore::accumulate.
// Head widths the fused kernels do not take (they take 32, 64, 128; the reference's own GPT
// test runs head_dim 2, tests/gpt.rs:38-49) go through the reference's op chain on the
// device instead, kernel by kernel (src/models/gpt.rs:139-144 forward; the backward bodies of
// src/ops.rs:1089-1101, 422-425, 1186-1251, 638-643), materialising [B,H,T,T] tensors the
// way the reference does; same op, same contract, only slower.
class FusedCausalAttention : public TensorOp {
 public:
  FusedCausalAttention(Tensor q, Tensor k, Tensor v, double scale);
  static Tensor forward(std::unique_ptr<FusedCausalAttention> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&q_, &k_, &v_}; }
  const char* name() const override { return "FusedCausalAttention"; }

 private:
  Tensor q_, k_, v_;
  double scale_;
  Tensor saved_o_, saved_lse_;  // set by forward, created with no op
  Tensor saved_p_, saved_lsm_;  // composed path: softmax [B,H,T,T] and its logarithm

  static bool fused_kernels_take(int64_t D) { return D == 32 || D == 64 || D == 128; }
  static Tensor forward_composed(std::unique_ptr<FusedCausalAttention> self);
  void backward_composed(GradientStore& grads, const Tensor& out_grad) const;
};

// src/ops.rs:1186-1251: log-softmax over the last axis in one kernel, its output saved
// for the backward (out_grad - exp(lsm) * rowsum(out_grad)).  Tensor::log_softmax takes
// this path when the axis is the last one (src/tensor.rs:408-427); other axes are not
// part of this host.
class FusedLogSoftmax : public TensorOp {
 public:
  FusedLogSoftmax(Tensor arg, size_t axis);  // std::logic_error unless axis is the last
  static Tensor forward(std::unique_ptr<FusedLogSoftmax> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "FusedLogSoftmax"; }

 private:
  Tensor arg_;
  size_t axis_;
  Tensor lsm_output_;  // no op, no grad: saved like the reference's lsm_output
};

// Rows of a [n, width] table picked by 1-D I64 indices (IndexSelect, src/ops.rs:1383-1447,
// dim 0 only: the embedding lookup of src/nn.rs:216-224).  The backward scatters the
// output gradient into zeros of the table's shape in ascending position order
// (index_add), so repeated tokens accumulate exactly as on the reference's CPU path.
class IndexSelect : public TensorOp {
 public:
  IndexSelect(Tensor arg, size_t dim, Tensor indices);
  static Tensor forward(std::unique_ptr<IndexSelect> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "IndexSelect"; }

 private:
  Tensor arg_, indices_;
};

// RMSNorm::forward (src/nn.rs:244-251), x * (mean(x^2, last) + eps)^-0.5, as one op with
// one kernel each way instead of the reference's chain of five ops.
class RmsNorm : public TensorOp {
 public:
  RmsNorm(Tensor arg, double eps) : arg_(std::move(arg)), eps_(eps) {}
  static Tensor forward(std::unique_ptr<RmsNorm> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "RmsNorm"; }

 private:
  Tensor arg_;  // compacted by forward
  double eps_;
};
Tensor rms_norm(const Tensor& x, double eps);

// relu(x)^2, the MLP activation `y.relu(); &y * &y` (src/models/gpt.rs:196-197), as one op.
class ReluSq : public TensorOp {
 public:
  explicit ReluSq(Tensor arg) : arg_(std::move(arg)) {}
  static Tensor forward(std::unique_ptr<ReluSq> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&arg_}; }
  const char* name() const override { return "ReluSq"; }

 private:
  Tensor arg_;
};
Tensor relu_sq(const Tensor& x);

// loss::cross_entropy (src/loss.rs:21-24) on logits [N, V] and I64 targets [N] as one op:
// the forward streams the logits once and keeps each row's ln-sum-exp, the backward
// writes (softmax - onehot) * upstream / N; the [N, V] log-probabilities of the
// reference's log_softmax + gather + sum chain are never materialised.  The loss is an
// F32 tensor of shape [1] whatever the logits' type.
class CrossEntropy : public TensorOp {
 public:
  CrossEntropy(Tensor logits, Tensor targets);
  static Tensor forward(std::unique_ptr<CrossEntropy> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&logits_}; }
  const char* name() const override { return "CrossEntropy"; }

 private:
  Tensor logits_, targets_;
  Tensor row_lse_;  // [N] f32, set by forward
  // d loss / d logits for an upstream gradient of one, written by a forward whose logits carry
  // a gradient; handed over (and released here) by the first backward
  mutable Tensor grad_for_one_;
};
Tensor cross_entropy(const Tensor& logits, const Tensor& targets);

// apply_rotary_emb on a [B,T,H,D] projection followed by permute([0,2,1,3])
// (src/models/gpt.rs:49-73, 135-136) as one op: returns the rotated heads as compact
// [B,H,T,D]; the backward hands the [B,T,H,D] gradient to the projection.  cos and
// sin are the tables of precompute_rotary_embeddings and carry no gradient.
class RotaryHeads : public TensorOp {
 public:
  RotaryHeads(Tensor x, Tensor cos, Tensor sin);
  static Tensor forward(std::unique_ptr<RotaryHeads> self);
  void backward(GradientStore& grads, const Tensor& out_grad) const override;
  std::vector<const Tensor*> dependencies() const override { return {&x_}; }
  const char* name() const override { return "RotaryHeads"; }

 private:
  Tensor x_, cos_, sin_;
};

// cos, sin tables [1,T,1,D/2] in `dtype` (src/models/gpt.rs:12-47): f32 arithmetic on
// the host, then one cast.
std::pair<Tensor, Tensor> precompute_rotary_embeddings(int64_t seq_len, int64_t head_dim,
                                                       float base, DType dtype);
Tensor rotary_heads(const Tensor& x, const Tensor& cos, const Tensor& sin);

// The call site of src/models/gpt.rs:139-144: scale = 1/sqrt(head_dim) computed in
// f64 and narrowed to f32 (src/storage.rs:115-117).
Tensor causal_self_attention(const Tensor& q, const Tensor& k, const Tensor& v);

// The attention module of src/models/gpt.rs:76-148 on the ROCm device: bias-free
// q/k/v/out projections with weights [in, out] (y = x @ W, src/nn.rs:183-190), RoPE on
// queries and keys, the fused causal attention core, head merge, output projection.
// Keys (rotated) and values of the tokens seen so far, [B,H,L_cap,D]; rows [0,len)
// are valid.  The reference keeps no cache and re-runs the whole window per generated
// token (examples/tinystories_train.rs:250-276).
// acc += a @ b in one launch; acc compact, of the product's shape and type.  Inference
// helper: nothing is recorded for autograd, the accumulator's storage is updated in place.
void matmul_add_into(const Tensor& a, const Tensor& b, const Tensor& acc);

// f(x) @ w, or acc += f(x) @ w when `acc` is given, for x [M,K] and w [K,N]; f is the
// weightless RMSNorm over x's rows (src/nn.rs:244-251) or relu(x)^2
// (src/models/gpt.rs:196-203).  The few rows of a generation step (f16, M <= 32) take one
// launch (deers_rocm_decode_linear); any other shape runs the separate ops.  Inference
// helper: nothing is recorded for autograd.
enum class LinearPrologue { Plain = 0, RmsNorm = 1, ReluSq = 2 };
Tensor fused_linear(const Tensor& x, const Tensor& w, LinearPrologue f, double eps, const Tensor* acc);
// A weight [K,N] as generation steps read it: beside the row-major tensor (shared with the
// model) a copy stored as [N/32][K][32], the layout in which the 32 columns one workgroup of
// the few-rows kernel streams are contiguous (f16, N % 32 == 0, K % 256 == 0; otherwise
// `tiles` stays undefined and the row-major tensor is used).
struct LinearWeight {
  Tensor w;      // [K,N] row-major
  Tensor tiles;  // packed copy, or undefined
  static LinearWeight pack(const Tensor& w);
};
// `next`: the weight of the product that follows this one, if known; its tiles are then
// pulled into L2 by CUs this launch leaves idle (deers_rocm_decode_linear_hint).
Tensor fused_linear(const Tensor& x, const LinearWeight& w, LinearPrologue f, double eps, const Tensor* acc,
                    const LinearWeight* next = nullptr);

struct KvCache {
  Tensor k, v;
  // [C, 3C] = (Wq | Wk | Wv), packed by the first decode_step that uses this cache so a
  // step runs one projection GEMM instead of three; the weights must not change while
  // the cache lives
  Tensor wqkv;
  // the block's four products of a generation step in the few-rows kernel's layout,
  // packed by the first decode_step (same proviso)
  LinearWeight step_qkv, step_out, step_up, step_down;
  int64_t len = 0, capacity = 0;
  static KvCache create(int64_t B, int64_t H, int64_t capacity, int64_t D, DType dtype);
};

class CausalSelfAttention {
 public:
  CausalSelfAttention(int64_t n_embd, int64_t n_head, Tensor wq, Tensor wk, Tensor wv, Tensor wo);
  // x [B,T,C] with the RoPE tables of precompute_rotary_embeddings -> [B,T,C]
  // with `residual` ([B,T,C]) the result is residual + attention(x), the sum riding on the
  // output projection
  Tensor forward(const Tensor& x, const Tensor& cos, const Tensor& sin, const Tensor* residual = nullptr) const;
  // One generation step (inference, no autograd): x_t [B,1,C] is the token at position
  // cache.len; its rotated key and its value are appended to the cache and the query
  // attends to all cache.len+1 positions through the decode kernel.  Returns [B,1,C],
  // equal to row cache.len of forward() on the whole prefix.
  // With `residual` ([B,1,C], compact) the output projection is added into it in place
  // (one launch for `residual + attn(x_t)`) and it is returned.
  // With `norm_eps` x_t is the un-normalised residual stream and its RMSNorm happens inside
  // the projection's launch.
  Tensor decode_step(const Tensor& x_t, KvCache& cache, const Tensor& cos, const Tensor& sin,
                     const Tensor* residual = nullptr, const double* norm_eps = nullptr) const;
  // The whole prompt at once (inference, no autograd): x [B,T,C] at positions [0,T) of an
  // empty cache.  Rotated keys and values go to rows [0,T) of the cache, the fused causal
  // forward reads them from there; returns [B,T,C] equal to forward() (same kernels), and
  // leaves the cache as T decode_steps would (to the rounding of the projection GEMMs).
  // `residual` ([B,T,C], compact) as in decode_step.
  Tensor prefill(const Tensor& x, KvCache& cache, const Tensor& cos, const Tensor& sin,
                 const Tensor* residual = nullptr) const;
  std::vector<Tensor> parameters() const { return {wq_, wk_, wv_, wo_}; }

 private:
  const Tensor& packed_qkv(KvCache& cache) const;  // packs (Wq | Wk | Wv) at first use
  int64_t n_head_, head_dim_;
  Tensor wq_, wk_, wv_, wo_;
};

// One query token per (b,h) against a KV cache: q [B,H,D], caches [B,H,L,D] compact;
// not differentiable (inference only).
Tensor attention_decode(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache);

}  // namespace deers_host
#endif
