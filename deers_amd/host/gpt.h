// The GPT model of src/models/gpt.rs on the ROCm device, in the C++ host: token
// embedding, pre-norm residual blocks (RMSNorm, causal self-attention with RoPE, RMSNorm,
// relu^2 MLP), final RMSNorm and a bias-free LM head.  Same structure, parameter order
// and shapes as the reference; each module runs on the fused device ops of ops.h.
#ifndef DEERS_HOST_GPT_H
#define DEERS_HOST_GPT_H

#include <cstdint>
#include <vector>

#include "ops.h"

namespace deers_host {

// src/nn.rs:203-229: weight [vocab, hidden]; indices of any shape -> [..., hidden].
class Embedding {
 public:
  explicit Embedding(Tensor weight);
  Tensor forward(const Tensor& indices) const;
  std::vector<Tensor> parameters() const { return {weight_}; }

 private:
  Tensor weight_;
};

// src/models/gpt.rs:168-207: down(relu(up(x))^2), weights [in, out], no bias.
class MLP {
 public:
  MLP(Tensor up_proj, Tensor down_proj);
  // [B,T,C] -> [B,T,C]; with `residual` the result is residual + mlp(x), the sum riding on the
  // down projection
  Tensor forward(const Tensor& x, const Tensor* residual = nullptr) const;
  // residual ([B,T,C], compact) += forward(x), the addition riding on the down projection
  // (inference: the residual's storage is updated in place)
  // With `norm_eps` x is the un-normalised stream and its RMSNorm is folded into the up
  // projection where one launch can do both (a generation step's few rows).
  // `cache`, when given, holds (and at first use receives) the two weights in the layout a
  // generation step streams fastest.
  // `after`: the weight of the product that follows the down projection (the next block's
  // packed projection in a generation step), for the prefetch hint.
  void forward_add_into(const Tensor& x, const Tensor& residual, const double* norm_eps = nullptr,
                        KvCache* cache = nullptr, const LinearWeight* after = nullptr) const;
  std::vector<Tensor> parameters() const { return {up_, down_}; }

 private:
  Tensor up_, down_;
};

// src/models/gpt.rs:209-257
class Block {
 public:
  Block(CausalSelfAttention attn, MLP mlp, double eps);
  Tensor forward(const Tensor& x, const Tensor& cos, const Tensor& sin) const;
  // One generated position: x_t [B,1,C] at position cache.len (inference, no autograd).
  // x_t's storage is overwritten with the result when x_t is compact.
  // `next_cache`: the following block's cache (its packed projection is prefetched while this
  // block's last product runs).
  Tensor decode_step(const Tensor& x_t, KvCache& cache, const Tensor& cos, const Tensor& sin,
                     KvCache* next_cache = nullptr) const;
  // The whole prompt x [B,T,C] into an empty cache (inference); x's storage is overwritten
  // like decode_step's.
  Tensor prefill(const Tensor& x, KvCache& cache, const Tensor& cos, const Tensor& sin) const;
  std::vector<Tensor> parameters() const;  // attention, then MLP

 private:
  CausalSelfAttention attn_;
  MLP mlp_;
  double eps_;
};

// src/models/gpt.rs:259-284
struct GPTConfig {
  int64_t vocab_size, sequence_len, n_layer, n_head, n_embd, mlp_hidden_dim;
  double rms_norm_eps;
  float rope_base;
  int64_t head_dim() const { return n_embd / n_head; }
};

// src/models/gpt.rs:286-377
class GPT {
 public:
  // `weights` in parameters() order: wte [V,C]; per block q, k, v, out [C,C], up [C,H],
  // down [H,C]; lm_head [C,V].  Each is attached as a trainable leaf.
  GPT(const GPTConfig& config, const std::vector<Tensor>& weights);
  // Reference initialisation: standard normal embedding (src/nn.rs:209-212), uniform
  // [-1/sqrt(in), 1/sqrt(in)] projections (src/nn.rs:150-170), from a host generator.
  static GPT init_random(const GPTConfig& config, uint64_t seed, DType dtype);

  Tensor forward(const Tensor& idx) const;  // I64 [B,T] -> logits [B,T,V]
  std::vector<Tensor> parameters() const;

  // Generation with a KV cache per block (f16 models; head width 32, 64 or 128).  The
  // reference has no cache: its sampling loop re-runs the whole window for every new
  // token (examples/tinystories_train.rs:250-276).  Here each token costs one pass over
  // the weights and one streaming pass over the cached keys and values.
  std::vector<KvCache> new_caches(int64_t batch, int64_t capacity) const;
  // idx_t I64 [B,1], the token at position caches[0].len -> logits [B,1,V]; equal to row
  // caches[0].len of forward() on the whole prefix.  Inference only.
  Tensor decode_step(const Tensor& idx_t, std::vector<KvCache>& caches) const;
  // The prompt in one pass: idx I64 [B,T0] into empty caches -> logits [B,1,V] of the last
  // prompt position (row T0-1 of forward()); afterwards caches[l].len == T0 and decode_step
  // continues from there.  Inference only.
  Tensor prefill(const Tensor& idx, std::vector<KvCache>& caches) const;
  // Greedy continuation of a prompt (host-side I64 [B, T0], row-major): the prompt goes
  // through prefill, then n_new argmax tokens are appended one decode_step at a time.
  // Returns [B, T0 + n_new] on the host.
  std::vector<int64_t> generate_greedy(const std::vector<int64_t>& prompt, int64_t batch,
                                       int64_t n_new) const;
  const GPTConfig& config() const { return config_; }

 private:
  GPTConfig config_;
  std::vector<Tensor> params_;  // the attached leaves, in parameters() order
  Embedding wte_;
  std::vector<Block> blocks_;
  Tensor lm_head_;
  Tensor cos_, sin_;  // [1, sequence_len, 1, head_dim/2]
};

}  // namespace deers_host
#endif
