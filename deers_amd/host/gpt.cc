#include "gpt.h"

#include "../../include/deers_rocm.h"

#include <cmath>
#include <cstring>
#include <random>

namespace deers_host {

Embedding::Embedding(Tensor weight) : weight_(std::move(weight)) {
  if (weight_.layout().ndim() != 2) throw std::logic_error("embedding weight must be [vocab, hidden]");
}

Tensor Embedding::forward(const Tensor& indices) const {
  const int64_t hidden = weight_.shape()[1];
  std::vector<int64_t> final_dims = indices.shape();
  final_dims.push_back(hidden);
  // indices.reshape([size]): an index tensor carries no gradient, so a plain view of the
  // compact data under the flat shape serves
  const Tensor ic = indices.compact();
  const Tensor flat(ic.storage(), Layout({(int64_t)ic.layout().size()}), false, nullptr);
  return weight_.index_select(0, flat).reshape(final_dims);
}

MLP::MLP(Tensor up_proj, Tensor down_proj) : up_(std::move(up_proj)), down_(std::move(down_proj)) {
  if (up_.layout().ndim() != 2 || down_.layout().ndim() != 2 || up_.shape()[1] != down_.shape()[0] ||
      up_.shape()[0] != down_.shape()[1])
    throw std::logic_error("MLP weights must be [n_embd, hidden] and [hidden, n_embd]");
}

Tensor MLP::forward(const Tensor& x, const Tensor* residual) const {
  if (x.layout().ndim() != 3) throw std::logic_error("MLP expects input shape [B, T, C]");
  const int64_t B = x.shape()[0], T = x.shape()[1], C = x.shape()[2];
  const Tensor y = relu_sq(x.reshape({B * T, C}).matmul(up_));  // [B*T, H]
  if (residual) return matmul_add(y, down_, residual->reshape({B * T, C})).reshape({B, T, C});
  return y.matmul(down_).reshape({B, T, C});
}

void MLP::forward_add_into(const Tensor& x, const Tensor& residual, const double* norm_eps,
                           KvCache* cache, const LinearWeight* after) const {
  NoGradGuard no_grad;
  if (x.layout().ndim() != 3) throw std::logic_error("MLP expects input shape [B, T, C]");
  const int64_t B = x.shape()[0], T = x.shape()[1], C = x.shape()[2];
  const Tensor res = residual.reshape({B * T, C});
  // [B*T, H] before the activation, which rides on the down projection
  LinearWeight up, down;
  if (cache) {
    if (!cache->step_up.w.defined()) {
      cache->step_up = LinearWeight::pack(up_);
      cache->step_down = LinearWeight::pack(down_);
    }
    up = cache->step_up;
    down = cache->step_down;
  } else {
    up.w = up_;
    down.w = down_;
  }
  const Tensor u = fused_linear(x.reshape({B * T, C}), up,
                                norm_eps ? LinearPrologue::RmsNorm : LinearPrologue::Plain,
                                norm_eps ? *norm_eps : 0.0, nullptr, &down);
  fused_linear(u, down, LinearPrologue::ReluSq, 0.0, &res, after);
}

Block::Block(CausalSelfAttention attn, MLP mlp, double eps)
    : attn_(std::move(attn)), mlp_(std::move(mlp)), eps_(eps) {}

Tensor Block::forward(const Tensor& x, const Tensor& cos, const Tensor& sin) const {
  // x + attn(norm(x)) and h + mlp(norm(h)) (src/models/gpt.rs:237-239), each sum riding on
  // the branch's last product
  const Tensor h = attn_.forward(rms_norm(x, eps_), cos, sin, &x);
  return mlp_.forward(rms_norm(h, eps_), &h);
}

Tensor Block::decode_step(const Tensor& x_t, KvCache& cache, const Tensor& cos, const Tensor& sin,
                          KvCache* next_cache) const {
  NoGradGuard no_grad;
  // the residual stream is updated in place: both additions ride on the last product of
  // their branch (x_t's storage is overwritten; inference only)
  const Tensor h = x_t.compact();
  attn_.decode_step(h, cache, cos, sin, &h, &eps_);
  mlp_.forward_add_into(h, h, &eps_, &cache, next_cache ? &next_cache->step_qkv : nullptr);
  return h;
}

Tensor Block::prefill(const Tensor& x, KvCache& cache, const Tensor& cos, const Tensor& sin) const {
  NoGradGuard no_grad;
  const Tensor h = x.compact();
  attn_.prefill(rms_norm(h, eps_), cache, cos, sin, &h);
  mlp_.forward_add_into(rms_norm(h, eps_), h);
  return h;
}

std::vector<Tensor> Block::parameters() const {
  std::vector<Tensor> p = attn_.parameters();
  for (const Tensor& t : mlp_.parameters()) p.push_back(t);
  return p;
}

// Attaches every weight as a trainable leaf (once: a leaf's id is what the gradient
// store and the optimizer key on) after checking count and the embedding's shape.
static std::vector<Tensor> checked_attach(const GPTConfig& c, const std::vector<Tensor>& ws) {
  if (c.n_embd % c.n_head) throw std::logic_error("n_embd must be divisible by n_head");
  if ((int64_t)ws.size() != 2 + 6 * c.n_layer)
    throw std::logic_error("GPT: expected " + std::to_string(2 + 6 * c.n_layer) + " weight tensors");
  if (ws[0].shape() != std::vector<int64_t>{c.vocab_size, c.n_embd})
    throw std::logic_error("GPT: wte must be [vocab_size, n_embd]");
  if (ws.back().shape() != std::vector<int64_t>{c.n_embd, c.vocab_size})
    throw std::logic_error("GPT: lm_head must be [n_embd, vocab_size]");
  std::vector<Tensor> out;
  out.reserve(ws.size());
  for (const Tensor& w : ws) out.push_back(w.requires_grad() && !w.op() ? w : w.attach());
  return out;
}

GPT::GPT(const GPTConfig& config, const std::vector<Tensor>& weights)
    : config_(config), params_(checked_attach(config, weights)), wte_(params_[0]) {
  for (int64_t l = 0; l < config.n_layer; ++l) {
    const Tensor* b = &params_[1 + 6 * l];
    blocks_.emplace_back(CausalSelfAttention(config.n_embd, config.n_head, b[0], b[1], b[2], b[3]),
                         MLP(b[4], b[5]), config.rms_norm_eps);
  }
  lm_head_ = params_.back();
  auto tables = precompute_rotary_embeddings(config.sequence_len, config.head_dim(), config.rope_base,
                                             params_[0].dtype());
  cos_ = tables.first;
  sin_ = tables.second;
}

GPT GPT::init_random(const GPTConfig& c, uint64_t seed, DType dtype) {
  if (dtype != DType::F32 && dtype != DType::F16) throw std::logic_error("GPT: f16 or f32 weights");
  std::mt19937_64 gen(seed);
  auto make = [&](int64_t rows, int64_t cols, bool normal) {
    std::vector<float> host((size_t)rows * cols);
    if (normal) {
      std::normal_distribution<float> d(0.f, 1.f);
      for (float& x : host) x = d(gen);
    } else {
      const float k = 1.0f / std::sqrt((float)rows);
      std::uniform_real_distribution<float> d(-k, k);
      for (float& x : host) x = d(gen);
    }
    if (dtype == DType::F32) return Tensor::from_host(host.data(), {rows, cols}, DType::F32);
    std::vector<uint16_t> half(host.size());
    for (size_t i = 0; i < host.size(); ++i) half[i] = f32_to_f16_bits(host[i]);
    return Tensor::from_host(half.data(), {rows, cols}, DType::F16);
  };
  std::vector<Tensor> w;
  w.push_back(make(c.vocab_size, c.n_embd, true));
  for (int64_t l = 0; l < c.n_layer; ++l) {
    for (int i = 0; i < 4; ++i) w.push_back(make(c.n_embd, c.n_embd, false));
    w.push_back(make(c.n_embd, c.mlp_hidden_dim, false));
    w.push_back(make(c.mlp_hidden_dim, c.n_embd, false));
  }
  w.push_back(make(c.n_embd, c.vocab_size, false));
  return GPT(c, w);
}

Tensor GPT::forward(const Tensor& idx) const {
  if (idx.layout().ndim() != 2) throw std::logic_error("GPT expects token ids with shape [B, T]");
  const int64_t B = idx.shape()[0], T = idx.shape()[1];
  if (T > cos_.shape()[1]) throw std::logic_error("sequence length exceeds rotary cache");
  // cos.narrow(1, 0, T): the first T rows of the compact [1, L, 1, D/2] tables
  const Layout rows({1, T, 1, cos_.shape()[3]});
  const Tensor cos(cos_.storage(), rows, false, nullptr), sin(sin_.storage(), rows, false, nullptr);
  Tensor x = wte_.forward(idx);  // [B, T, C]
  for (const Block& block : blocks_) x = block.forward(x, cos, sin);
  x = rms_norm(x, config_.rms_norm_eps);
  const Tensor logits = x.reshape({B * T, config_.n_embd}).matmul(lm_head_);  // [B*T, V]
  return logits.reshape({B, T, config_.vocab_size});
}

std::vector<Tensor> GPT::parameters() const { return params_; }

std::vector<KvCache> GPT::new_caches(int64_t batch, int64_t capacity) const {
  if (capacity > config_.sequence_len) throw std::logic_error("cache capacity exceeds rotary cache");
  std::vector<KvCache> caches;
  for (int64_t l = 0; l < config_.n_layer; ++l)
    caches.push_back(KvCache::create(batch, config_.n_head, capacity, config_.head_dim(), params_[0].dtype()));
  return caches;
}

Tensor GPT::decode_step(const Tensor& idx_t, std::vector<KvCache>& caches) const {
  NoGradGuard no_grad;
  if (idx_t.layout().ndim() != 2 || idx_t.shape()[1] != 1)
    throw std::logic_error("decode_step expects token ids with shape [B, 1]");
  if ((int64_t)caches.size() != config_.n_layer) throw std::logic_error("decode_step: one cache per block");
  const int64_t B = idx_t.shape()[0];
  Tensor x = wte_.forward(idx_t);  // [B, 1, C]
  for (size_t l = 0; l < blocks_.size(); ++l)
    x = blocks_[l].decode_step(x, caches[l], cos_, sin_, l + 1 < blocks_.size() ? &caches[l + 1] : nullptr);
  x = rms_norm(x, config_.rms_norm_eps);
  return x.reshape({B, config_.n_embd}).matmul(lm_head_).reshape({B, 1, config_.vocab_size});
}

Tensor GPT::prefill(const Tensor& idx, std::vector<KvCache>& caches) const {
  NoGradGuard no_grad;
  if (idx.layout().ndim() != 2) throw std::logic_error("prefill expects token ids with shape [B, T]");
  if ((int64_t)caches.size() != config_.n_layer) throw std::logic_error("prefill: one cache per block");
  const int64_t B = idx.shape()[0], T = idx.shape()[1], C = config_.n_embd;
  Tensor x = wte_.forward(idx);  // [B, T, C]
  for (size_t l = 0; l < blocks_.size(); ++l) x = blocks_[l].prefill(x, caches[l], cos_, sin_);
  // only the last position's logits are needed: its rows out of the residual stream first
  Tensor last(std::make_shared<RocmStorage>((size_t)(B * C), x.dtype(), true), Layout({B, C}), false, nullptr);
  const int64_t shape[2] = {B, C}, src[2] = {T * C, 1}, dst[2] = {C, 1};
  const size_t el = size_in_bytes(x.dtype());
  check(deers_rocm_copy_view((int)x.dtype(), (const char*)x.data() + (T - 1) * C * el, src, last.data(), dst,
                             shape, 2));
  last = rms_norm(last, config_.rms_norm_eps);
  return last.matmul(lm_head_).reshape({B, 1, config_.vocab_size});
}

std::vector<int64_t> GPT::generate_greedy(const std::vector<int64_t>& prompt, int64_t batch,
                                          int64_t n_new) const {
  if (batch < 1 || prompt.empty() || prompt.size() % (size_t)batch)
    throw std::logic_error("generate: the prompt is [batch, T0] with T0 >= 1");
  NoGradGuard no_grad;
  const int64_t t0 = (int64_t)prompt.size() / batch, total = t0 + n_new, V = config_.vocab_size;
  std::vector<KvCache> caches = new_caches(batch, total);
  // the prompt goes through the batched forward once; after it each step's ids are the
  // previous step's argmax, picked on the device: nothing in the loop waits for the host
  std::vector<Tensor> picked;  // one [batch] id tensor per generated position
  auto pick = [&](const Tensor& logits) {  // [batch, 1, V], compact
    auto st = std::make_shared<RocmStorage>((size_t)batch, DType::I64, true);
    Tensor next(st, Layout({batch}), false, nullptr);
    check(deers_rocm_argmax_rows((int)logits.dtype(), logits.data(), (int64_t*)next.data(), batch, V));
    picked.push_back(next);
  };
  if (n_new > 0) pick(prefill(Tensor::from_host(prompt.data(), {batch, t0}, DType::I64), caches));
  for (int64_t t = t0; t < total - 1; ++t) {
    const Tensor ids_t(picked.back().storage(), Layout({batch, 1}), false, nullptr);
    pick(decode_step(ids_t, caches));
  }
  std::vector<int64_t> out((size_t)(batch * total));
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t t = 0; t < t0; ++t) out[b * total + t] = prompt[b * t0 + t];
  std::vector<int64_t> col((size_t)batch);
  for (size_t i = 0; i < picked.size(); ++i) {
    picked[i].to_host(col.data());
    for (int64_t b = 0; b < batch; ++b) out[b * total + t0 + (int64_t)i] = col[b];
  }
  return out;
}

}  // namespace deers_host
