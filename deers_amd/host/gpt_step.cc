// Times the end-to-end GPT training step on the ROCm device: forward, cross-entropy,
// reverse sweep, gradient-norm clipping and AdamW, on synthetic token ids and
// random-init weights (the reference's loop: examples/tinystories_train.rs).  Prints one
// JSON line: wall time per step between two stream synchronisations, tokens per second,
// and, from a second profiled pass, the time per kernel family.
//
//   gpt_step vocab seq n_layer n_head n_embd mlp_hidden batch steps warmup [tune]
// `tune` lets the first step pick the fastest library GEMM kernel per problem.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "../../include/deers_rocm.h"
#include "gpt.h"
#include "optim.h"

using namespace deers_host;

// gpt_step generate vocab seq n_layer n_head n_embd mlp_hidden batch prompt_len new_tokens [tune]:
// greedy generation with KV caches on an f16 model; times the decode steps that follow
// the prompt.  `tune` picks the library GEMM kernel of each of the step's four problems by
// timing during the prompt.
static int run_generate(int argc, char** argv) {
  if (argc < 11) {
    std::fprintf(stderr, "usage: gpt_step generate vocab seq n_layer n_head n_embd mlp_hidden batch prompt_len new_tokens [tune]\n");
    return 2;
  }
  check(deers_rocm_init(0));
  const bool tune = argc > 11 && std::string(argv[11]) == "tune";
  check(deers_rocm_matmul_tune(tune ? 1 : 0));
  GPTConfig cfg;
  cfg.vocab_size = std::atoll(argv[2]);
  cfg.sequence_len = std::atoll(argv[3]);
  cfg.n_layer = std::atoll(argv[4]);
  cfg.n_head = std::atoll(argv[5]);
  cfg.n_embd = std::atoll(argv[6]);
  cfg.mlp_hidden_dim = std::atoll(argv[7]);
  cfg.rms_norm_eps = 1e-5;
  cfg.rope_base = 10000.0f;
  const int64_t B = std::atoll(argv[8]), t0 = std::atoll(argv[9]), n_new = std::atoll(argv[10]);
  GPT model = GPT::init_random(cfg, 1234, DType::F16);
  std::mt19937_64 gen(7);
  std::uniform_int_distribution<int64_t> tok(0, cfg.vocab_size - 1);
  std::vector<int64_t> prompt((size_t)(B * t0));
  for (auto& x : prompt) x = tok(gen);
  const Tensor prompt_dev = Tensor::from_host(prompt.data(), {B, t0}, DType::I64);
  // the prompt fills the caches in one prefill pass: once untimed (first-use set-up), then
  // timed on fresh caches
  std::vector<KvCache> caches = model.new_caches(B, t0 + n_new);
  Tensor logits = model.prefill(prompt_dev, caches);
  check(deers_rocm_sync());
  double prefill_ms = 1e30;
  for (int rep = 0; rep < 3; ++rep) {
    caches = model.new_caches(B, t0 + n_new);
    check(deers_rocm_sync());
    const auto p0 = std::chrono::steady_clock::now();
    logits = model.prefill(prompt_dev, caches);
    check(deers_rocm_sync());
    prefill_ms = std::min(prefill_ms, std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - p0).count());
  }
  // the generated part: every step's ids are the previous step's argmax, picked on the
  // device, so the host only enqueues
  const auto s0 = std::chrono::steady_clock::now();
  for (int64_t t = 0; t < n_new; ++t) {
    auto st = std::make_shared<RocmStorage>((size_t)B, DType::I64, true);
    Tensor next(st, Layout({B, 1}), false, nullptr);
    check(deers_rocm_argmax_rows((int)logits.dtype(), logits.data(), (int64_t*)next.data(), B, cfg.vocab_size));
    logits = model.decode_step(next, caches);
  }
  // how long the host needed to enqueue the steps: close to the wall time means the loop is
  // bound by the launch rate, well below it means the device is the limit
  const double enqueue_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - s0).count() / n_new;
  check(deers_rocm_sync());
  const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - s0).count() / n_new;
  // a few more steps with every launch bracketed by events: device time per kernel family
  std::string kernels = "{";
  {
    const int prof_steps = 8;
    std::vector<KvCache> c2 = model.new_caches(B, t0 + prof_steps);
    logits = model.prefill(prompt_dev, c2);
    check(deers_rocm_sync());
    check(deers_rocm_profile_enable(1));
    for (int t = 0; t < prof_steps; ++t) {
      auto st = std::make_shared<RocmStorage>((size_t)B, DType::I64, true);
      Tensor next(st, Layout({B, 1}), false, nullptr);
      check(deers_rocm_argmax_rows((int)logits.dtype(), logits.data(), (int64_t*)next.data(), B, cfg.vocab_size));
      logits = model.decode_step(next, c2);
    }
    int rows = 0;
    check(deers_rocm_profile_collect(&rows));
    for (int r = 0; r < rows; ++r) {
      const char* name = nullptr;
      int64_t calls = 0;
      float total_ms = 0;
      check(deers_rocm_profile_row(r, &name, &calls, &total_ms));
      char buf[256];
      std::snprintf(buf, sizeof(buf), "%s\"%s\": {\"calls_per_step\": %.1f, \"us_per_step\": %.1f}", r ? ", " : "",
                    name, (double)calls / prof_steps, 1e3 * total_ms / prof_steps);
      kernels += buf;
    }
    check(deers_rocm_profile_enable(0));
  }
  kernels += "}";
  int64_t n_params = 0;
  for (const Tensor& p : model.parameters()) n_params += (int64_t)p.layout().size();
  const double kv_bytes = 2.0 * cfg.n_layer * B * cfg.n_head * (t0 + n_new / 2.0) * cfg.head_dim() * 2;
  const double w_bytes = 2.0 * (n_params - cfg.vocab_size * cfg.n_embd);  // every weight but the embedding table
  std::printf("{\"mode\": \"generate\", \"ms_per_token_step\": %.4f, \"tokens_per_s\": %.1f, \"batch\": %lld, "
              "\"context\": %lld, \"new_tokens\": %lld, \"bytes_per_step\": %.0f, \"GB_per_s\": %.1f, "
              "\"host_enqueue_ms_per_step\": %.4f, \"prefill_ms\": %.3f, \"prefill_tokens_per_s\": %.0f, \"kernels\": %s}\n",
              ms, 1e3 * B / ms, (long long)B, (long long)t0, (long long)n_new, kv_bytes + w_bytes,
              (kv_bytes + w_bytes) / (ms * 1e-3) / 1e9, enqueue_ms, prefill_ms, 1e3 * B * t0 / prefill_ms, kernels.c_str());
  return 0;
}

int main(int argc, char** argv) {
  if (argc > 1 && std::string(argv[1]) == "generate") {
    try {
      return run_generate(argc, argv);
    } catch (const std::exception& e) {
      std::fprintf(stderr, "gpt_step: %s\n", e.what());
      return 1;
    }
  }
  if (argc < 10) {
    std::fprintf(stderr, "usage: gpt_step vocab seq n_layer n_head n_embd mlp_hidden batch steps warmup\n");
    return 2;
  }
  try {
    check(deers_rocm_init(0));
    const bool tune = argc > 10 && std::string(argv[10]) == "tune";
    check(deers_rocm_matmul_tune(tune ? 1 : 0));
    GPTConfig cfg;
    cfg.vocab_size = std::atoll(argv[1]);
    cfg.sequence_len = std::atoll(argv[2]);
    cfg.n_layer = std::atoll(argv[3]);
    cfg.n_head = std::atoll(argv[4]);
    cfg.n_embd = std::atoll(argv[5]);
    cfg.mlp_hidden_dim = std::atoll(argv[6]);
    cfg.rms_norm_eps = 1e-5;
    cfg.rope_base = 10000.0f;
    const int64_t B = std::atoll(argv[7]), T = cfg.sequence_len;
    const int steps = std::atoi(argv[8]), warmup = std::atoi(argv[9]);

    GPT model = GPT::init_random(cfg, 1234, DType::F32);
    std::vector<Tensor> params = model.parameters();
    int64_t n_params = 0;
    for (const Tensor& p : params) n_params += (int64_t)p.layout().size();

    std::mt19937_64 gen(99);
    std::uniform_int_distribution<int64_t> tok(0, cfg.vocab_size - 1);
    std::vector<int64_t> h_ids((size_t)(B * T)), h_tg((size_t)(B * T));
    for (auto& x : h_ids) x = tok(gen);
    for (auto& x : h_tg) x = tok(gen);
    Tensor ids = Tensor::from_host(h_ids.data(), {B, T}, DType::I64);
    Tensor targets = Tensor::from_host(h_tg.data(), {B * T}, DType::I64);

    AdamW opt = AdamWConfig(3e-4).betas(0.9, 0.95).weight_decay(0.1).build(params);
    float last_loss = 0.f, last_norm = 0.f;
    std::vector<float> losses, norms;  // every step of the run, in order (warm-up first)
    auto step = [&]() {
      Tensor loss = cross_entropy(model.forward(ids).reshape({B * T, cfg.vocab_size}), targets);
      GradientStore grads = loss.backward();
      double scale = 1.0;
      last_norm = clip_grad_scale(params, grads, 1.0, &scale);  // reads 4 bytes back: one sync per step
      opt.step_with_grads(grads, scale);
      loss.to_host(&last_loss);
      losses.push_back(last_loss);
      norms.push_back(last_norm);
    };
    for (int i = 0; i < warmup; ++i) step();
    const float first_loss = last_loss;
    check(deers_rocm_sync());
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < steps; ++i) step();
    check(deers_rocm_sync());
    const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count() / steps;

    // profiled pass: every launch bracketed by events
    check(deers_rocm_profile_enable(1));
    const int prof_steps = steps < 3 ? steps : 3;
    for (int i = 0; i < prof_steps; ++i) step();
    int rows = 0;
    check(deers_rocm_profile_collect(&rows));
    std::string kernels = "{";
    for (int r = 0; r < rows; ++r) {
      const char* name = nullptr;
      int64_t calls = 0;
      float total_ms = 0;
      check(deers_rocm_profile_row(r, &name, &calls, &total_ms));
      char buf[256];
      std::snprintf(buf, sizeof(buf), "%s\"%s\": {\"calls_per_step\": %.1f, \"ms_per_step\": %.4f}", r ? ", " : "",
                    name, (double)calls / prof_steps, total_ms / prof_steps);
      kernels += buf;
    }
    kernels += "}";
    check(deers_rocm_profile_enable(0));

    auto join = [](const std::vector<float>& v) {
      std::string out = "[";
      char buf[32];
      for (size_t i = 0; i < v.size(); ++i) {
        std::snprintf(buf, sizeof(buf), "%s%.5f", i ? ", " : "", v[i]);
        out += buf;
      }
      return out + "]";
    };
    std::printf(
        "{\"gemm_tuning\": %s, \"ms_per_step\": %.3f, \"tokens_per_s\": %.1f, \"parameters\": %lld, \"batch\": %lld, \"seq_len\": %lld, "
        "\"loss_first\": %.4f, \"loss_last\": %.4f, \"grad_norm\": %.4f, \"losses\": %s, \"grad_norms\": %s, \"kernels\": %s}\n",
        tune ? "true" : "false", ms, 1e3 * (double)(B * T) / ms, (long long)n_params, (long long)B, (long long)T, first_loss, last_loss,
        last_norm, join(losses).c_str(), join(norms).c_str(), kernels.c_str());
    return 0;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "gpt_step: %s\n", e.what());
    return 1;
  }
}
