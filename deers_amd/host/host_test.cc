// Test driver of the C++ host side.
//   host_test graph            graph / layout logic on unbacked tensors (no GPU)
//   host_test gpu <dir>        runs the fused op on the inputs in <dir> (written by
//                              the Python tests) and writes its outputs there
//   host_test module <dir>     the whole attention module (projections, RoPE, core,
//                              head merge, output projection), forward and backward
// The graph cases restate the reference's own autograd tests
// (src/backprop.rs:142-201): linear chain, diamond, no-grad skip, accumulation = 2.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <string>
#include <vector>

#include "../../include/deers_rocm.h"
#include "ops.h"
#include "gpt.h"
#include "optim.h"

using namespace deers_host;

static int g_failed = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) {                                                          \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);           \
      ++g_failed;                                                           \
    }                                                                       \
  } while (0)

static void test_layout() {
  Layout l({2, 3, 4, 5});
  EXPECT(l.is_compact());
  EXPECT((l.strides == std::vector<int64_t>{60, 20, 5, 1}));
  Layout p = l.permute({0, 2, 1, 3});
  EXPECT((p.shape == std::vector<int64_t>{2, 4, 3, 5}));
  EXPECT((p.strides == std::vector<int64_t>{60, 5, 20, 1}));
  EXPECT(!p.is_compact());
  EXPECT(p.permute({0, 2, 1, 3}).is_compact());
  EXPECT(l.transpose(2, 3).strides.back() == 5);
  EXPECT(l.size() == 120);
  bool threw = false;
  try { (void)l.permute({0, 1}); } catch (const std::logic_error&) { threw = true; }
  EXPECT(threw);
  std::printf("ok layout\n");
}

static void test_sorted_nodes_linear_chain() {
  Tensor a = Tensor::unbacked({2, 3}, DType::F32).attach();
  Tensor b = a.neg(), c = b.neg(), d = c.neg();
  auto sorted = d.sorted_nodes();
  EXPECT(sorted.size() == 4);
  if (sorted.size() == 4) {
    EXPECT(*sorted[0] == d);
    EXPECT(*sorted[1] == c);
    EXPECT(*sorted[2] == b);
    EXPECT(*sorted[3] == a);
  }
  std::printf("ok sorted_nodes_linear_chain\n");
}

static void test_sorted_nodes_diamond() {
  Tensor a = Tensor::unbacked({2}, DType::F32).attach();
  Tensor b = a.neg(), c = a.neg();
  Tensor d = b.add(c);
  auto sorted = d.sorted_nodes();
  EXPECT(sorted.size() == 4);  // no duplicates
  if (sorted.size() == 4) {
    EXPECT(*sorted.front() == d);
    EXPECT(*sorted.back() == a);  // shared input last
  }
  std::printf("ok sorted_nodes_diamond\n");
}

static void test_sorted_nodes_skips_no_grad() {
  Tensor a = Tensor::unbacked({2}, DType::F32).attach();
  Tensor b = Tensor::unbacked({2}, DType::F32);  // no grad
  Tensor c = a.add(b);
  auto sorted = c.sorted_nodes();
  EXPECT(sorted.size() == 2);
  if (sorted.size() == 2) {
    EXPECT(*sorted[0] == c);
    EXPECT(*sorted[1] == a);
  }
  // nothing requires grad: the op is dropped and the sweep is empty
  Tensor e = b.neg();
  EXPECT(!e.requires_grad());
  EXPECT(e.op() == nullptr);
  EXPECT(e.sorted_nodes().empty());
  // NO_GRAD drops tracking even for attached inputs
  {
    NoGradGuard g;
    Tensor f = a.neg();
    EXPECT(!f.requires_grad());
    EXPECT(f.op() == nullptr);
  }
  EXPECT(a.neg().requires_grad());
  std::printf("ok sorted_nodes_skips_no_grad\n");
}

static void test_graph_of_attention_views() {
  // the shape of the sub-graph at src/models/gpt.rs:135-144: projections [B,T,H,D],
  // permuted to [B,H,T,D]; backward through Permute returns the gradient to the
  // [B,T,H,D] leaf as the inverse-permuted view
  Tensor x = Tensor::unbacked({2, 5, 3, 8}, DType::F16).attach();
  Tensor v = x.permute({0, 2, 1, 3});
  EXPECT((v.shape() == std::vector<int64_t>{2, 3, 5, 8}));
  EXPECT((v.layout().strides == std::vector<int64_t>{120, 8, 24, 1}));
  EXPECT(v.requires_grad());
  EXPECT(std::string(v.op()->name()) == "Permute");
  GradientStore grads = v.backward();
  const Tensor* gx = grads.get(x.id());
  EXPECT(gx != nullptr);
  if (gx) EXPECT(gx->shape() == x.shape());
  std::printf("ok graph_of_attention_views\n");
}

// ---- GPU cases ----

static std::vector<char> read_file(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) { std::printf("FAIL cannot read %s\n", path.c_str()); std::exit(2); }
  return std::vector<char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}
static void write_file(const std::string& path, const void* p, size_t n) {
  std::ofstream f(path, std::ios::binary);
  f.write(static_cast<const char*>(p), (std::streamsize)n);
}
static void dump(const Tensor& t, const std::string& path) {
  std::vector<char> host(t.layout().size() * size_in_bytes(t.dtype()));
  t.to_host(host.data());
  write_file(path, host.data(), host.size());
}

static void test_backward_accumulates_diamond_grads() {
  Tensor a = Tensor::ones({2}, DType::F32).attach();
  Tensor b = a.add(a);
  GradientStore grads = b.backward();  // seeded with ones, like sum().backward()
  const Tensor* ga = grads.get(a.id());
  EXPECT(ga != nullptr);
  if (ga) {
    float h[2] = {0, 0};
    ga->to_host(h);
    EXPECT(h[0] == 2.0f && h[1] == 2.0f);  // a is used twice
  }
  std::printf("ok backward_accumulates_diamond_grads\n");
}

// matmul_add(a, b, c) against a.matmul(b).add(c): values and all three gradients; a is used by
// two products, so its second gradient rides on a product as well (accumulate of a MatMul's
// gradient onto one the store already holds, src/backprop.rs:101-112).
static void test_matmul_add_matches_matmul_then_add() {
  const int64_t M = 6, K = 8, N = 5;
  std::vector<float> ha(M * K), hb(K * N), hc(M * N), hb2(K * N);
  for (size_t i = 0; i < ha.size(); ++i) ha[i] = 0.25f * (float)((int)(i * 7 % 11) - 5);
  for (size_t i = 0; i < hb.size(); ++i) hb[i] = 0.5f * (float)((int)(i * 5 % 7) - 3);
  for (size_t i = 0; i < hb2.size(); ++i) hb2[i] = 0.125f * (float)((int)(i * 3 % 13) - 6);
  for (size_t i = 0; i < hc.size(); ++i) hc[i] = (float)((int)(i % 9) - 4);
  std::vector<std::vector<float>> got[2];
  for (int fused = 0; fused < 2; ++fused) {
    Tensor a = Tensor::from_host(ha.data(), {M, K}, DType::F32).attach();
    Tensor b = Tensor::from_host(hb.data(), {K, N}, DType::F32).attach();
    Tensor b2 = Tensor::from_host(hb2.data(), {K, N}, DType::F32).attach();
    Tensor c = Tensor::from_host(hc.data(), {M, N}, DType::F32).attach();
    const Tensor y = fused ? matmul_add(a, b, c) : a.matmul(b).add(c);
    const Tensor z = y.add(a.matmul(b2));  // a second product through a
    GradientStore grads = z.backward();
    std::vector<float> hy(M * N);
    y.to_host(hy.data());
    got[fused].push_back(hy);
    for (const Tensor* t : {&a, &b, &b2, &c}) {
      const Tensor* g = grads.get(t->id());
      EXPECT(g != nullptr && g->shape() == t->shape());
      std::vector<float> hg(t->layout().size(), -1.f);
      if (g) g->to_host(hg.data());
      got[fused].push_back(hg);
    }
  }
  for (size_t k = 0; k < got[0].size(); ++k)
    for (size_t i = 0; i < got[0][k].size(); ++i) EXPECT(got[0][k][i] == got[1][k][i]);  // small integers over 8: exact
  std::printf("ok matmul_add_matches_matmul_then_add\n");
}

static int run_gpu(const std::string& dir) {
  check(deers_rocm_init(0));
  test_backward_accumulates_diamond_grads();
  test_matmul_add_matches_matmul_then_add();

  // case.txt: dtype B H T D L   (dtype 0 = f16, 1 = f32; L = decode cache length or 0)
  int dt, B, H, T, D, L;
  {
    std::ifstream f(dir + "/case.txt");
    if (!(f >> dt >> B >> H >> T >> D >> L)) { std::printf("FAIL bad case.txt\n"); return 2; }
  }
  const DType dtype = dt == 0 ? DType::F16 : DType::F32;
  const std::vector<int64_t> bthd{B, T, H, D};
  auto load = [&](const char* name, const std::vector<int64_t>& shape) {
    auto bytes = read_file(dir + "/" + name);
    Layout l(shape);
    if (bytes.size() != l.size() * size_in_bytes(dtype)) { std::printf("FAIL size of %s\n", name); std::exit(2); }
    return Tensor::from_host(bytes.data(), shape, dtype);
  };
  // Projections arrive as [B,T,H,D] and are permuted to [B,H,T,D] (gpt.rs:135-137).
  Tensor xq = load("q.bin", bthd).attach(), xk = load("k.bin", bthd).attach(), xv = load("v.bin", bthd).attach();
  Tensor seed = load("do.bin", bthd);  // d loss / d y in the [B,T,H,D] order y is reshaped from
  Tensor q = xq.permute({0, 2, 1, 3}), k = xk.permute({0, 2, 1, 3}), v = xv.permute({0, 2, 1, 3});
  Tensor y = causal_self_attention(q, k, v);           // [B,H,T,D] over [B,T,H,D] memory
  EXPECT(y.permute({0, 2, 1, 3}).is_compact());        // the head merge is a view
  EXPECT(std::string(y.op()->name()) == "FusedCausalAttention");
  Tensor y_bthd = y.permute({0, 2, 1, 3}).compact();   // what reshape does (ops.rs:913)
  dump(y_bthd, dir + "/y.bin");
  GradientStore grads = y_bthd.backward_from(seed);
  for (auto [t, name] : {std::pair<const Tensor*, const char*>{&xq, "dq.bin"}, {&xk, "dk.bin"}, {&xv, "dv.bin"}}) {
    const Tensor* g = grads.get(t->id());
    EXPECT(g != nullptr);
    if (g) {
      EXPECT(g->shape() == t->shape());
      dump(*g, dir + "/" + name);
    }
  }
  // the same inputs through two attention ops: every gradient doubles exactly
  {
    Tensor y2 = causal_self_attention(q, k, v).add(causal_self_attention(q, k, v));
    GradientStore g2 = y2.permute({0, 2, 1, 3}).compact().backward_from(seed);
    const Tensor* a = grads.get(xv.id());
    const Tensor* b2 = g2.get(xv.id());
    EXPECT(a && b2);
    if (a && b2) {
      const size_t n = a->layout().size();
      if (dtype == DType::F32) {
        std::vector<float> ha(n), hb(n);
        a->to_host(ha.data());
        b2->to_host(hb.data());
        size_t bad = 0;
        for (size_t i = 0; i < n; ++i) bad += (hb[i] != 2.0f * ha[i]);
        EXPECT(bad == 0);
      } else {
        dump(*b2, dir + "/dv_twice.bin");
      }
    }
  }
  // no-grad inputs: the op is dropped, nothing to sweep
  {
    Tensor yn = causal_self_attention(q.detach(), k.detach(), v.detach());
    EXPECT(!yn.requires_grad() && yn.op() == nullptr);
  }
  // the whole sub-graph of src/models/gpt.rs:135-147: RoPE on the q and k projections,
  // v as a permuted view, fused attention, head merge, reverse sweep
  {
    auto [cos, sin] = precompute_rotary_embeddings(T, D, 10000.0f, dtype);
    Tensor qr = rotary_heads(xq, cos, sin), kr = rotary_heads(xk, cos, sin);
    EXPECT(qr.is_compact() && (qr.shape() == std::vector<int64_t>{B, H, T, D}));
    EXPECT(std::string(qr.op()->name()) == "RotaryHeads");
    Tensor yr = causal_self_attention(qr, kr, v).permute({0, 2, 1, 3}).compact();
    dump(yr, dir + "/y_rope.bin");
    GradientStore gr = yr.backward_from(seed);
    for (auto [t, name] : {std::pair<const Tensor*, const char*>{&xq, "dq_rope.bin"}, {&xk, "dk_rope.bin"}, {&xv, "dv_rope.bin"}}) {
      const Tensor* g = gr.get(t->id());
      EXPECT(g != nullptr);
      if (g) {
        EXPECT(g->shape() == t->shape());
        dump(*g, dir + "/" + name);
      }
    }
  }
  if (L > 0) {
    Tensor dq = load("dec_q.bin", {B, H, D});
    Tensor kc = load("dec_k.bin", {B, H, L, D}), vc = load("dec_v.bin", {B, H, L, D});
    dump(attention_decode(dq, kc, vc), dir + "/dec_o.bin");
  }
  // backend failures surface as RocmError carrying the library's message
  {
    bool threw = false;
    try {
      // the fused kernels take head widths 32, 64, 128 only (the op routes other widths
      // through the unfused chain; the entry point itself refuses them)
      Tensor bad = Tensor::zeros({1, 1, 8, 48}, dtype);
      Tensor lse = Tensor::zeros({1, 1, 8}, DType::F32);
      check(deers_rocm_attn_fwd((int)dtype, bad.data(), nullptr, bad.data(), nullptr, bad.data(), nullptr,
                                bad.data(), nullptr, (float*)lse.data(), 1, 1, 8, 48, 0.125f));
    } catch (const RocmError& e) {
      threw = std::strlen(e.what()) > 0;
    }
    EXPECT(threw);
  }
  check(deers_rocm_sync());
  std::printf("ok gpu\n");
  return 0;
}

// The whole attention module (src/models/gpt.rs:101-147) forward and backward.
static int run_module(const std::string& dir) {
  check(deers_rocm_init(0));
  int dt, B, T, C, H;
  {
    std::ifstream f(dir + "/module.txt");  // dtype B T C H
    if (!(f >> dt >> B >> T >> C >> H)) { std::printf("FAIL bad module.txt\n"); return 2; }
  }
  const DType dtype = dt == 0 ? DType::F16 : DType::F32;
  auto load = [&](const char* name, const std::vector<int64_t>& shape) {
    auto bytes = read_file(dir + "/" + name);
    Layout l(shape);
    if (bytes.size() != l.size() * size_in_bytes(dtype)) { std::printf("FAIL size of %s\n", name); std::exit(2); }
    return Tensor::from_host(bytes.data(), shape, dtype);
  };
  Tensor x = load("x.bin", {B, T, C}).attach();
  Tensor wq = load("wq.bin", {C, C}).attach(), wk = load("wk.bin", {C, C}).attach();
  Tensor wv = load("wv.bin", {C, C}).attach(), wo = load("wo.bin", {C, C}).attach();
  Tensor seed = load("dy.bin", {B, T, C});
  CausalSelfAttention attn(C, H, wq, wk, wv, wo);
  auto [cos, sin] = precompute_rotary_embeddings(T, C / H, 10000.0f, dtype);
  Tensor y = attn.forward(x, cos, sin);
  EXPECT((y.shape() == std::vector<int64_t>{B, T, C}));
  dump(y, dir + "/y.bin");
  GradientStore grads = y.backward_from(seed);
  for (auto [t, name] : {std::pair<const Tensor*, const char*>{&x, "dx.bin"}, {&wq, "dwq.bin"}, {&wk, "dwk.bin"},
                         {&wv, "dwv.bin"}, {&wo, "dwo.bin"}}) {
    const Tensor* g = grads.get(t->id());
    EXPECT(g != nullptr);
    if (g) {
      EXPECT(g->shape() == t->shape());
      dump(*g, dir + "/" + name);
    }
  }
  // generation with a KV cache, teacher-forced with the same inputs: step t must give
  // row t of the full causal forward (f16 only: the decode kernel is f16)
  if (dtype == DType::F16 && (C / H == 64 || C / H == 128)) {
    std::vector<char> xh((size_t)B * T * C * 2), step((size_t)B * C * 2), ys((size_t)B * T * C * 2);
    x.to_host(xh.data());
    KvCache cache = KvCache::create(B, H, T + 7, C / H, dtype);  // spare capacity on purpose
    for (int t = 0; t < T; ++t) {
      for (int b = 0; b < B; ++b)
        std::memcpy(&step[(size_t)b * C * 2], &xh[((size_t)b * T + t) * C * 2], (size_t)C * 2);
      Tensor xt = Tensor::from_host(step.data(), {B, 1, C}, dtype);
      Tensor yt = attn.decode_step(xt, cache, cos, sin);
      EXPECT(!yt.requires_grad());
      yt.to_host(step.data());
      for (int b = 0; b < B; ++b)
        std::memcpy(&ys[((size_t)b * T + t) * C * 2], &step[(size_t)b * C * 2], (size_t)C * 2);
    }
    EXPECT(cache.len == T);
    write_file(dir + "/y_decode.bin", ys.data(), ys.size());
  }
  // op names along the graph, output first: the fused ops are really in it
  bool saw_attn = false, saw_rope = false, saw_matmul = false;
  for (const Tensor* n : y.sorted_nodes())
    if (n->op()) {
      const std::string nm = n->op()->name();
      saw_attn |= nm == "FusedCausalAttention";
      saw_rope |= nm == "RotaryHeads";
      saw_matmul |= nm == "MatMul";
    }
  EXPECT(saw_attn && saw_rope && saw_matmul);
  check(deers_rocm_sync());
  std::printf("ok module\n");
  return 0;
}

// Log-softmax through the graph: x [outer, inner] -> log_softmax(1), swept backward from
// a given output gradient, and the reference's own case (loss = sum, tests/tensor.rs:323-351).
static int run_log_softmax(const std::string& dir) {
  check(deers_rocm_init(0));
  int dt, outer, inner;
  {
    std::ifstream f(dir + "/case.txt");
    if (!(f >> dt >> outer >> inner)) { std::printf("FAIL bad case.txt\n"); return 2; }
  }
  const DType dtype = dt == 0 ? DType::F16 : DType::F32;
  const std::vector<int64_t> shape{outer, inner};
  auto load = [&](const char* name) {
    auto bytes = read_file(dir + "/" + name);
    if (bytes.size() != (size_t)outer * inner * size_in_bytes(dtype)) { std::printf("FAIL size of %s\n", name); std::exit(2); }
    return Tensor::from_host(bytes.data(), shape, dtype);
  };
  Tensor x = load("x.bin").attach();
  Tensor seed = load("g.bin");
  Tensor y = x.log_softmax(1);
  EXPECT(y.requires_grad() && std::string(y.op()->name()) == "FusedLogSoftmax");
  dump(y, dir + "/y.bin");
  GradientStore grads = y.backward_from(seed);
  const Tensor* gx = grads.get(x.id());
  EXPECT(gx != nullptr);
  if (gx) dump(*gx, dir + "/dx.bin");
  // a transposed (non-compact) view is compacted first, as the op does in the reference
  Tensor xt = load("x.bin").attach();
  Tensor yt = xt.transpose().log_softmax(1);  // [inner, outer], rows = columns of x
  EXPECT(yt.is_compact());
  dump(yt, dir + "/yt.bin");
  GradientStore gt = yt.backward();  // loss = sum(log_softmax)
  const Tensor* gxt = gt.get(xt.id());
  EXPECT(gxt != nullptr);
  if (gxt) {
    EXPECT(gxt->shape() == xt.shape());
    dump(*gxt, dir + "/dxt.bin");
  }
  bool threw = false;
  try { x.log_softmax(0); } catch (const std::logic_error&) { threw = true; }
  EXPECT(threw);
  {
    NoGradGuard guard;
    Tensor yn = x.log_softmax(1);
    EXPECT(!yn.requires_grad() && yn.op() == nullptr);
  }
  std::printf("ok log_softmax\n");
  return 0;
}

// K optimizer steps on two parameters with injected gradients, clipped to max_norm:
// odd steps through clip_grad_norm (rescaled copies in the store), even steps through
// clip_grad_scale folded into the step.  Writes the norms and the final w, m, v.
static int run_optim(const std::string& dir) {
  check(deers_rocm_init(0));
  int dt, n0, n1, steps;
  double lr, wd, max_norm;
  {
    std::ifstream f(dir + "/case.txt");
    if (!(f >> dt >> n0 >> n1 >> steps >> lr >> wd >> max_norm)) { std::printf("FAIL bad case.txt\n"); return 2; }
  }
  const DType dtype = dt == 0 ? DType::F16 : DType::F32;
  auto load = [&](const std::string& name, int64_t n) {
    auto bytes = read_file(dir + "/" + name);
    if (bytes.size() != (size_t)n * size_in_bytes(dtype)) { std::printf("FAIL size of %s\n", name.c_str()); std::exit(2); }
    return Tensor::from_host(bytes.data(), {n}, dtype);
  };
  Tensor p0 = load("w0.bin", n0).attach(), p1 = load("w1.bin", n1).attach();
  Tensor frozen = load("w1.bin", n1).attach();  // a parameter that never gets a gradient
  const TensorId id0 = p0.id();
  AdamW opt = AdamWConfig(lr).betas(0.9, 0.95).weight_decay(wd).build({p0, p1, frozen});
  EXPECT(opt.step_count() == 0 && !opt.state_for(p0).has_value());
  std::vector<float> norms;
  for (int t = 1; t <= steps; ++t) {
    GradientStore grads;
    Tensor g0 = load("g0_" + std::to_string(t) + ".bin", n0);
    grads.insert(p0.id(), g0);
    grads.insert(p1.id(), load("g1_" + std::to_string(t) + ".bin", n1));
    if (t % 2) {
      norms.push_back(clip_grad_norm({p0, p1, frozen}, grads, max_norm));
      EXPECT(norms.back() <= (float)max_norm || !(*grads.get(p0.id()) == g0));  // clipped => replaced
      opt.step_with_grads(grads);
    } else {
      double scale = 1.0;
      norms.push_back(clip_grad_scale({p0, p1, frozen}, grads, max_norm, &scale));
      EXPECT(*grads.get(p0.id()) == g0);  // untouched
      opt.step_with_grads(grads, scale);
    }
  }
  EXPECT(opt.step_count() == (size_t)steps);
  EXPECT(p0.id() == id0 && p0.requires_grad());
  EXPECT(!opt.state_for(frozen).has_value());
  write_file(dir + "/norms.bin", norms.data(), norms.size() * sizeof(float));
  dump(p0, dir + "/w0_out.bin");
  dump(p1, dir + "/w1_out.bin");
  auto st = opt.state_for(p0);
  EXPECT(st.has_value());
  if (st) {
    dump(st->first, dir + "/m0_out.bin");
    dump(st->second, dir + "/v0_out.bin");
  }
  // moments can be loaded back (checkpoint resume, src/optim.rs:156-160)
  if (st) {
    AdamW resumed = AdamWConfig(lr).build({p0});
    resumed.load_state_for(p0, st->first, st->second);
    resumed.set_step_count(opt.step_count());
    EXPECT(resumed.state_for(p0).has_value() && resumed.step_count() == (size_t)steps);
  }
  bool threw = false;
  try { GradientStore g; clip_grad_norm({p0}, g, 0.0); } catch (const std::logic_error&) { threw = true; }
  EXPECT(threw);
  {
    GradientStore g;
    EXPECT(clip_grad_norm({}, g, 1.0) == 0.0f);
  }
  std::printf("ok optim\n");
  return 0;
}

// The whole model: GPT forward, cross-entropy, reverse sweep, then `steps` training steps
// (clip_grad_scale folded into AdamW), the way examples/tinystories_train.rs drives the
// reference.  Writes logits, loss, every parameter's gradient, the per-step losses and
// norms, and the final parameters.
static int run_gpt(const std::string& dir) {
  check(deers_rocm_init(0));
  GPTConfig cfg;
  int64_t B, T;
  int steps;
  double lr, wd, max_norm;
  {
    std::ifstream f(dir + "/case.txt");
    if (!(f >> cfg.vocab_size >> cfg.sequence_len >> cfg.n_layer >> cfg.n_head >> cfg.n_embd >>
          cfg.mlp_hidden_dim >> cfg.rms_norm_eps >> cfg.rope_base >> B >> T >> steps >> lr >> wd >> max_norm)) {
      std::printf("FAIL bad case.txt\n");
      return 2;
    }
  }
  const int64_t C = cfg.n_embd, Hd = cfg.mlp_hidden_dim, V = cfg.vocab_size;
  std::vector<std::vector<int64_t>> shapes{{V, C}};
  for (int64_t l = 0; l < cfg.n_layer; ++l)
    for (auto s : std::vector<std::vector<int64_t>>{{C, C}, {C, C}, {C, C}, {C, C}, {C, Hd}, {Hd, C}}) shapes.push_back(s);
  shapes.push_back({C, V});
  std::vector<Tensor> weights;
  for (size_t i = 0; i < shapes.size(); ++i) {
    auto bytes = read_file(dir + "/w" + std::to_string(i) + ".bin");
    if (bytes.size() != (size_t)(shapes[i][0] * shapes[i][1]) * 4) { std::printf("FAIL size of w%zu\n", i); return 2; }
    weights.push_back(Tensor::from_host(bytes.data(), shapes[i], DType::F32));
  }
  auto ids_b = read_file(dir + "/ids.bin"), tg_b = read_file(dir + "/targets.bin");
  if (ids_b.size() != (size_t)(B * T) * 8 || tg_b.size() != (size_t)(B * T) * 8) { std::printf("FAIL ids/targets size\n"); return 2; }
  Tensor ids = Tensor::from_host(ids_b.data(), {B, T}, DType::I64);
  Tensor targets = Tensor::from_host(tg_b.data(), {B * T}, DType::I64);

  GPT model(cfg, weights);
  std::vector<Tensor> params = model.parameters();
  EXPECT(params.size() == shapes.size());
  for (const Tensor& p : params) EXPECT(p.requires_grad() && p.op() == nullptr);

  Tensor logits = model.forward(ids);
  EXPECT((logits.shape() == std::vector<int64_t>{B, T, V}));
  dump(logits, dir + "/logits.bin");
  Tensor loss = cross_entropy(logits.reshape({B * T, V}), targets);
  EXPECT(loss.requires_grad() && std::string(loss.op()->name()) == "CrossEntropy");
  dump(loss, dir + "/loss.bin");
  {
    GradientStore grads = loss.backward();
    for (size_t i = 0; i < params.size(); ++i) {
      const Tensor* g = grads.get(params[i].id());
      EXPECT(g != nullptr);
      if (g) {
        EXPECT(g->shape() == params[i].shape());
        dump(*g, dir + "/g" + std::to_string(i) + ".bin");
      }
    }
  }
  // inference under NoGradGuard builds no graph
  {
    NoGradGuard guard;
    Tensor l2 = model.forward(ids);
    EXPECT(!l2.requires_grad() && l2.op() == nullptr);
  }
  AdamW opt = AdamWConfig(lr).betas(0.9, 0.95).weight_decay(wd).build(params);
  std::vector<float> losses, norms;
  for (int t = 0; t < steps; ++t) {
    Tensor l = cross_entropy(model.forward(ids).reshape({B * T, V}), targets);
    float lv = 0;
    l.to_host(&lv);
    losses.push_back(lv);
    GradientStore grads = l.backward();
    double scale = 1.0;
    norms.push_back(clip_grad_scale(params, grads, max_norm, &scale));
    opt.step_with_grads(grads, scale);
  }
  write_file(dir + "/losses.bin", losses.data(), losses.size() * sizeof(float));
  write_file(dir + "/norms.bin", norms.data(), norms.size() * sizeof(float));
  for (size_t i = 0; i < params.size(); ++i) dump(params[i], dir + "/w" + std::to_string(i) + "_out.bin");
  // a token id outside the vocabulary is reported, not followed
  {
    std::vector<int64_t> bad((size_t)(B * T), 0);
    bad[0] = V;
    Tensor bad_ids = Tensor::from_host(bad.data(), {B, T}, DType::I64);
    bool threw = false;
    try {
      NoGradGuard guard;
      Tensor l = model.forward(bad_ids);
      check(deers_rocm_sync());  // the next synchronising call reports it
    } catch (const RocmError&) { threw = true; }
    EXPECT(threw);
  }
  std::printf("ok gpt\n");
  return 0;
}

// Generation with per-block KV caches on an f16 model: the logits of every decode step
// next to the full causal forward over the same tokens, and a greedy continuation.
static int run_generate(const std::string& dir) {
  check(deers_rocm_init(0));
  GPTConfig cfg;
  int64_t B, T, n_new;
  {
    std::ifstream f(dir + "/case.txt");
    if (!(f >> cfg.vocab_size >> cfg.sequence_len >> cfg.n_layer >> cfg.n_head >> cfg.n_embd >>
          cfg.mlp_hidden_dim >> cfg.rms_norm_eps >> cfg.rope_base >> B >> T >> n_new)) {
      std::printf("FAIL bad case.txt\n");
      return 2;
    }
  }
  const int64_t C = cfg.n_embd, Hd = cfg.mlp_hidden_dim, V = cfg.vocab_size;
  std::vector<std::vector<int64_t>> shapes{{V, C}};
  for (int64_t l = 0; l < cfg.n_layer; ++l)
    for (auto s : std::vector<std::vector<int64_t>>{{C, C}, {C, C}, {C, C}, {C, C}, {C, Hd}, {Hd, C}}) shapes.push_back(s);
  shapes.push_back({C, V});
  std::vector<Tensor> weights;
  for (size_t i = 0; i < shapes.size(); ++i) {
    auto bytes = read_file(dir + "/w" + std::to_string(i) + ".bin");
    if (bytes.size() != (size_t)(shapes[i][0] * shapes[i][1]) * 2) { std::printf("FAIL size of w%zu\n", i); return 2; }
    weights.push_back(Tensor::from_host(bytes.data(), shapes[i], DType::F16));
  }
  auto ids_b = read_file(dir + "/ids.bin");
  if (ids_b.size() != (size_t)(B * T) * 8) { std::printf("FAIL ids size\n"); return 2; }
  const int64_t* h_ids = (const int64_t*)ids_b.data();
  GPT model(cfg, weights);
  // full forward for comparison
  {
    NoGradGuard guard;
    Tensor logits = model.forward(Tensor::from_host(ids_b.data(), {B, T}, DType::I64));
    dump(logits, dir + "/logits_full.bin");
  }
  // the same tokens one position at a time through the caches
  std::vector<KvCache> caches = model.new_caches(B, T);
  std::vector<char> all((size_t)(B * T * V) * 2);
  std::vector<char> one((size_t)(B * V) * 2);
  std::vector<int64_t> cur((size_t)B);
  for (int64_t t = 0; t < T; ++t) {
    for (int64_t b = 0; b < B; ++b) cur[b] = h_ids[b * T + t];
    Tensor l = model.decode_step(Tensor::from_host(cur.data(), {B, 1}, DType::I64), caches);
    EXPECT((l.shape() == std::vector<int64_t>{B, 1, V}) && !l.requires_grad());
    l.to_host(one.data());
    for (int64_t b = 0; b < B; ++b)
      std::memcpy(all.data() + ((b * T + t) * V) * 2, one.data() + (b * V) * 2, (size_t)V * 2);
  }
  EXPECT(caches[0].len == T);
  write_file(dir + "/logits_steps.bin", all.data(), all.size());
  bool threw = false;
  try { model.decode_step(Tensor::from_host(cur.data(), {B, 1}, DType::I64), caches); } catch (const std::logic_error&) { threw = true; }
  EXPECT(threw);  // the caches are full
  const int64_t t0 = T / 2;
  std::vector<int64_t> prompt((size_t)(B * t0));
  for (int64_t b = 0; b < B; ++b)
    for (int64_t t = 0; t < t0; ++t) prompt[b * t0 + t] = h_ids[b * T + t];
  // the first T0 = T/2 tokens in one prefill pass, the others step by step from there
  {
    std::vector<KvCache> c2 = model.new_caches(B, T);
    Tensor lp = model.prefill(Tensor::from_host(prompt.data(), {B, t0}, DType::I64), c2);
    EXPECT((lp.shape() == std::vector<int64_t>{B, 1, V}) && !lp.requires_grad());
    for (const KvCache& c : c2) EXPECT(c.len == t0);
    dump(lp, dir + "/logits_prefill.bin");
    dump(c2.back().k, dir + "/k_cache_prefill.bin");
    dump(c2.back().v, dir + "/v_cache_prefill.bin");
    dump(caches.back().k, dir + "/k_cache_steps.bin");
    dump(caches.back().v, dir + "/v_cache_steps.bin");
    std::vector<char> rest((size_t)(B * (T - t0) * V) * 2);
    for (int64_t t = t0; t < T; ++t) {
      for (int64_t b = 0; b < B; ++b) cur[b] = h_ids[b * T + t];
      Tensor l = model.decode_step(Tensor::from_host(cur.data(), {B, 1}, DType::I64), c2);
      l.to_host(one.data());
      for (int64_t b = 0; b < B; ++b)
        std::memcpy(rest.data() + ((b * (T - t0) + (t - t0)) * V) * 2, one.data() + (b * V) * 2, (size_t)V * 2);
    }
    write_file(dir + "/logits_after_prefill.bin", rest.data(), rest.size());
    threw = false;
    try { model.prefill(Tensor::from_host(prompt.data(), {B, t0}, DType::I64), c2); } catch (const std::logic_error&) { threw = true; }
    EXPECT(threw);  // prefill wants empty caches
  }
  // greedy continuation of the same prompt
  std::vector<int64_t> gen = model.generate_greedy(prompt, B, n_new);
  EXPECT((int64_t)gen.size() == B * (t0 + n_new));
  write_file(dir + "/generated.bin", gen.data(), gen.size() * 8);
  // teacher-forced full forward over what was generated: its argmax must be the next token
  {
    NoGradGuard guard;
    Tensor l = model.forward(Tensor::from_host(gen.data(), {B, t0 + n_new}, DType::I64));
    dump(l, dir + "/logits_generated.bin");
  }
  std::printf("ok generate\n");
  return 0;
}

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "graph";
  try {
    if (mode == "graph") {
      test_layout();
      test_sorted_nodes_linear_chain();
      test_sorted_nodes_diamond();
      test_sorted_nodes_skips_no_grad();
      test_graph_of_attention_views();
    } else if (mode == "gpu" && argc > 2) {
      if (int rc = run_gpu(argv[2])) return rc;
    } else if (mode == "lsm" && argc > 2) {
      if (int rc = run_log_softmax(argv[2])) return rc;
    } else if (mode == "optim" && argc > 2) {
      if (int rc = run_optim(argv[2])) return rc;
    } else if (mode == "gpt" && argc > 2) {
      if (int rc = run_gpt(argv[2])) return rc;
    } else if (mode == "generate" && argc > 2) {
      if (int rc = run_generate(argv[2])) return rc;
    } else if (mode == "module" && argc > 2) {
      if (int rc = run_module(argv[2])) return rc;
    } else {
      std::printf("usage: host_test graph | gpu <dir> | lsm <dir> | optim <dir> | gpt <dir> | generate <dir> | module <dir>\n");
      return 2;
    }
  } catch (const std::exception& e) {
    std::printf("FAIL exception: %s\n", e.what());
    return 1;
  }
  std::printf(g_failed ? "FAILED %d checks\n" : "all passed\n", g_failed);
  return g_failed ? 1 : 0;
}
