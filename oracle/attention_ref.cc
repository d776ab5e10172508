// TEST INFRASTRUCTURE — NOT PRODUCT CODE.
//
// CPU restatement of the causal self-attention path of vitillo/deers, used only
// as the checker for the HIP kernels (tests, smoke, and the CPU-baseline leg of
// the benchmark).  Nothing in the shipped library links or calls this file.
//
// The reference computes attention as a chain of primitive tensor ops that each
// materialise a full [B,H,Tq,Tk] tensor (src/models/gpt.rs:139-144):
//
//   scores = q.matmul(k.transpose(2,3)) * scale
//   mask   = causal_mask(B, T, 0, ..)              [B,1,T,T], 0 / -inf
//   attn   = (scores + mask).softmax(3)            softmax = exp(x - lse(x))
//   y      = attn.matmul(v)
//
// and differentiates it op by op through its autograd engine
// (src/backprop.rs:52-66).  Every function below restates one of those ops in
// the same arithmetic order, and the two composite entry points chain them in
// the order the reference executes them.
//
// Parity status per function (what pins it is exercised in tests/test_oracle*.py):
//   oracle_causal_mask      pinned: literal vectors of tests/nn.rs:193-232
//   oracle_matmul           pinned to 1e-4 by exact integer products
//                           (tests/tensor.rs:83-291); the bit-level summation
//                           order of the third-party `gemm` crate 0.19.0 used at
//                           src/storage/cpu.rs:110-132 is NOT pinned ("parity
//                           unpinned" at the ulp level; irrelevant to the 1e-4 /
//                           5e-3 contract)
//   oracle_scalar_mul       pinned: closed form, src/storage.rs:105-123
//   oracle_log_sum_exp      pinned: closed form on the reference's literal input
//                           [1,2,3,1.5,0.5,-1] (tests/tensor.rs:1887)
//   oracle_attn_fwd         pinned: brute-force f64 definition, invariants, and a
//                           library routine (torch SDPA, is_causal=True)
//   oracle_attn_bwd         pinned: central finite differences in f64, invariants,
//                           torch autograd
//
// Template parameter R is the real type: float follows the reference's f32 path
// op for op (built with -ffp-contract=off, so a multiply and an add stay two roundings
// as in the element-wise Rust code; the GEMM inner loops of crate `gemm` may fuse them,
// which is the unpinned ulp-level order named above); double exists only so
// finite-difference tests have head-room.

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

// ---------------------------------------------------------------------------
// Batched strided GEMM.  Follows CpuStorage::matmul (src/storage/cpu.rs:688-753)
// and gemm_strided (src/storage/cpu.rs:93-133): one GEMM per batch element,
// batches visited sequentially, each GEMM parallel over all host threads
// (reference: gemm::Parallelism::Rayon(0), src/storage/cpu.rs:130), operand
// strides taken from the layouts, output compact row-major [batch, m, n].
// Each output element is a k-ordered sum starting from 0 (dst is not read:
// alpha(dst)=0, beta=1).
// ---------------------------------------------------------------------------
template <typename R>
void gemm_one(const R* a, int64_t a_rs, int64_t a_cs, const R* b, int64_t b_rs, int64_t b_cs,
              R* out, int64_t m, int64_t n, int64_t k, int nthreads) {
  // Pack the right operand to [k][n] so the inner loop is unit stride whatever
  // view (transposed or not) the caller passed.
  std::vector<R> packed;
  const R* bp = b;
  if (!(b_cs == 1 && b_rs == n)) {
    packed.resize(static_cast<size_t>(k) * n);
#pragma omp parallel for num_threads(nthreads) schedule(static) if (nthreads > 1)
    for (int64_t kk = 0; kk < k; ++kk)
      for (int64_t j = 0; j < n; ++j) packed[kk * n + j] = b[kk * b_rs + j * b_cs];
    bp = packed.data();
  }
#pragma omp parallel for num_threads(nthreads) schedule(static) if (nthreads > 1)
  for (int64_t i = 0; i < m; ++i) {
    R* row = out + i * n;
    for (int64_t j = 0; j < n; ++j) row[j] = R(0);
    for (int64_t kk = 0; kk < k; ++kk) {
      const R aik = a[i * a_rs + kk * a_cs];
      const R* brow = bp + kk * n;
      for (int64_t j = 0; j < n; ++j) row[j] += aik * brow[j];
    }
  }
}

template <typename R>
void matmul(const R* a, int64_t a_bs, int64_t a_rs, int64_t a_cs, const R* b, int64_t b_bs,
            int64_t b_rs, int64_t b_cs, R* out, int64_t batch, int64_t m, int64_t n, int64_t k,
            int nthreads) {
  for (int64_t i = 0; i < batch; ++i)
    gemm_one(a + i * a_bs, a_rs, a_cs, b + i * b_bs, b_rs, b_cs, out + i * m * n, m, n, k,
             nthreads);
}

// ScalarMul::forward -> unary_op(ScalarMul(s)): `v * self.0 as f32`
// (src/ops.rs:625-636, src/storage.rs:105-123).  The f64 scalar is narrowed to
// the element type first, then multiplied.
template <typename R>
void scalar_mul(const R* x, size_t n, double s, R* out) {
  const R sr = static_cast<R>(s);
  for (size_t i = 0; i < n; ++i) out[i] = x[i] * sr;
}

// causal_mask (src/nn/functional.rs:12-55): [batch,1,tgt,tgt+off]; -inf iff
// j >= off && j - off > i.
template <typename R>
void causal_mask(int64_t batch, int64_t tgt, int64_t off, R* out) {
  const int64_t total = tgt + off;
  for (int64_t b = 0; b < batch; ++b)
    for (int64_t i = 0; i < tgt; ++i)
      for (int64_t j = 0; j < total; ++j)
        out[(b * tgt + i) * total + j] =
            (j >= off && j - off > i) ? -std::numeric_limits<R>::infinity() : R(0);
}

// `&scores + &mask`: the mask [B,1,Tq,Tk] is broadcast over heads as a stride-0
// view (src/tensor.rs:499-510, src/ops.rs:749-775) and added element-wise into a
// fresh compact tensor (src/storage/cpu.rs:289-320, 982-1019).
template <typename R>
void add_mask(const R* scores, const R* mask, int64_t B, int64_t H, int64_t tq, int64_t tk,
              R* out) {
  const int64_t plane = tq * tk;
  for (int64_t b = 0; b < B; ++b)
    for (int64_t h = 0; h < H; ++h) {
      const R* s = scores + (b * H + h) * plane;
      const R* mk = mask + b * plane;
      R* o = out + (b * H + h) * plane;
      for (int64_t e = 0; e < plane; ++e) o[e] = s[e] + mk[e];
    }
}

// CpuStorage::log_sum_exp (src/storage/cpu.rs:755-771): per row, max by a left
// fold from -inf, then a left-to-right sum of exp(x - max), then ln(sum) + max.
template <typename R>
void log_sum_exp(const R* x, int64_t rows, int64_t cols, R* out) {
  for (int64_t r = 0; r < rows; ++r) {
    const R* s = x + r * cols;
    R mx = -std::numeric_limits<R>::infinity();
    for (int64_t j = 0; j < cols; ++j) mx = std::max(mx, s[j]);
    R sum = R(0);
    for (int64_t j = 0; j < cols; ++j) sum += std::exp(s[j] - mx);
    out[r] = std::log(sum) + mx;
  }
}

// log_softmax primitive path (src/tensor.rs:419-424): lse reshaped to [..,1],
// broadcast along the last axis, `self - &lse`.
template <typename R>
void sub_row(const R* x, const R* row_val, int64_t rows, int64_t cols, R* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int64_t j = 0; j < cols; ++j) out[r * cols + j] = x[r * cols + j] - row_val[r];
}

// EWiseExp::forward (src/ops.rs:409-420): libm-accurate exp, not a fast-math one.
template <typename R>
void ewise_exp(const R* x, size_t n, R* out) {
  for (size_t i = 0; i < n; ++i) out[i] = std::exp(x[i]);
}

// ---------------------------------------------------------------------------
// Forward composite: src/models/gpt.rs:139-144 with q [N,Tq,D], k,v [N,Tk,D]
// compact (N = B*H), seqlen_offset = Tk - Tq.  Decode is the same math with
// Tq = 1 (mask row all zero, tests/nn.rs:223-232).
// Optional outputs (may be null): lse [N,Tq] of the masked, scaled scores and
// attn [N,Tq,Tk].
// ---------------------------------------------------------------------------
template <typename R>
void attn_fwd(const R* q, const R* k, const R* v, int64_t B, int64_t H, int64_t tq, int64_t tk,
              int64_t D, double scale, R* y, R* lse_out, R* attn_out, int nthreads) {
  const int64_t N = B * H;
  const size_t plane = static_cast<size_t>(tq) * tk;
  std::vector<R> scores(N * plane), scaled(N * plane), mask(B * plane), x(N * plane),
      lse(static_cast<size_t>(N) * tq), lsm(N * plane), attn_local;
  // scores = q @ k^T : the transpose is a view, rs=1, cs=D (src/ops.rs:1067-1087)
  matmul<R>(q, tq * D, D, 1, k, tk * D, 1, D, scores.data(), N, tq, tk, D, nthreads);
  scalar_mul<R>(scores.data(), scores.size(), scale, scaled.data());
  causal_mask<R>(B, tq, tk - tq, mask.data());
  add_mask<R>(scaled.data(), mask.data(), B, H, tq, tk, x.data());
  // softmax(3) = log_softmax(3).exp() (src/tensor.rs:456-458)
  log_sum_exp<R>(x.data(), N * tq, tk, lse.data());
  sub_row<R>(x.data(), lse.data(), N * tq, tk, lsm.data());
  R* attn = attn_out;
  if (!attn) {
    attn_local.resize(N * plane);
    attn = attn_local.data();
  }
  ewise_exp<R>(lsm.data(), lsm.size(), attn);
  // y = attn @ v
  matmul<R>(attn, plane, tk, 1, v, tk * D, D, 1, y, N, tq, D, tk, nthreads);
  if (lse_out) std::memcpy(lse_out, lse.data(), lse.size() * sizeof(R));
}

// ---------------------------------------------------------------------------
// Backward composite: the reverse sweep of src/backprop.rs:52-66 over the graph
// built by attn_fwd, op by op:
//   MatMul(attn,v).backward      dAttn = dY @ v^T ; dV = attn^T @ dY   src/ops.rs:1089-1101
//   EWiseExp.backward            dLsm = dAttn * exp(lsm) (recomputed)  src/ops.rs:422-425
//   EWiseSub.backward            dX  = dLsm ; dLseB = -dLsm            src/ops.rs:210-214
//   Broadcast/Reshape.backward   dLse = sum over last axis of dLseB    src/ops.rs:777-799, 925-929
//   LogSumExp.backward           dX += exp(x - lse) * dLse             src/ops.rs:1162-1175
//   EWiseAdd.backward            dScaled = dX (mask needs no grad)     src/backprop.rs:34-39
//   ScalarMul.backward           dScores = dScaled * scale             src/ops.rs:638-643
//   MatMul(q,k^T).backward       dQ = dScores @ k ; dK^T = q^T @ dScores
// The forward intermediates are recomputed here exactly as attn_fwd does.
// ---------------------------------------------------------------------------
template <typename R>
void attn_bwd(const R* q, const R* k, const R* v, const R* dy, int64_t B, int64_t H, int64_t tq,
              int64_t tk, int64_t D, double scale, R* dq, R* dk, R* dv, int nthreads) {
  const int64_t N = B * H;
  const size_t plane = static_cast<size_t>(tq) * tk;
  const size_t tot = N * plane;
  std::vector<R> x(tot), lse(static_cast<size_t>(N) * tq), lsm(tot), attn(tot);
  {
    std::vector<R> scores(tot), scaled(tot), mask(B * plane);
    matmul<R>(q, tq * D, D, 1, k, tk * D, 1, D, scores.data(), N, tq, tk, D, nthreads);
    scalar_mul<R>(scores.data(), tot, scale, scaled.data());
    causal_mask<R>(B, tq, tk - tq, mask.data());
    add_mask<R>(scaled.data(), mask.data(), B, H, tq, tk, x.data());
    log_sum_exp<R>(x.data(), N * tq, tk, lse.data());
    sub_row<R>(x.data(), lse.data(), N * tq, tk, lsm.data());
    ewise_exp<R>(lsm.data(), tot, attn.data());
  }
  // dAttn = dY @ v^T   [N,Tq,Tk];  dV = attn^T @ dY   [N,Tk,D]
  std::vector<R> dattn(tot);
  matmul<R>(dy, tq * D, D, 1, v, tk * D, 1, D, dattn.data(), N, tq, tk, D, nthreads);
  matmul<R>(attn.data(), plane, 1, tk, dy, tq * D, D, 1, dv, N, tk, D, tq, nthreads);
  // dLsm = dAttn * exp(lsm): the reference calls `self.arg.exp()` again.
  std::vector<R> dlsm(tot);
  {
    std::vector<R> e(tot);
    ewise_exp<R>(lsm.data(), tot, e.data());
    for (size_t i = 0; i < tot; ++i) dlsm[i] = dattn[i] * e[i];
  }
  // dLse[r] = sum_j (-dLsm[r][j]), left-to-right as the CPU row reduce does.
  std::vector<R> dlse(static_cast<size_t>(N) * tq);
  for (int64_t r = 0; r < N * tq; ++r) {
    R s = R(0);
    for (int64_t j = 0; j < tk; ++j) s += -dlsm[r * tk + j];
    dlse[r] = s;
  }
  // dX = dLsm + exp(x - lse) * dLse   (GradientStore::accumulate: existing + grad)
  std::vector<R> dx(tot);
  {
    std::vector<R> t(tot), sm(tot);
    sub_row<R>(x.data(), lse.data(), N * tq, tk, t.data());
    ewise_exp<R>(t.data(), tot, sm.data());
    for (int64_t r = 0; r < N * tq; ++r)
      for (int64_t j = 0; j < tk; ++j) {
        const size_t i = r * tk + j;
        dx[i] = dlsm[i] + sm[i] * dlse[r];
      }
  }
  // dScores = dX * scale (`out_grad * self.scalar`, scalar narrowed as in forward)
  std::vector<R> ds(tot);
  scalar_mul<R>(dx.data(), tot, scale, ds.data());
  // dQ = dScores @ (k^T)^T = dScores @ k ; d(k^T) = q^T @ dScores, then the
  // Permute backward hands dK back as its transpose view: dK[j][d] = d(k^T)[d][j].
  matmul<R>(ds.data(), plane, tk, 1, k, tk * D, D, 1, dq, N, tq, D, tk, nthreads);
  std::vector<R> dkt(static_cast<size_t>(N) * D * tk);
  matmul<R>(q, tq * D, 1, D, ds.data(), plane, tk, 1, dkt.data(), N, D, tk, tq, nthreads);
  for (int64_t nidx = 0; nidx < N; ++nidx)
    for (int64_t j = 0; j < tk; ++j)
      for (int64_t d = 0; d < D; ++d)
        dk[(nidx * tk + j) * D + d] = dkt[(nidx * D + d) * tk + j];
}

int resolve_threads(int nthreads) {
  if (nthreads > 0) return nthreads;
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // namespace

extern "C" {

int oracle_max_threads(void) { return resolve_threads(0); }

#define ORACLE_INSTANTIATE(SUF, R)                                                               \
  void oracle_matmul_##SUF(const R* a, int64_t a_bs, int64_t a_rs, int64_t a_cs, const R* b,     \
                           int64_t b_bs, int64_t b_rs, int64_t b_cs, R* out, int64_t batch,      \
                           int64_t m, int64_t n, int64_t k, int nthreads) {                      \
    matmul<R>(a, a_bs, a_rs, a_cs, b, b_bs, b_rs, b_cs, out, batch, m, n, k,                     \
              resolve_threads(nthreads));                                                        \
  }                                                                                              \
  void oracle_scalar_mul_##SUF(const R* x, int64_t n, double s, R* out) {                        \
    scalar_mul<R>(x, static_cast<size_t>(n), s, out);                                            \
  }                                                                                              \
  void oracle_causal_mask_##SUF(int64_t batch, int64_t tgt, int64_t off, R* out) {               \
    causal_mask<R>(batch, tgt, off, out);                                                        \
  }                                                                                              \
  void oracle_log_sum_exp_##SUF(const R* x, int64_t rows, int64_t cols, R* out) {                \
    log_sum_exp<R>(x, rows, cols, out);                                                          \
  }                                                                                              \
  void oracle_softmax_##SUF(const R* x, int64_t rows, int64_t cols, R* out) {                    \
    std::vector<R> lse(rows), lsm(static_cast<size_t>(rows) * cols);                             \
    log_sum_exp<R>(x, rows, cols, lse.data());                                                   \
    sub_row<R>(x, lse.data(), rows, cols, lsm.data());                                           \
    ewise_exp<R>(lsm.data(), lsm.size(), out);                                                   \
  }                                                                                              \
  void oracle_attn_fwd_##SUF(const R* q, const R* k, const R* v, int64_t B, int64_t H,           \
                             int64_t tq, int64_t tk, int64_t D, double scale, R* y, R* lse,      \
                             R* attn, int nthreads) {                                            \
    attn_fwd<R>(q, k, v, B, H, tq, tk, D, scale, y, lse, attn, resolve_threads(nthreads));       \
  }                                                                                              \
  void oracle_attn_bwd_##SUF(const R* q, const R* k, const R* v, const R* dy, int64_t B,         \
                             int64_t H, int64_t tq, int64_t tk, int64_t D, double scale, R* dq,  \
                             R* dk, R* dv, int nthreads) {                                       \
    attn_bwd<R>(q, k, v, dy, B, H, tq, tk, D, scale, dq, dk, dv, resolve_threads(nthreads));     \
  }

ORACLE_INSTANTIATE(f32, float)
ORACLE_INSTANTIATE(f64, double)

}  // extern "C"
