// The remaining device ops of a GPT training step around the attention module
// (src/models/gpt.rs:170-355, src/nn.rs:203-251, src/loss.rs:11-24):
//
//   index_select / index_add   token embedding and its gradient
//                              (src/storage/cpu.rs:555-660, 936-975)
//   rms_norm fwd / bwd         x * (mean(x^2) + eps)^-0.5   (src/nn.rs:244-251, weightless)
//   relu_sq fwd / bwd          relu(x)^2, the MLP activation (src/models/gpt.rs:196-197)
//   cross_entropy fwd / bwd    -mean_i log_softmax(logits)_i[target_i]  (src/loss.rs:11-24)
//
// The reference composes the last three from primitive tensor ops (4, 3 and 5 kernels
// with as many intermediate tensors); here each is one pass forward and one backward.
// All are HBM-bound.  Arithmetic is f32 whatever the storage type, rounded once.
#include "common.h"

namespace deers {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <typename T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T* p) {
  return __builtin_bit_cast(Vec16<T>, *reinterpret_cast<const u32x4*>(p));
}
template <typename T>
__device__ __forceinline__ Vec16<T> load16_stream(const T* p) {
  return __builtin_bit_cast(Vec16<T>, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
template <typename T>
__device__ __forceinline__ void store16(const Vec16<T>& x, T* p) {
  *reinterpret_cast<u32x4*>(p) = __builtin_bit_cast(u32x4, x);
}
template <typename T>
__device__ __forceinline__ void store16_stream(const Vec16<T>& x, T* p) {
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4, x), reinterpret_cast<u32x4*>(p));
}

__device__ __forceinline__ float wave_sum(float s) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
  return s;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// ---- index_select (dim 0): out[i, :] = table[idx[i], :] ----
// One wavefront per output row.  An index outside [0, n_rows) writes a row of zeros and
// raises the sticky device error flag that the next synchronising call reports.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void index_select_kernel(const T* table, const int64_t* idx, T* out,
                                                           int64_t n_rows, int64_t n_idx, int width,
                                                           int* error_flag) {
  constexpr int kEpc = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t i = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= n_idx) return;
  const int64_t r = idx[i];
  const bool ok = r >= 0 && r < n_rows;
  if (!ok && lane == 0) atomicOr(error_flag, 1);
  const T* src = table + (ok ? r : 0) * width;
  T* dst = out + i * width;
  if constexpr (VEC) {
    for (int c = lane; c < width / kEpc; c += 64) {
      Vec16<T> v = load16(src + c * kEpc);
      if (!ok) v = Vec16<T>{};
      store16_stream(v, dst + c * kEpc);
    }
  } else {
    for (int c = lane; c < width; c += 64) dst[c] = ok ? src[c] : (T)0.f;
  }
}

// ---- index_add (dim 0): dst[idx[i], :] += src[i, :], in ascending i ----
// The order of additions is the reference's (src/storage/cpu.rs:954-975), so the result
// is the same bits and the same from run to run: workgroup i owns the destination row
// idx[i] if no earlier position names it, finds every later position that does (a
// bitmap in LDS, built from the index vector, which stays in L2), and adds their source
// rows in order.  Other workgroups leave at once.  A launch covers at most
// kIndexAddChunk positions (every workgroup scans its launch's whole index slice, so the
// cost of a launch grows with the square of its length); longer index vectors take one
// launch per slice, in order, which keeps the order of additions: a later slice adds to
// what the earlier ones left.
constexpr int kIndexAddChunk = 1 << 14;  // bitmap of 2 KB of dynamic LDS

template <typename T>
__global__ __launch_bounds__(256) void index_add_kernel(const T* src, const int64_t* idx, T* dst,
                                                        int64_t n_rows, int n_idx, int width,
                                                        int* error_flag) {
  extern __shared__ unsigned int bitmap[];  // one bit per position, 2 words per 64 positions
  __shared__ int not_leader;
  const int i = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t r = idx[i];
  if (r < 0 || r >= n_rows) {
    if (tid == 0) atomicOr(error_flag, 1);
    return;
  }
  if (tid == 0) not_leader = 0;
  __syncthreads();
  // each wavefront compares 64 consecutive positions per step (one coalesced load)
  const int groups = (n_idx + 63) / 64;
  for (int gq = wave; gq < groups; gq += 4) {
    const int pos = gq * 64 + lane;
    const bool match = pos < n_idx && idx[pos] == r;
    const unsigned long long mask = __ballot(match);
    if (lane == 0) {
      bitmap[2 * gq] = (unsigned int)mask;
      bitmap[2 * gq + 1] = (unsigned int)(mask >> 32);
      const int base = gq * 64;
      if (base < i) {
        const unsigned long long before =
            base + 64 <= i ? mask : mask & ((1ull << (i - base)) - 1ull);
        if (before) not_leader = 1;  // benign race: every writer stores 1
      }
    }
  }
  __syncthreads();
  if (not_leader) return;
  const int words = 2 * groups;
  T* out = dst + r * width;
  for (int c = tid; c < width; c += 256) {
    float acc = (float)out[c];
    for (int w = i / 32; w < words; ++w) {
      unsigned int bits = bitmap[w];
      while (bits) {
        const int b = __builtin_ctz(bits);
        bits &= bits - 1;
        // rounding to T after each addition, as `+=` on the storage type does
        acc = (float)(T)(acc + (float)src[(int64_t)(w * 32 + b) * width + c]);
      }
    }
    out[c] = (T)acc;
  }
}

// ---- rms_norm: y = x * (mean(x^2) + eps)^-0.5 over the last axis ----
// One wavefront per row (rows of a transformer are 192 .. 8192 wide, a few KB): the
// second sweep over the row is served by L1/L2, so x crosses HBM once.

template <typename T, bool VEC>
__device__ __forceinline__ float row_sum_prod(const T* a, const T* b, int width, int lane) {
  constexpr int kEpc = 16 / sizeof(T);
  float s = 0.f;
  if constexpr (VEC) {
    for (int c = lane; c < width / kEpc; c += 64) {
      const Vec16<T> va = load16(a + c * kEpc), vb = load16(b + c * kEpc);
#pragma unroll
      for (int e = 0; e < kEpc; ++e) s = fmaf((float)va.e[e], (float)vb.e[e], s);
    }
  } else {
    for (int c = lane; c < width; c += 64) s = fmaf((float)a[c], (float)b[c], s);
  }
  return wave_sum(s);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rms_norm_fwd_kernel(const T* x, T* y, int64_t outer, int width,
                                                           float eps) {
  constexpr int kEpc = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= outer) return;
  const T* row = x + r * width;
  T* orow = y + r * width;
  const float inv = 1.0f / sqrtf(row_sum_prod<T, VEC>(row, row, width, lane) / (float)width + eps);
  if constexpr (VEC) {
    for (int c = lane; c < width / kEpc; c += 64) {
      Vec16<T> v = load16(row + c * kEpc);
#pragma unroll
      for (int e = 0; e < kEpc; ++e) v.e[e] = (T)((float)v.e[e] * inv);
      store16(v, orow + c * kEpc);
    }
  } else {
    for (int c = lane; c < width; c += 64) orow[c] = (T)((float)row[c] * inv);
  }
}

// The forward for rows of at most 64 * RES 16-byte chunks (aligned): the row stays in the
// wave's registers between the sum of squares and the scaling.  Same bits as the general kernel.
template <typename T, int RES>
__global__ __launch_bounds__(256) void rms_norm_fwd_resident_kernel(const T* x, T* y, int64_t outer, int width,
                                                                    float eps) {
  constexpr int kEpc = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= outer) return;
  const T* row = x + r * width;
  T* orow = y + r * width;
  const int n_chunks = width / kEpc;
  Vec16<T> v[RES];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < RES; ++i) {
    const int c = lane + 64 * i;
    if (c < n_chunks) {
      v[i] = load16(row + c * kEpc);
#pragma unroll
      for (int e = 0; e < kEpc; ++e) s = fmaf((float)v[i].e[e], (float)v[i].e[e], s);
    }
  }
  const float inv = 1.0f / sqrtf(wave_sum(s) / (float)width + eps);
#pragma unroll
  for (int i = 0; i < RES; ++i) {
    const int c = lane + 64 * i;
    if (c >= n_chunks) continue;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) v[i].e[e] = (T)((float)v[i].e[e] * inv);
    store16(v[i], orow + c * kEpc);
  }
}

// dx = inv * dy - x * (inv^3 / n) * sum(dy * x), plus `addend` where one is given: the
// gradient is rounded to the storage type before the addition, as a separate add would see it
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rms_norm_bwd_kernel(const T* x, const T* dy, const T* addend, T* dx,
                                                           int64_t outer, int width, float eps) {
  constexpr int kEpc = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= outer) return;
  const T* row = x + r * width;
  const T* grow = dy + r * width;
  T* orow = dx + r * width;
  const T* arow = addend ? addend + r * width : nullptr;
  const float inv = 1.0f / sqrtf(row_sum_prod<T, VEC>(row, row, width, lane) / (float)width + eps);
  const float dot = row_sum_prod<T, VEC>(row, grow, width, lane);
  const float k = dot * inv * inv * inv / (float)width;
  if constexpr (VEC) {
    for (int c = lane; c < width / kEpc; c += 64) {
      const Vec16<T> vx = load16(row + c * kEpc), vg = load16(grow + c * kEpc);
      Vec16<T> o;
#pragma unroll
      for (int e = 0; e < kEpc; ++e) o.e[e] = (T)((float)vg.e[e] * inv - (float)vx.e[e] * k);
      if (arow) {
        const Vec16<T> va = load16(arow + c * kEpc);
#pragma unroll
        for (int e = 0; e < kEpc; ++e) o.e[e] = (T)((float)va.e[e] + (float)o.e[e]);
      }
      store16(o, orow + c * kEpc);
    }
  } else {
    for (int c = lane; c < width; c += 64) {
      const T g = (T)((float)grow[c] * inv - (float)row[c] * k);
      orow[c] = arow ? (T)((float)arow[c] + (float)g) : g;
    }
  }
}

// The same for rows of at most 64 * RES 16-byte chunks (aligned): a wave keeps its row of x
// and dy in registers, so each is read once instead of three and two times.  Sums run in
// the order of the general kernel: same bits.
template <typename T, int RES>
__global__ __launch_bounds__(256) void rms_norm_bwd_resident_kernel(const T* x, const T* dy, const T* addend,
                                                                    T* dx, int64_t outer, int width, float eps) {
  constexpr int kEpc = 16 / sizeof(T);
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= outer) return;
  const T* row = x + r * width;
  const T* grow = dy + r * width;
  T* orow = dx + r * width;
  const T* arow = addend ? addend + r * width : nullptr;
  const int n_chunks = width / kEpc;
  Vec16<T> vx[RES], vg[RES];
#pragma unroll
  for (int i = 0; i < RES; ++i) {
    const int c = lane + 64 * i;
    if (c < n_chunks) {
      vx[i] = load16(row + c * kEpc);
      vg[i] = load16(grow + c * kEpc);
    } else {
#pragma unroll
      for (int e = 0; e < kEpc; ++e) {
        vx[i].e[e] = (T)0.f;
        vg[i].e[e] = (T)0.f;
      }
    }
  }
  float sxx = 0.f, sxg = 0.f;
#pragma unroll
  for (int i = 0; i < RES; ++i)
#pragma unroll
    for (int e = 0; e < kEpc; ++e) {
      sxx = fmaf((float)vx[i].e[e], (float)vx[i].e[e], sxx);
      sxg = fmaf((float)vx[i].e[e], (float)vg[i].e[e], sxg);
    }
  const float inv = 1.0f / sqrtf(wave_sum(sxx) / (float)width + eps);
  const float k = wave_sum(sxg) * inv * inv * inv / (float)width;
#pragma unroll
  for (int i = 0; i < RES; ++i) {
    const int c = lane + 64 * i;
    if (c >= n_chunks) continue;
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) o.e[e] = (T)((float)vg[i].e[e] * inv - (float)vx[i].e[e] * k);
    if (arow) {
      const Vec16<T> va = load16(arow + c * kEpc);
#pragma unroll
      for (int e = 0; e < kEpc; ++e) o.e[e] = (T)((float)va.e[e] + (float)o.e[e]);
    }
    store16(o, orow + c * kEpc);
  }
}

// ---- relu_sq: y = relu(x)^2; dx = dy * 2 * relu(x) ----
// The reference's autograd adds the two equal contributions dy * r of `r * r`
// (src/ops.rs EWiseMul backward): rounding dy * r to the storage type first and then
// doubling keeps the same bits, also where the product is subnormal in f16.
template <typename T>
__device__ __forceinline__ T relu_sq_grad(float dy, float r) {
  const float g = (float)(T)(dy * r);
  return (T)(g + g);
}
template <typename T, bool BWD>
__global__ __launch_bounds__(256) void relu_sq_kernel(const T* x, const T* dy, T* out, int64_t n) {
  constexpr int kEpc = 16 / sizeof(T);
  const int64_t n_chunks = n / kEpc;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (int64_t c = tid; c < n_chunks; c += stride) {
    const Vec16<T> vx = load16_stream(x + c * kEpc);
    Vec16<T> vg, o;
    if constexpr (BWD) vg = load16_stream(dy + c * kEpc);
#pragma unroll
    for (int e = 0; e < kEpc; ++e) {
      const float r = fmaxf((float)vx.e[e], 0.f);
      if constexpr (BWD) o.e[e] = relu_sq_grad<T>((float)vg.e[e], r);
      else o.e[e] = (T)(r * r);
    }
    store16_stream(o, out + c * kEpc);
  }
  const int64_t i = n_chunks * kEpc + tid;
  if (i < n) {
    const float r = fmaxf((float)x[i], 0.f);
    if constexpr (BWD) out[i] = relu_sq_grad<T>((float)dy[i], r);
    else out[i] = (T)(r * r);
  }
}
template <typename T, bool BWD>
__global__ __launch_bounds__(256) void relu_sq_unaligned_kernel(const T* x, const T* dy, T* out,
                                                                int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float r = fmaxf((float)x[i], 0.f);
    if constexpr (BWD) out[i] = relu_sq_grad<T>((float)dy[i], r);
    else out[i] = (T)(r * r);
  }
}

// ---- cross entropy ----
// Forward: one workgroup per row streams the logits once with an online (max, sum)
// pair and keeps lse_i = ln sum exp(x_i) and loss_i = lse_i - x_i[target_i]; a second
// tiny kernel averages the per-row losses in a fixed order.  The log-probabilities are
// never written.  Rows start at any element (50257 is odd): the sweep runs over 16-byte
// chunks counted from the 16-byte boundary at or before the row start, with the two
// edge chunks masked.
constexpr int kCeThreads = 512;
constexpr int kCeInFlight = 4;

__device__ __forceinline__ void merge_ms(float& m, float& s, float m2, float s2) {
  const float mn = fmaxf(m, m2);
  const float a = (m == -INFINITY) ? 0.f : __expf(m - mn);
  const float b = (m2 == -INFINITY) ? 0.f : __expf(m2 - mn);
  s = s * a + s2 * b;
  m = mn;
}

// MODE 0: the forward.  MODE 1 and 2 also write dlogits[r, c] = (exp(x - lse) - [c == target]) *
// inv_n, the gradient of the mean loss for an upstream gradient of one: same expression, same
// bits as cross_entropy_bwd_kernel's.  In MODE 2 the workgroup keeps the whole row in registers
// between the reduction and the gradient (rows of up to kCeThreads * ce_keep<T>() 16-byte chunks:
// 57344 floats or 65536 halves), so the logits are read once; MODE 1 walks longer rows a second
// time.  The reduction takes the chunks in the same groups and order in every mode: same lse,
// same loss.
template <typename T>
constexpr int ce_keep() {  // chunks per thread MODE 2 holds (a multiple of kCeInFlight)
  return sizeof(T) == 2 ? 16 : 28;
}

template <typename T, int MODE>
__global__ __launch_bounds__(kCeThreads) void cross_entropy_fwd_kernel(
    const T* logits, const int64_t* targets, float* row_lse, float* row_loss, T* dlogits, float inv_n,
    int width, int* error_flag) {
  __shared__ float red_m[kCeThreads / 64], red_s[kCeThreads / 64];
  __shared__ float lse_all;
  constexpr int kEpc = 16 / sizeof(T);
  const int tid = threadIdx.x;
  const int64_t r = blockIdx.x;
  const T* row = logits + r * width;
  const int head = (int)((uintptr_t)row & 15) / (int)sizeof(T);
  const T* base = row - head;  // 16-byte aligned
  const int n_chunks = (head + width + kEpc - 1) / kEpc;
  constexpr int kCeKeep = ce_keep<T>();
  static_assert(kCeKeep % kCeInFlight == 0, "whole groups");
  float m = -INFINITY, s = 0.f;
  // one group of kCeInFlight chunks: the running maximum and sum take them in
  auto take_group = [&](int c0, const Vec16<T>* v) {
    float f[kCeInFlight][kEpc];
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < kCeInFlight; ++u) {
      const int lo = (c0 + u * kCeThreads) * kEpc - head;  // row position of element 0
#pragma unroll
      for (int e = 0; e < kEpc; ++e) {
        const bool in = (c0 + u * kCeThreads) < n_chunks && lo + e >= 0 && lo + e < width;
        f[u][e] = in ? (float)v[u].e[e] : -INFINITY;
        mx = fmaxf(mx, f[u][e]);
      }
    }
    if (mx > m) {
      s *= (m == -INFINITY) ? 0.f : __expf(m - mx);
      m = mx;
    }
    if (m != -INFINITY) {
#pragma unroll
      for (int u = 0; u < kCeInFlight; ++u)
#pragma unroll
        for (int e = 0; e < kEpc; ++e) s += __expf(f[u][e] - m);
    }
  };
  Vec16<T> keep[MODE == 2 ? kCeKeep : 1];
  if constexpr (MODE == 2) {
#pragma unroll
    for (int i = 0; i < kCeKeep; ++i) {  // every load of the row is in flight at once
      const int c = tid + i * kCeThreads;
      keep[i] = Vec16<T>{};
      if (c < n_chunks) keep[i] = load16_stream(base + c * kEpc);
    }
#pragma unroll
    for (int gq = 0; gq < kCeKeep / kCeInFlight; ++gq) {
      const int c0 = tid + gq * kCeInFlight * kCeThreads;
      if (c0 < n_chunks) take_group(c0, keep + gq * kCeInFlight);
    }
  } else {
    for (int c0 = tid; c0 < n_chunks; c0 += kCeThreads * kCeInFlight) {
      Vec16<T> v[kCeInFlight];
#pragma unroll
      for (int u = 0; u < kCeInFlight; ++u) {
        const int c = c0 + u * kCeThreads;
        v[u] = Vec16<T>{};
        if (c < n_chunks) v[u] = MODE == 1 ? load16(base + c * kEpc) : load16_stream(base + c * kEpc);
      }
      take_group(c0, v);
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(s, off, 64);
    merge_ms(m, s, m2, s2);
  }
  if ((tid & 63) == 0) {
    red_m[tid >> 6] = m;
    red_s[tid >> 6] = s;
  }
  __syncthreads();
  if (tid == 0) {
    m = red_m[0];
    s = red_s[0];
    for (int w = 1; w < kCeThreads / 64; ++w) merge_ms(m, s, red_m[w], red_s[w]);
    const float lse = __logf(s) + m;
    const int64_t t = targets[r];
    const bool ok = t >= 0 && t < width;
    if (!ok) atomicOr(error_flag, 1);
    row_lse[r] = lse;
    row_loss[r] = ok ? lse - (float)row[t] : 0.f;
    if (MODE != 0) lse_all = lse;
  }
  if constexpr (MODE != 0) {
    __syncthreads();
    const float lse = lse_all;
    const int64_t t = targets[r];
    T* obase = dlogits + r * width - head;  // the chunk grid of the input row
    // 16-byte stores need the output row at the input row's offset from a 16-byte boundary
    const bool same_phase = (((uintptr_t)(dlogits + r * width)) & 15) == ((uintptr_t)row & 15);
    auto write_chunk = [&](int c, const Vec16<T>& v) {
      const int lo = c * kEpc - head;  // row position of element 0
      Vec16<T> o;
#pragma unroll
      for (int e = 0; e < kEpc; ++e) {
        const float pr = __expf((float)v.e[e] - lse);
        o.e[e] = (T)((pr - (t == lo + e ? 1.0f : 0.0f)) * inv_n);
      }
      if (same_phase && lo >= 0 && lo + kEpc <= width) {
        store16_stream(o, obase + c * kEpc);
      } else {  // an edge chunk shares its 16 bytes with the neighbouring row
#pragma unroll
        for (int e = 0; e < kEpc; ++e)
          if (lo + e >= 0 && lo + e < width) obase[c * kEpc + e] = o.e[e];
      }
    };
    if constexpr (MODE == 2) {
#pragma unroll
      for (int i = 0; i < kCeKeep; ++i) {
        const int c = tid + i * kCeThreads;
        if (c < n_chunks) write_chunk(c, keep[i]);
      }
    } else {
      for (int c = tid; c < n_chunks; c += kCeThreads) write_chunk(c, load16(base + c * kEpc));
    }
  }
}

// x *= *factor, skipped where the factor is one (the gradient of a loss that is the root of
// the graph): every block reads the factor and leaves.
template <typename T>
__global__ __launch_bounds__(256) void scale_by_device_scalar_kernel(T* x, int64_t n, const float* factor) {
  const float f = *factor;
  if (f == 1.0f) return;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    x[i] = (T)((float)x[i] * f);
}

// loss = scale * sum(row_loss), additions in a fixed order
__global__ __launch_bounds__(256) void mean_rows_kernel(const float* row_loss, int64_t n, float scale,
                                                        float* loss) {
  __shared__ float red[4];
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < n; i += 256) s += row_loss[i];
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) *loss = ((red[0] + red[1]) + (red[2] + red[3])) * scale;
}

// Backward: dlogits[i, c] = (exp(x[i, c] - lse_i) - [c == target_i]) * upstream / N, one
// streaming pass over the flat [N * V] array in aligned 16-byte chunks (a chunk may
// straddle two rows).  `upstream` is the gradient of the scalar loss, in device memory.
constexpr int kCeSlab = 1024;  // 16-byte chunks per block

template <typename T>
__global__ __launch_bounds__(256) void cross_entropy_bwd_kernel(
    const T* logits, const int64_t* targets, const float* row_lse, const float* upstream, T* dlogits,
    int64_t n_rows, int width, float inv_n) {
  constexpr int kEpc = 16 / sizeof(T);
  const int64_t total = n_rows * width;
  // flat elements before the first 16-byte boundary, then whole chunks, then the tail
  const int lead = (int)(((16 - ((uintptr_t)logits & 15)) & 15) / sizeof(T));
  const float g = (upstream ? *upstream : 1.0f) * inv_n;
  auto element = [&](int64_t flat, float x) -> float {
    const int64_t r = flat / width;
    const int c = (int)(flat - r * width);
    const float p = __expf(x - row_lse[r]);
    return (p - (targets[r] == c ? 1.0f : 0.0f)) * g;
  };
  const int64_t n_chunks = total > lead ? (total - lead) / kEpc : 0;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  // each block owns one contiguous slab of kCeSlab chunks (16 KB per array): with a read
  // and a write stream, neighbouring blocks on neighbouring addresses move more bytes per
  // second than a grid-stride sweep
  const int64_t slab0 = (int64_t)blockIdx.x * kCeSlab;
  const int64_t slab1 = slab0 + kCeSlab < n_chunks ? slab0 + kCeSlab : n_chunks;
  for (int64_t c = slab0 + threadIdx.x; c < slab1; c += 256) {
    const int64_t flat0 = lead + c * kEpc;
    const Vec16<T> vx = load16_stream(logits + flat0);
    // one division per chunk; the elements after a row boundary step to the next row
    int64_t r = flat0 / width;
    int col = (int)(flat0 - r * width);
    float lse = row_lse[r];
    int64_t t = targets[r];
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) {
      if (col == width) {
        col = 0;
        ++r;
        lse = row_lse[r];
        t = targets[r];
      }
      const float p = __expf((float)vx.e[e] - lse);
      o.e[e] = (T)((p - (t == col ? 1.0f : 0.0f)) * g);
      ++col;
    }
    store16_stream(o, dlogits + flat0);
  }
  // edge elements: fewer than 2 chunks' worth, by the first threads
  const int64_t n_edge = total - n_chunks * kEpc;
  if (tid < n_edge) {
    const int64_t flat = tid < lead ? tid : n_chunks * kEpc + tid;
    dlogits[flat] = (T)element(flat, (float)logits[flat]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void cross_entropy_bwd_unaligned_kernel(
    const T* logits, const int64_t* targets, const float* row_lse, const float* upstream, T* dlogits,
    int64_t n_rows, int width, float inv_n) {
  const int64_t total = n_rows * width;
  const float g = (upstream ? *upstream : 1.0f) * inv_n;
  for (int64_t flat = (int64_t)blockIdx.x * 256 + threadIdx.x; flat < total;
       flat += (int64_t)gridDim.x * 256) {
    const int64_t r = flat / width;
    const int c = (int)(flat - r * width);
    const float p = __expf((float)logits[flat] - row_lse[r]);
    dlogits[flat] = (T)((p - (targets[r] == c ? 1.0f : 0.0f)) * g);
  }
}

// ---- argmax over the last axis: the greedy sampling step, kept on the device so that a
// generation loop never waits for the host ----
// One workgroup per row; ties go to the lowest index; NaNs are never selected.
// 1024 threads: a 50257-wide row is then two rounds of four 16-byte loads per thread (with
// 256 threads it was six dependent rounds, 14.6 us for 32 rows).
constexpr int kArgmaxThreads = 1024;
template <typename T>
__global__ __launch_bounds__(kArgmaxThreads) void argmax_rows_kernel(const T* x, int64_t* out, int width) {
  __shared__ float red_v[kArgmaxThreads / 64];
  __shared__ int red_i[kArgmaxThreads / 64];
  constexpr int kEpc = 16 / sizeof(T);
  constexpr int kInFlight = 4;
  const T* row = x + (int64_t)blockIdx.x * width;
  // 16-byte chunks counted from the 16-byte boundary at or before the row start (rows
  // start at any element), the two edge chunks masked; several chunks in flight per
  // thread: a row of 50257 logits is otherwise a chain of dependent round trips
  const int head = (int)((uintptr_t)row & 15) / (int)sizeof(T);
  const T* base = row - head;
  const int n_chunks = (head + width + kEpc - 1) / kEpc;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int c0 = threadIdx.x; c0 < n_chunks; c0 += kArgmaxThreads * kInFlight) {
    Vec16<T> v[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      v[u] = Vec16<T>{};
      if (c0 + kArgmaxThreads * u < n_chunks) v[u] = load16_stream(base + (c0 + kArgmaxThreads * u) * kEpc);
    }
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      const int lo = (c0 + kArgmaxThreads * u) * kEpc - head;  // row position of element 0 of the chunk
#pragma unroll
      for (int e = 0; e < kEpc; ++e) {
        const int c = lo + e;
        const float f = (float)v[u].e[e];
        // positions ascend within a thread, so a strict comparison keeps the lowest index
        if (c >= 0 && c < width && c0 + kArgmaxThreads * u < n_chunks && f > best) {
          best = f;
          best_i = c;
        }
      }
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float v2 = __shfl_xor(best, off, 64);
    const int i2 = __shfl_xor(best_i, off, 64);
    if (v2 > best || (v2 == best && i2 < best_i)) {
      best = v2;
      best_i = i2;
    }
  }
  if ((threadIdx.x & 63) == 0) {
    red_v[threadIdx.x >> 6] = best;
    red_i[threadIdx.x >> 6] = best_i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxThreads / 64; ++w)
      if (red_v[w] > best || (red_v[w] == best && red_i[w] < best_i)) {
        best = red_v[w];
        best_i = red_i[w];
      }
    out[blockIdx.x] = best_i == 0x7fffffff ? 0 : best_i;  // a row of NaNs / -inf picks 0
  }
}

unsigned stream_grid(int64_t work_items) {
  const int64_t blocks = (work_items + 255) / 256;
  const int64_t cap = 256 * 16;
  return (unsigned)(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
}

}  // namespace

template <typename T>
static void index_select_t(const T* table, const int64_t* idx, T* out, int64_t n_rows, int64_t n_idx,
                           int width, int* flag, hipStream_t stream) {
  const bool vec = aligned16(table) && aligned16(out) && (width * sizeof(T)) % 16 == 0;
  const dim3 grid((unsigned)((n_idx + 3) / 4));
  if (vec)
    hipLaunchKernelGGL((index_select_kernel<T, true>), grid, dim3(256), 0, stream, table, idx, out,
                       n_rows, n_idx, width, flag);
  else
    hipLaunchKernelGGL((index_select_kernel<T, false>), grid, dim3(256), 0, stream, table, idx, out,
                       n_rows, n_idx, width, flag);
}

void launch_index_select(int dtype_f16, const void* table, const int64_t* idx, void* out,
                         int64_t n_rows, int64_t n_idx, int width, int* flag, hipStream_t stream) {
  LaunchScope scope("index_select", stream);
  if (dtype_f16)
    index_select_t((const half_t*)table, idx, (half_t*)out, n_rows, n_idx, width, flag, stream);
  else
    index_select_t((const float*)table, idx, (float*)out, n_rows, n_idx, width, flag, stream);
}

void launch_index_add(int dtype_f16, const void* src, const int64_t* idx, void* dst, int64_t n_rows,
                      int64_t n_idx, int width, int* flag, hipStream_t stream) {
  LaunchScope scope("index_add", stream);
  for (int64_t first = 0; first < n_idx; first += kIndexAddChunk) {
    const int n = (int)(n_idx - first < kIndexAddChunk ? n_idx - first : kIndexAddChunk);
    const size_t lds = (size_t)((n + 63) / 64) * 2 * sizeof(unsigned int);
    if (dtype_f16)
      hipLaunchKernelGGL(index_add_kernel<half_t>, dim3((unsigned)n), dim3(256), lds, stream,
                         (const half_t*)src + first * width, idx + first, (half_t*)dst, n_rows, n, width,
                         flag);
    else
      hipLaunchKernelGGL(index_add_kernel<float>, dim3((unsigned)n), dim3(256), lds, stream,
                         (const float*)src + first * width, idx + first, (float*)dst, n_rows, n, width,
                         flag);
  }
}

template <typename T>
static void rms_norm_t(const T* x, const T* dy, const T* addend, T* out, int64_t outer, int width, float eps,
                       bool bwd, hipStream_t stream) {
  const bool vec = aligned16(x) && aligned16(out) && (!bwd || aligned16(dy)) && aligned16(addend) &&
                   (width * sizeof(T)) % 16 == 0;
  const dim3 grid((unsigned)((outer + 3) / 4));
  constexpr int kResident = 4;  // 16-byte chunks per lane the resident backward holds of x and of dy
  if (bwd && vec && width / (int)(16 / sizeof(T)) <= 64 * kResident) {
    hipLaunchKernelGGL((rms_norm_bwd_resident_kernel<T, kResident>), grid, dim3(256), 0, stream, x, dy, addend,
                       out, outer, width, eps);
  } else if (bwd) {
    if (vec)
      hipLaunchKernelGGL((rms_norm_bwd_kernel<T, true>), grid, dim3(256), 0, stream, x, dy, addend, out,
                         outer, width, eps);
    else
      hipLaunchKernelGGL((rms_norm_bwd_kernel<T, false>), grid, dim3(256), 0, stream, x, dy, addend, out,
                         outer, width, eps);
  } else if (vec && width / (int)(16 / sizeof(T)) <= 64 * kResident) {
    hipLaunchKernelGGL((rms_norm_fwd_resident_kernel<T, kResident>), grid, dim3(256), 0, stream, x, out, outer,
                       width, eps);
  } else {
    if (vec)
      hipLaunchKernelGGL((rms_norm_fwd_kernel<T, true>), grid, dim3(256), 0, stream, x, out, outer,
                         width, eps);
    else
      hipLaunchKernelGGL((rms_norm_fwd_kernel<T, false>), grid, dim3(256), 0, stream, x, out, outer,
                         width, eps);
  }
}

void launch_rms_norm(int dtype_f16, const void* x, const void* dy, const void* addend, void* out, int64_t outer,
                     int width, float eps, int bwd, hipStream_t stream) {
  LaunchScope scope(bwd ? "rms_norm_bwd" : "rms_norm_fwd", stream);
  if (dtype_f16)
    rms_norm_t((const half_t*)x, (const half_t*)dy, (const half_t*)addend, (half_t*)out, outer, width, eps,
               bwd != 0, stream);
  else
    rms_norm_t((const float*)x, (const float*)dy, (const float*)addend, (float*)out, outer, width, eps,
               bwd != 0, stream);
}

template <typename T, bool BWD>
static void relu_sq_t(const T* x, const T* dy, T* out, int64_t n, hipStream_t stream) {
  const bool vec = aligned16(x) && aligned16(out) && (!BWD || aligned16(dy));
  if (vec)
    hipLaunchKernelGGL((relu_sq_kernel<T, BWD>), dim3(stream_grid(n / (16 / sizeof(T)) + 16)),
                       dim3(256), 0, stream, x, dy, out, n);
  else
    hipLaunchKernelGGL((relu_sq_unaligned_kernel<T, BWD>), dim3(stream_grid(n)), dim3(256), 0, stream,
                       x, dy, out, n);
}

void launch_relu_sq(int dtype_f16, const void* x, const void* dy, void* out, int64_t n, int bwd,
                    hipStream_t stream) {
  LaunchScope scope(bwd ? "relu_sq_bwd" : "relu_sq_fwd", stream);
  if (dtype_f16) {
    if (bwd) relu_sq_t<half_t, true>((const half_t*)x, (const half_t*)dy, (half_t*)out, n, stream);
    else relu_sq_t<half_t, false>((const half_t*)x, nullptr, (half_t*)out, n, stream);
  } else {
    if (bwd) relu_sq_t<float, true>((const float*)x, (const float*)dy, (float*)out, n, stream);
    else relu_sq_t<float, false>((const float*)x, nullptr, (float*)out, n, stream);
  }
}

void launch_argmax_rows(int dtype_f16, const void* x, int64_t* out, int64_t outer, int width,
                        hipStream_t stream) {
  LaunchScope scope("argmax_rows", stream);
  if (dtype_f16)
    hipLaunchKernelGGL(argmax_rows_kernel<half_t>, dim3((unsigned)outer), dim3(kArgmaxThreads), 0, stream,
                       (const half_t*)x, out, width);
  else
    hipLaunchKernelGGL(argmax_rows_kernel<float>, dim3((unsigned)outer), dim3(kArgmaxThreads), 0, stream,
                       (const float*)x, out, width);
}

void launch_cross_entropy_fwd(int dtype_f16, const void* logits, const int64_t* targets, float* row_lse,
                              float* row_loss, float* loss, void* dlogits, int64_t n_rows, int width,
                              int* flag, hipStream_t stream) {
  LaunchScope scope(dlogits ? "cross_entropy_fwd_grad" : "cross_entropy_fwd", stream);
  const float inv_n = (float)(1.0 / (double)n_rows);
  const dim3 grid((unsigned)n_rows), block(kCeThreads);
  // a row and its possible lead-in fit the registers of a workgroup?
  const bool resident = (int64_t)width + 16 <= (int64_t)kCeThreads * (dtype_f16 ? ce_keep<half_t>() * 8 : ce_keep<float>() * 4);
  auto go = [&](auto kernel, auto* x, auto* dx) {
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, x, targets, row_lse, row_loss, dx, inv_n, width, flag);
  };
  if (dtype_f16) {
    const half_t* x = (const half_t*)logits;
    half_t* dx = (half_t*)dlogits;
    if (!dlogits) go(cross_entropy_fwd_kernel<half_t, 0>, x, dx);
    else if (resident) go(cross_entropy_fwd_kernel<half_t, 2>, x, dx);
    else go(cross_entropy_fwd_kernel<half_t, 1>, x, dx);
  } else {
    const float* x = (const float*)logits;
    float* dx = (float*)dlogits;
    if (!dlogits) go(cross_entropy_fwd_kernel<float, 0>, x, dx);
    else if (resident) go(cross_entropy_fwd_kernel<float, 2>, x, dx);
    else go(cross_entropy_fwd_kernel<float, 1>, x, dx);
  }
  hipLaunchKernelGGL(mean_rows_kernel, dim3(1), dim3(256), 0, stream, row_loss, n_rows,
                     (float)(1.0 / (double)n_rows), loss);
}

void launch_scale_by_device_scalar(int dtype_f16, void* x, int64_t n, const float* factor, hipStream_t stream) {
  LaunchScope scope("scale_by_scalar", stream);
  if (dtype_f16)
    hipLaunchKernelGGL(scale_by_device_scalar_kernel<half_t>, dim3(stream_grid(n)), dim3(256), 0, stream,
                       (half_t*)x, n, factor);
  else
    hipLaunchKernelGGL(scale_by_device_scalar_kernel<float>, dim3(stream_grid(n)), dim3(256), 0, stream,
                       (float*)x, n, factor);
}

void launch_cross_entropy_bwd(int dtype_f16, const void* logits, const int64_t* targets,
                              const float* row_lse, const float* upstream, void* dlogits,
                              int64_t n_rows, int width, hipStream_t stream) {
  LaunchScope scope("cross_entropy_bwd", stream);
  const float inv_n = (float)(1.0 / (double)n_rows);
  const int64_t total = n_rows * width;
  const bool same_phase = (((uintptr_t)logits ^ (uintptr_t)dlogits) & 15) == 0;
  if (dtype_f16) {
    if (same_phase)
      hipLaunchKernelGGL(cross_entropy_bwd_kernel<half_t>, dim3((unsigned)(total / 8 / kCeSlab + 1)), dim3(256),
                         0, stream, (const half_t*)logits, targets, row_lse, upstream,
                         (half_t*)dlogits, n_rows, width, inv_n);
    else
      hipLaunchKernelGGL(cross_entropy_bwd_unaligned_kernel<half_t>, dim3(stream_grid(total)),
                         dim3(256), 0, stream, (const half_t*)logits, targets, row_lse, upstream,
                         (half_t*)dlogits, n_rows, width, inv_n);
  } else {
    if (same_phase)
      hipLaunchKernelGGL(cross_entropy_bwd_kernel<float>, dim3((unsigned)(total / 4 / kCeSlab + 1)), dim3(256),
                         0, stream, (const float*)logits, targets, row_lse, upstream, (float*)dlogits,
                         n_rows, width, inv_n);
    else
      hipLaunchKernelGGL(cross_entropy_bwd_unaligned_kernel<float>, dim3(stream_grid(total)), dim3(256),
                         0, stream, (const float*)logits, targets, row_lse, upstream, (float*)dlogits,
                         n_rows, width, inv_n);
  }
}

}  // namespace deers
