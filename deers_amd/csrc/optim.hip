// Fused AdamW step, sum of squares and in-place scaling: the optimizer side of a
// training step.
//
// The reference runs AdamW::step_with_grads (src/optim.rs:214-251) as a chain of
// thirteen element-wise tensor ops per parameter, each a pass over HBM with a rounded
// intermediate tensor, and clip_grad_norm (src/optim.rs:258-296) as a square, a
// reduction and a scaling pass per gradient.  Here one kernel reads w, g, m, v once
// and writes w, m, v once (28 B per f32 parameter, 14 B per f16), with the gradient
// scaling of clip_grad_norm folded in.
//
// The arithmetic keeps the reference's order and rounds after every operation to the
// tensor's type (the ops are separate kernels there), so results are the same bits:
// no fused multiply-add may be formed (contraction is switched off below), and
// division and square root are the correctly rounded ones.  For f16 tensors that
// includes the reference's quirks: every scalar is rounded to f16 first, so the default
// eps = 1e-8 becomes 0.
#include "common.h"

namespace deers {

namespace {

constexpr int kOptThreads = 256;

// Rounds an f32 intermediate to the tensor's element type.
template <typename T> __device__ __forceinline__ float rnd(float x) { return (float)(T)x; }
template <> __device__ __forceinline__ float rnd<float>(float x) { return x; }

struct AdamWScalars {  // already cast the way storage::ScalarMul / ScalarAdd cast (src/storage.rs:108-123)
  float beta1, one_minus_beta1, beta2, one_minus_beta2, inv_bc1, inv_bc2, decay, eps, lr, grad_scale;
  int use_decay, use_grad_scale;
};

template <typename T>
__device__ __forceinline__ void adamw_element(float& w, float g, float& m, float& v,
                                              const AdamWScalars& k) {
#pragma clang fp contract(off)
  if (k.use_grad_scale) g = rnd<T>(g * k.grad_scale);              // clip_grad_norm's grad * scale
  const float m1 = rnd<T>(m * k.beta1);
  const float m2 = rnd<T>(g * k.one_minus_beta1);
  m = rnd<T>(m1 + m2);                                             // m = b1*m + (1-b1)*g
  const float gg = rnd<T>(g * g);
  const float v1 = rnd<T>(v * k.beta2);
  const float v2 = rnd<T>(gg * k.one_minus_beta2);
  v = rnd<T>(v1 + v2);                                             // v = b2*v + (1-b2)*g^2
  const float m_hat = rnd<T>(m * k.inv_bc1);
  const float v_hat = rnd<T>(v * k.inv_bc2);
  const float decayed = k.use_decay ? rnd<T>(w * k.decay) : w;     // w * (1 - lr*lambda)
  const float den = rnd<T>(rnd<T>(sqrtf(v_hat)) + k.eps);
  const float update = rnd<T>(m_hat / den);
  w = rnd<T>(decayed - rnd<T>(update * k.lr));
}

template <typename T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// All four streams are touched once per step: non-temporal accesses keep them from
// displacing each other in L2.
template <typename T>
__device__ __forceinline__ Vec16<T> stream_load(const T* p) {
  return __builtin_bit_cast(Vec16<T>, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
template <typename T>
__device__ __forceinline__ void stream_store(const Vec16<T>& x, T* p) {
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4, x), reinterpret_cast<u32x4*>(p));
}

// Element-wise path for operands that are not 16-byte aligned.
template <typename T>
__global__ __launch_bounds__(kOptThreads) void adamw_unaligned_kernel(T* w, const T* g, T* m, T* v,
                                                                      int64_t n, AdamWScalars k) {
  const int64_t stride = (int64_t)gridDim.x * kOptThreads;
  for (int64_t i = (int64_t)blockIdx.x * kOptThreads + threadIdx.x; i < n; i += stride) {
    float fw = (float)w[i], fm = (float)m[i], fv = (float)v[i];
    adamw_element<T>(fw, (float)g[i], fm, fv, k);
    w[i] = (T)fw;
    m[i] = (T)fm;
    v[i] = (T)fv;
  }
}

// ---- sum of squares: fixed partition, fixed order, so the result is reproducible ----
constexpr int kSumsqBlocks = 2048;  // 8 workgroups per CU

template <typename T>
__global__ __launch_bounds__(kOptThreads) void sumsq_partial_kernel(const T* g, int64_t n,
                                                                    float* partial) {
  __shared__ float red[kOptThreads / 64];
  constexpr int kEpc = 16 / sizeof(T);
  constexpr int kAcc = 4;  // independent chunks in flight per thread
  // elements before the first 16-byte boundary, whole chunks, elements after the last
  const int64_t lead_all = (int64_t)((16 - ((uintptr_t)g & 15)) & 15) / (int64_t)sizeof(T);
  const int64_t lead = lead_all < n ? lead_all : n;
  const int64_t n_chunks = (n - lead) / kEpc;
  const T* body = g + lead;
  float acc[kAcc] = {0.f, 0.f, 0.f, 0.f};
  const int64_t tid = (int64_t)blockIdx.x * kOptThreads + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * kOptThreads;
  for (int64_t c0 = tid; c0 < n_chunks; c0 += stride * kAcc) {
    Vec16<T> x[kAcc];
#pragma unroll
    for (int u = 0; u < kAcc; ++u)
      if (c0 + u * stride < n_chunks) x[u] = stream_load(body + (c0 + u * stride) * kEpc);
#pragma unroll
    for (int u = 0; u < kAcc; ++u)
      if (c0 + u * stride < n_chunks) {
#pragma unroll
        for (int e = 0; e < kEpc; ++e) acc[u] = fmaf((float)x[u].e[e], (float)x[u].e[e], acc[u]);
      }
  }
  float s = (acc[0] + acc[1]) + (acc[2] + acc[3]);
  // the fewer than 2 * kEpc edge elements go to the first threads of the grid
  const int64_t n_edge = n - n_chunks * kEpc;
  if (tid < n_edge) {
    const float x = (float)(tid < lead ? g[tid] : g[n_chunks * kEpc + tid]);
    s = fmaf(x, x, s);
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(kOptThreads) void sumsq_final_kernel(const float* partial, int n_partial,
                                                                  float* out, int accumulate) {
  __shared__ float red[kOptThreads / 64];
  float s = 0.f;
  for (int i = threadIdx.x; i < n_partial; i += kOptThreads) s += partial[i];
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float total = (red[0] + red[1]) + (red[2] + red[3]);
    *out = accumulate ? *out + total : total;
  }
}

template <typename T>
__global__ __launch_bounds__(kOptThreads) void scale_kernel(T* x, int64_t n, float scale) {
  const int64_t stride = (int64_t)gridDim.x * kOptThreads;
  for (int64_t i = (int64_t)blockIdx.x * kOptThreads + threadIdx.x; i < n; i += stride)
    x[i] = (T)((float)x[i] * scale);
}

// ---- many tensors in one launch ----
// A training step updates ~150 parameter tensors, most of them small; one launch per
// tensor costs more in dispatch than in data movement.  Each block owns one contiguous
// 16 KB slab of each array, which also moves more bytes per second than a grid-stride
// sweep over the four arrays did (5.5 against 4.5 TB/s on 162 M parameters).  Up to kMultiMax tensors travel in
// the kernel arguments; block b finds its tensor by binary search over the prefix of
// blocks per tensor and works on kMultiElems consecutive elements of it.
constexpr int kMultiMax = 48;
constexpr int kMultiElemsBytes = 16384;  // bytes of each array one block handles

struct MultiAdamW {
  void* w[kMultiMax];
  const void* g[kMultiMax];
  void* m[kMultiMax];
  void* v[kMultiMax];
  int64_t n[kMultiMax];
  int first_block[kMultiMax + 1];
  int count;
};
struct MultiSumsq {
  const void* x[kMultiMax];
  int64_t n[kMultiMax];
  int first_block[kMultiMax + 1];
  int count;
};

__device__ __forceinline__ int find_tensor(const int* first_block, int count, int block) {
  int lo = 0, hi = count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (first_block[mid] <= block) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

template <typename T>
__global__ __launch_bounds__(kOptThreads) void adamw_multi_kernel(MultiAdamW t, AdamWScalars k) {
  constexpr int kEpc = 16 / sizeof(T);
  constexpr int kElems = kMultiElemsBytes / sizeof(T);
  const int ti = find_tensor(t.first_block, t.count, blockIdx.x);
  const int64_t begin = (int64_t)(blockIdx.x - t.first_block[ti]) * kElems;
  const int64_t n = t.n[ti];
  const int64_t end = begin + kElems < n ? begin + kElems : n;
  T* w = (T*)t.w[ti] + begin;
  const T* g = (const T*)t.g[ti] + begin;
  T* m = (T*)t.m[ti] + begin;
  T* v = (T*)t.v[ti] + begin;
  const int len = (int)(end - begin);
  const int n_chunks = len / kEpc;  // operands are 16-byte aligned and begin is a multiple of kElems
  for (int c = threadIdx.x; c < n_chunks; c += kOptThreads) {
    Vec16<T> cw = stream_load(w + c * kEpc), cm = stream_load(m + c * kEpc), cv = stream_load(v + c * kEpc);
    const Vec16<T> cg = stream_load(g + c * kEpc);
#pragma unroll
    for (int e = 0; e < kEpc; ++e) {
      float fw = (float)cw.e[e], fm = (float)cm.e[e], fv = (float)cv.e[e];
      adamw_element<T>(fw, (float)cg.e[e], fm, fv, k);
      cw.e[e] = (T)fw;
      cm.e[e] = (T)fm;
      cv.e[e] = (T)fv;
    }
    stream_store(cw, w + c * kEpc);
    stream_store(cm, m + c * kEpc);
    stream_store(cv, v + c * kEpc);
  }
  const int i = n_chunks * kEpc + threadIdx.x;
  if (i < len) {
    float fw = (float)w[i], fm = (float)m[i], fv = (float)v[i];
    adamw_element<T>(fw, (float)g[i], fm, fv, k);
    w[i] = (T)fw;
    m[i] = (T)fm;
    v[i] = (T)fv;
  }
}

template <typename T>
__global__ __launch_bounds__(kOptThreads) void sumsq_multi_kernel(MultiSumsq t, float* partial) {
  __shared__ float red[kOptThreads / 64];
  constexpr int kEpc = 16 / sizeof(T);
  constexpr int kElems = kMultiElemsBytes / sizeof(T);
  const int ti = find_tensor(t.first_block, t.count, blockIdx.x);
  const int64_t begin = (int64_t)(blockIdx.x - t.first_block[ti]) * kElems;
  const int64_t n = t.n[ti];
  const int64_t end = begin + kElems < n ? begin + kElems : n;
  const T* x = (const T*)t.x[ti] + begin;
  const int len = (int)(end - begin);
  const int n_chunks = len / kEpc;
  float s = 0.f;
  for (int c = threadIdx.x; c < n_chunks; c += kOptThreads) {
    const Vec16<T> cx = stream_load(x + c * kEpc);
#pragma unroll
    for (int e = 0; e < kEpc; ++e) s = fmaf((float)cx.e[e], (float)cx.e[e], s);
  }
  const int i = n_chunks * kEpc + threadIdx.x;
  if (i < len) s = fmaf((float)x[i], (float)x[i], s);
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) partial[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

// Casts a host-side f64 scalar the way the reference's scalar ops do: to f32, and for
// f16 tensors on to f16 (src/storage.rs:108-123).
float cast_scalar(double x, int dtype_f16) {
  const float f = (float)x;
  return dtype_f16 ? (float)(half_t)f : f;
}

// f64 power by repeated squaring, the algorithm behind Rust's f64::powi.
double powi(double a, int b) {
  const bool recip = b < 0;
  double r = 1.0;
  while (true) {
    if (b & 1) r *= a;
    b /= 2;
    if (b == 0) break;
    a *= a;
  }
  return recip ? 1.0 / r : r;
}

unsigned grid_for(int64_t work_items) {
  const int64_t blocks = (work_items + kOptThreads - 1) / kOptThreads;
  const int64_t cap = 256 * 16;  // 16 workgroups of 256 threads per CU keep the loop short
  return (unsigned)(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
}

}  // namespace

int sumsq_partial_count() { return kSumsqBlocks; }

static AdamWScalars make_scalars(int dtype_f16, double lr, double beta1, double beta2, double eps,
                                 double weight_decay, int step, double grad_scale) {
  // the derived scalars exactly as src/optim.rs:217-246 forms them in f64
  AdamWScalars k;
  const double bc1 = 1.0 - powi(beta1, step), bc2 = 1.0 - powi(beta2, step);
  k.beta1 = cast_scalar(beta1, dtype_f16);
  k.one_minus_beta1 = cast_scalar(1.0 - beta1, dtype_f16);
  k.beta2 = cast_scalar(beta2, dtype_f16);
  k.one_minus_beta2 = cast_scalar(1.0 - beta2, dtype_f16);
  k.inv_bc1 = cast_scalar(1.0 / bc1, dtype_f16);
  k.inv_bc2 = cast_scalar(1.0 / bc2, dtype_f16);
  k.decay = cast_scalar(1.0 - lr * weight_decay, dtype_f16);
  k.eps = cast_scalar(eps, dtype_f16);
  k.lr = cast_scalar(lr, dtype_f16);
  k.grad_scale = cast_scalar(grad_scale, dtype_f16);
  k.use_decay = weight_decay > 0.0;
  k.use_grad_scale = grad_scale != 1.0;
  return k;
}

void launch_adamw_multi(int dtype_f16, int count, void* const* w, const void* const* g, void* const* m,
                        void* const* v, const int64_t* sizes, double lr, double beta1, double beta2,
                        double eps, double weight_decay, int step, double grad_scale,
                        hipStream_t stream);

void launch_adamw(int dtype_f16, void* w, const void* g, void* m, void* v, int64_t n, double lr,
                  double beta1, double beta2, double eps, double weight_decay, int step,
                  double grad_scale, hipStream_t stream) {
  const bool aligned =
      (((uintptr_t)w | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v) & 15) == 0;
  if (aligned) {  // the slab kernel, as a group of one
    launch_adamw_multi(dtype_f16, 1, &w, &g, &m, &v, &n, lr, beta1, beta2, eps, weight_decay, step,
                       grad_scale, stream);
    return;
  }
  const AdamWScalars k = make_scalars(dtype_f16, lr, beta1, beta2, eps, weight_decay, step, grad_scale);
  LaunchScope scope("adamw_step", stream);
  if (dtype_f16)
    hipLaunchKernelGGL(adamw_unaligned_kernel<half_t>, dim3(grid_for(n)), dim3(kOptThreads), 0, stream,
                       (half_t*)w, (const half_t*)g, (half_t*)m, (half_t*)v, n, k);
  else
    hipLaunchKernelGGL(adamw_unaligned_kernel<float>, dim3(grid_for(n)), dim3(kOptThreads), 0, stream,
                       (float*)w, (const float*)g, (float*)m, (float*)v, n, k);
}

int multi_max_tensors() { return kMultiMax; }

int64_t multi_blocks(int dtype_f16, int64_t n) {
  const int64_t elems = kMultiElemsBytes / (dtype_f16 ? 2 : 4);
  return (n + elems - 1) / elems;
}

// One launch over up to kMultiMax tensors (all 16-byte aligned, sizes > 0).
void launch_adamw_multi(int dtype_f16, int count, void* const* w, const void* const* g, void* const* m,
                        void* const* v, const int64_t* sizes, double lr, double beta1, double beta2,
                        double eps, double weight_decay, int step, double grad_scale,
                        hipStream_t stream) {
  MultiAdamW t;
  int blocks = 0;
  for (int i = 0; i < count; ++i) {
    t.w[i] = w[i];
    t.g[i] = g[i];
    t.m[i] = m[i];
    t.v[i] = v[i];
    t.n[i] = sizes[i];
    t.first_block[i] = blocks;
    blocks += (int)multi_blocks(dtype_f16, sizes[i]);
  }
  t.first_block[count] = blocks;
  t.count = count;
  const AdamWScalars k = make_scalars(dtype_f16, lr, beta1, beta2, eps, weight_decay, step, grad_scale);
  LaunchScope scope("adamw_step", stream);
  if (dtype_f16)
    hipLaunchKernelGGL(adamw_multi_kernel<half_t>, dim3(blocks), dim3(kOptThreads), 0, stream, t, k);
  else
    hipLaunchKernelGGL(adamw_multi_kernel<float>, dim3(blocks), dim3(kOptThreads), 0, stream, t, k);
}

// Partial sums of up to kMultiMax tensors into partial[partial_offset ...]; returns the
// number of partials written.
int launch_sumsq_multi(int dtype_f16, int count, const void* const* x, const int64_t* sizes,
                       float* partial, hipStream_t stream) {
  MultiSumsq t;
  int blocks = 0;
  for (int i = 0; i < count; ++i) {
    t.x[i] = x[i];
    t.n[i] = sizes[i];
    t.first_block[i] = blocks;
    blocks += (int)multi_blocks(dtype_f16, sizes[i]);
  }
  t.first_block[count] = blocks;
  t.count = count;
  LaunchScope scope("sumsq", stream);
  if (dtype_f16)
    hipLaunchKernelGGL(sumsq_multi_kernel<half_t>, dim3(blocks), dim3(kOptThreads), 0, stream, t, partial);
  else
    hipLaunchKernelGGL(sumsq_multi_kernel<float>, dim3(blocks), dim3(kOptThreads), 0, stream, t, partial);
  return blocks;
}

void launch_sumsq_final(const float* partial, int n_partial, float* out, int accumulate,
                        hipStream_t stream) {
  LaunchScope scope("sumsq", stream);
  hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), dim3(kOptThreads), 0, stream, partial, n_partial, out,
                     accumulate);
}

void launch_sumsq(int dtype_f16, const void* g, int64_t n, float* partial, float* out,
                  int accumulate, hipStream_t stream) {
  LaunchScope scope("sumsq", stream);
  const int64_t want = (n / (dtype_f16 ? 8 : 4) + kOptThreads - 1) / kOptThreads;
  const int blocks = (int)(want < 1 ? 1 : (want < kSumsqBlocks ? want : kSumsqBlocks));
  if (dtype_f16)
    hipLaunchKernelGGL(sumsq_partial_kernel<half_t>, dim3(blocks), dim3(kOptThreads), 0, stream,
                       (const half_t*)g, n, partial);
  else
    hipLaunchKernelGGL(sumsq_partial_kernel<float>, dim3(blocks), dim3(kOptThreads), 0, stream,
                       (const float*)g, n, partial);
  hipLaunchKernelGGL(sumsq_final_kernel, dim3(1), dim3(kOptThreads), 0, stream, partial, blocks, out,
                     accumulate);
}

void launch_scale(int dtype_f16, void* x, int64_t n, double scale, hipStream_t stream) {
  LaunchScope scope("scale", stream);
  const float s = cast_scalar(scale, dtype_f16);
  if (dtype_f16)
    hipLaunchKernelGGL(scale_kernel<half_t>, dim3(grid_for(n)), dim3(kOptThreads), 0, stream,
                       (half_t*)x, n, s);
  else
    hipLaunchKernelGGL(scale_kernel<float>, dim3(grid_for(n)), dim3(kOptThreads), 0, stream,
                       (float*)x, n, s);
}

}  // namespace deers
