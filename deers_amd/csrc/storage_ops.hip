// The generic kernels of BackendStorage (src/storage.rs:227-306) that the fused ops do
// not replace: element-wise unary / scalar / binary kernels over strided layouts,
// row reductions, log-sum-exp, gather and scatter_add.
//
//   unary      src/storage.rs:32-123 (Neg, Exp, Log, Sin, Cos, Tanh, Relu, ReluBackward,
//              ScalarAdd/Mul/Div) and ewise_powf; CPU src/storage/cpu.rs:203-265
//   binary     src/storage.rs:126-190 (add, sub, mul, div, powf, eq) over two layouts of
//              one shape (a broadcast operand has stride 0); CPU src/storage/cpu.rs:267-321
//   reduce     sum / max of each run of reduce_size elements of a compact buffer;
//              CPU src/storage/cpu.rs:323-357
//   lse        ln sum exp per row; CPU src/storage/cpu.rs:755-791
//   gather / scatter_add along one dimension of a compact [left, dim, right] buffer;
//              CPU src/storage/cpu.rs:398-553, 891-934
//
// Outputs are compact, as the trait requires.  Arithmetic is f32 for both storage
// types with one rounding to the storage type (the reference's f16 kernels convert to
// f32, operate and convert back); a scalar operand is rounded to the storage type first,
// as `f16::from_f32(s as f32)` does, the exponent of ewise_powf is not.  Rows of up to
// 32 elements are reduced left to right in the storage type, exactly as the reference
// does; longer rows are summed in f32 in a fixed tree order: reproducible, but not the
// reference's left-to-right order (and for f16 more accurate than its f16 accumulator).  scatter_add
// keeps the reference's order: one thread owns an output column and applies that
// column's additions in ascending source position.  This file is compiled with NaNs
// and infinities honoured.
#include "common.h"
#include "storage_ops.h"

namespace deers {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <typename T> struct alignas(16) Vec16 { T e[16 / sizeof(T)]; };
template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T* p) {
  return __builtin_bit_cast(Vec16<T>, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
template <typename T>
__device__ __forceinline__ void store16(const Vec16<T>& x, T* p) {
  __builtin_nontemporal_store(__builtin_bit_cast(u32x4, x), reinterpret_cast<u32x4*>(p));
}
inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

inline int stream_blocks(int64_t work_items) {
  const int64_t b = (work_items + 255) / 256;
  return (int)std::min<int64_t>(std::max<int64_t>(b, 1), 256 * 32);
}

// ---- scalar functions ----
template <int OP> __device__ __forceinline__ float unary_fn(float v, float p) {
  if constexpr (OP == kUnaryNeg) return -v;
  else if constexpr (OP == kUnaryExp) return expf(v);
  else if constexpr (OP == kUnaryLog) return logf(v);
  else if constexpr (OP == kUnarySin) return sinf(v);
  else if constexpr (OP == kUnaryCos) return cosf(v);
  else if constexpr (OP == kUnaryTanh) return tanhf(v);
  else if constexpr (OP == kUnaryRelu) return fmaxf(v, 0.f);  // NaN -> 0, as f32::max
  else if constexpr (OP == kUnaryReluBackward) return v > 0.f ? 1.f : 0.f;
  else if constexpr (OP == kUnaryScalarAdd) return v + p;
  else if constexpr (OP == kUnaryScalarMul) return v * p;
  else if constexpr (OP == kUnaryScalarDiv) return v / p;
  else return powf(v, p);
}
template <int OP> __device__ __forceinline__ float binary_fn(float a, float b) {
  if constexpr (OP == kBinaryAdd) return a + b;
  else if constexpr (OP == kBinarySub) return a - b;
  else if constexpr (OP == kBinaryMul) return a * b;
  else if constexpr (OP == kBinaryDiv) return a / b;
  else if constexpr (OP == kBinaryPow) return powf(a, b);
  else return a == b ? 1.f : 0.f;
}

// element offset of linear index i (row-major over v.shape) in a strided view
__device__ __forceinline__ int64_t view_offset(const StridedView& v, uint32_t i) {
  int64_t off = 0;
  for (int d = v.ndim - 1; d > 0; --d) {
    const uint32_t q = i / v.shape[d];
    off += (int64_t)(i - q * v.shape[d]) * v.stride[d];
    i = q;
  }
  return off + (int64_t)i * v.stride[0];
}

// ---- element-wise kernels ----
template <typename T, int OP>
__global__ __launch_bounds__(256) void unary_compact_kernel(const T* x, T* out, int64_t n, float p) {
  constexpr int kEpc = 16 / sizeof(T);
  const int64_t n_chunks = n / kEpc;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (int64_t c = tid; c < n_chunks; c += stride) {
    const Vec16<T> vx = load16(x + c * kEpc);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) o.e[e] = (T)unary_fn<OP>((float)vx.e[e], p);
    store16(o, out + c * kEpc);
  }
  const int64_t i = n_chunks * kEpc + tid;
  if (i < n) out[i] = (T)unary_fn<OP>((float)x[i], p);
}
template <typename T, int OP>
__global__ __launch_bounds__(256) void unary_strided_kernel(const T* x, StridedView v, T* out,
                                                            uint32_t n, float p) {
  const uint32_t stride = gridDim.x * 256u;
  for (uint64_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride)
    out[i] = (T)unary_fn<OP>((float)x[view_offset(v, (uint32_t)i)], p);
}
template <typename T, int OP>
__global__ __launch_bounds__(256) void binary_compact_kernel(const T* a, const T* b, T* out,
                                                             int64_t n) {
  constexpr int kEpc = 16 / sizeof(T);
  const int64_t n_chunks = n / kEpc;
  const int64_t stride = (int64_t)gridDim.x * 256;
  const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (int64_t c = tid; c < n_chunks; c += stride) {
    const Vec16<T> va = load16(a + c * kEpc), vb = load16(b + c * kEpc);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) o.e[e] = (T)binary_fn<OP>((float)va.e[e], (float)vb.e[e]);
    store16(o, out + c * kEpc);
  }
  const int64_t i = n_chunks * kEpc + tid;
  if (i < n) out[i] = (T)binary_fn<OP>((float)a[i], (float)b[i]);
}
template <typename T, int OP>
__global__ __launch_bounds__(256) void binary_strided_kernel(const T* a, StridedView va, const T* b,
                                                             StridedView vb, T* out, uint32_t n) {
  const uint32_t stride = gridDim.x * 256u;
  for (uint64_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += stride)
    out[i] = (T)binary_fn<OP>((float)a[view_offset(va, (uint32_t)i)],
                              (float)b[view_offset(vb, (uint32_t)i)]);
}

// Strided operands whose innermost dimension is contiguous (stride 1) or broadcast
// (stride 0), with an extent that is a multiple of a 16-byte chunk and chunk-aligned
// outer strides: one index decomposition per chunk, 16-byte loads (or one scalar load
// fanned out).  This is the shape of the attention chain's broadcasts: a [B,1,T,T] mask
// over the heads, a [B,H,T,1] row statistic over the keys.
template <typename T>
__device__ __forceinline__ Vec16<T> load_chunk(const T* base, const StridedView& v, uint32_t elem) {
  const T* p = base + view_offset(v, elem);
  if (v.stride[v.ndim - 1] != 0) return *reinterpret_cast<const Vec16<T>*>(p);
  Vec16<T> r;
  const T x = *p;
#pragma unroll
  for (int e = 0; e < (int)(16 / sizeof(T)); ++e) r.e[e] = x;
  return r;
}
template <typename T, int OP>
__global__ __launch_bounds__(256) void unary_rows_kernel(const T* x, StridedView v, T* out,
                                                         uint32_t n_chunks, float p) {
  constexpr int kEpc = 16 / sizeof(T);
  const uint32_t stride = gridDim.x * 256u;
  for (uint64_t c = blockIdx.x * 256u + threadIdx.x; c < n_chunks; c += stride) {
    const Vec16<T> vx = load_chunk(x, v, (uint32_t)c * kEpc);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) o.e[e] = (T)unary_fn<OP>((float)vx.e[e], p);
    store16(o, out + c * kEpc);
  }
}
template <typename T, int OP>
__global__ __launch_bounds__(256) void binary_rows_kernel(const T* a, StridedView va, const T* b,
                                                          StridedView vb, T* out, uint32_t n_chunks) {
  constexpr int kEpc = 16 / sizeof(T);
  const uint32_t stride = gridDim.x * 256u;
  for (uint64_t c = blockIdx.x * 256u + threadIdx.x; c < n_chunks; c += stride) {
    const Vec16<T> xa = load_chunk(a, va, (uint32_t)c * kEpc), xb = load_chunk(b, vb, (uint32_t)c * kEpc);
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < kEpc; ++e) o.e[e] = (T)binary_fn<OP>((float)xa.e[e], (float)xb.e[e]);
    store16(o, out + c * kEpc);
  }
}
// true if a chunk of 16 / elem_bytes consecutive elements (in row-major order over the
// view's shape, starting at a multiple of the chunk) never straddles the view's
// innermost dimension and can be fetched as described above
inline bool chunkable(const void* base, const StridedView& v, int elem_bytes) {
  const int epc = 16 / elem_bytes;
  const int64_t s_in = v.stride[v.ndim - 1];
  if (v.shape[v.ndim - 1] % epc != 0) return false;
  if (s_in == 0) return true;  // scalar loads: no alignment needed
  if (s_in != 1 || !aligned16(base)) return false;
  for (int d = 0; d + 1 < v.ndim; ++d)
    if (v.stride[d] % epc != 0) return false;
  return true;
}

// ---- row reductions ----
struct SumOp {
  static constexpr float kIdentity = 0.f;
  static __device__ __forceinline__ float f(float a, float b) { return a + b; }
};
struct MaxOp {  // f32::max ignores a NaN operand, so NaN is its identity (an all-NaN row gives NaN)
  static constexpr float kIdentity = __builtin_nanf("");
  static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
};
struct MaxFromNegInf {  // fold(NEG_INFINITY, f32::max) of the reference's log_sum_exp
  static constexpr float kIdentity = -INFINITY;
  static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
};
template <typename R>
__device__ __forceinline__ float wave_reduce(float s) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s = R::f(s, __shfl_xor(s, off, 64));
  return s;
}
// this lane's share of a row: elements lane, lane + n_lanes, ... (16-byte pieces when
// the row allows it), each passed through `map` first
struct Identity {
  __device__ __forceinline__ float operator()(float x) const { return x; }
};
template <typename T, typename R, typename Map>
__device__ __forceinline__ float row_partial(const T* row, int64_t rs, int lane, int n_lanes, Map map) {
  constexpr int kEpc = 16 / sizeof(T);
  float acc[4] = {R::kIdentity, R::kIdentity, R::kIdentity, R::kIdentity};
  if ((((uintptr_t)row) & 15) == 0 && rs % kEpc == 0) {
    const int64_t n_chunks = rs / kEpc;
    for (int64_t c = lane; c < n_chunks; c += n_lanes) {
      const Vec16<T> v = *reinterpret_cast<const Vec16<T>*>(row + c * kEpc);
#pragma unroll
      for (int e = 0; e < kEpc; ++e) acc[e & 3] = R::f(acc[e & 3], map((float)v.e[e]));
    }
  } else {
    for (int64_t i = lane; i < rs; i += n_lanes) acc[0] = R::f(acc[0], map((float)row[i]));
  }
  return R::f(R::f(acc[0], acc[1]), R::f(acc[2], acc[3]));
}
// rows of up to 32 elements: one thread per row, left to right (the reference's order)
template <typename T, typename R>
__global__ __launch_bounds__(256) void reduce_thread_kernel(const T* x, T* out, int64_t outer, int rs) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= outer) return;
  const T* row = x + r * rs;
  float acc = (float)row[0];
  for (int i = 1; i < rs; ++i) acc = (float)(T)R::f(acc, (float)row[i]);  // accumulator of type T
  out[r] = (T)acc;
}
// one wavefront per row
template <typename T, typename R>
__global__ __launch_bounds__(256) void reduce_wave_kernel(const T* x, T* out, int64_t outer, int64_t rs) {
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= outer) return;
  const float s = wave_reduce<R>(row_partial<T, R>(x + r * rs, rs, threadIdx.x & 63, 64, Identity{}));
  if ((threadIdx.x & 63) == 0) out[r] = (T)s;
}
// one workgroup per row
constexpr int kRowBlock = 1024;
template <typename T, typename R>
__global__ __launch_bounds__(kRowBlock) void reduce_block_kernel(const T* x, T* out, int64_t rs) {
  __shared__ float part[kRowBlock / 64];
  const int64_t r = blockIdx.x;
  float s = wave_reduce<R>(row_partial<T, R>(x + r * rs, rs, threadIdx.x, kRowBlock, Identity{}));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x < 64) {
    s = threadIdx.x < kRowBlock / 64 ? part[threadIdx.x] : R::kIdentity;
    s = wave_reduce<R>(s);
    if (threadIdx.x == 0) out[r] = (T)s;
  }
}

// ---- log-sum-exp per row, in the reference's two sweeps: the maximum (NaNs ignored),
// then the sum of exp(x - maximum); the second sweep finds the row in cache.  Special
// values come out as they do there (a row of -inf, or one holding +inf, gives NaN).
struct ExpMinus {
  float m;
  __device__ __forceinline__ float operator()(float x) const { return expf(x - m); }
};
template <typename T>
__global__ __launch_bounds__(256) void lse_wave_kernel(const T* x, T* out, int64_t outer, int64_t rs) {
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= outer) return;
  const T* row = x + r * rs;
  const int lane = threadIdx.x & 63;
  const float m = wave_reduce<MaxFromNegInf>(row_partial<T, MaxFromNegInf>(row, rs, lane, 64, Identity{}));
  const float s = wave_reduce<SumOp>(row_partial<T, SumOp>(row, rs, lane, 64, ExpMinus{m}));
  if (lane == 0) out[r] = (T)(logf(s) + m);
}
template <typename R>
__device__ __forceinline__ float block_reduce(float s, float* part) {  // result in every thread
  s = wave_reduce<R>(s);
  __syncthreads();  // part may still be read from an earlier reduction
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
  __syncthreads();
  s = (threadIdx.x & 63) < kRowBlock / 64 ? part[threadIdx.x & 63] : R::kIdentity;
  return wave_reduce<R>(s);
}
template <typename T>
__global__ __launch_bounds__(kRowBlock) void lse_block_kernel(const T* x, T* out, int64_t rs) {
  __shared__ float part[kRowBlock / 64];
  const int64_t r = blockIdx.x;
  const T* row = x + r * rs;
  const float m = block_reduce<MaxFromNegInf>(row_partial<T, MaxFromNegInf>(row, rs, threadIdx.x, kRowBlock, Identity{}), part);
  const float s = block_reduce<SumOp>(row_partial<T, SumOp>(row, rs, threadIdx.x, kRowBlock, ExpMinus{m}), part);
  if (threadIdx.x == 0) out[r] = (T)(logf(s) + m);
}

// ---- gather / scatter_add along the middle dimension of [left, dim, right] ----
// out[l, i, r] = src[l, idx[l, i, r], r]
template <typename T>
__global__ __launch_bounds__(256) void gather_kernel(const T* src, const int64_t* idx, T* out,
                                                     int64_t n_out, int64_t src_dim, int64_t index_len,
                                                     int64_t right, int* error_flag) {
  const int64_t stride = (int64_t)gridDim.x * 256;
  bool bad = false;
  for (int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x; o < n_out; o += stride) {
    const int64_t l = o / (index_len * right);
    const int64_t r = o % right;
    const int64_t k = idx[o];
    if (k < 0 || k >= src_dim) {
      bad = true;
      continue;
    }
    out[o] = src[(l * src_dim + k) * right + r];
  }
  if (bad) *error_flag = 1;
}
// dst[l, idx[l, i, r], r] += src[l, i, r], i ascending: thread (l, r) owns column (l, :, r)
template <typename T>
__global__ __launch_bounds__(256) void scatter_add_kernel(const T* src, const int64_t* idx, T* dst,
                                                          int64_t left, int64_t dst_dim,
                                                          int64_t index_len, int64_t right,
                                                          int* error_flag) {
  const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (col >= left * right) return;
  const int64_t l = col / right, r = col % right;
  const T* s = src + l * index_len * right + r;
  const int64_t* ix = idx + l * index_len * right + r;
  T* d = dst + l * dst_dim * right + r;
  bool bad = false;
  for (int64_t i = 0; i < index_len; ++i) {
    const int64_t k = ix[i * right];
    if (k < 0 || k >= dst_dim) {
      bad = true;
      continue;
    }
    // the reference adds in the storage type: f16 += f16 rounds after every addition
    d[k * right] = (T)((float)d[k * right] + (float)s[i * right]);
  }
  if (bad) *error_flag = 1;
}

template <typename T, int OP>
void unary_t(const T* x, const StridedView* view, T* out, int64_t n, float p, hipStream_t stream) {
  if (!view) {
    if (aligned16(x) && aligned16(out)) {
      hipLaunchKernelGGL((unary_compact_kernel<T, OP>), dim3(stream_blocks(n / (16 / sizeof(T)) + 256)),
                         dim3(256), 0, stream, x, out, n, p);
      return;
    }
    StridedView flat{};
    flat.ndim = 1;
    flat.shape[0] = (uint32_t)n;
    flat.stride[0] = 1;
    hipLaunchKernelGGL((unary_strided_kernel<T, OP>), dim3(stream_blocks(n)), dim3(256), 0, stream, x,
                       flat, out, (uint32_t)n, p);
    return;
  }
  if (aligned16(out) && chunkable(x, *view, sizeof(T))) {
    const uint32_t n_chunks = (uint32_t)(n / (16 / sizeof(T)));
    hipLaunchKernelGGL((unary_rows_kernel<T, OP>), dim3(stream_blocks(n_chunks)), dim3(256), 0, stream, x,
                       *view, out, n_chunks, p);
    return;
  }
  hipLaunchKernelGGL((unary_strided_kernel<T, OP>), dim3(stream_blocks(n)), dim3(256), 0, stream, x,
                     *view, out, (uint32_t)n, p);
}
template <typename T, int OP>
void binary_t(const T* a, const StridedView* va, const T* b, const StridedView* vb, T* out, int64_t n,
              hipStream_t stream) {
  if (!va && !vb && aligned16(a) && aligned16(b) && aligned16(out)) {
    hipLaunchKernelGGL((binary_compact_kernel<T, OP>), dim3(stream_blocks(n / (16 / sizeof(T)) + 256)),
                       dim3(256), 0, stream, a, b, out, n);
    return;
  }
  StridedView flat{};
  flat.ndim = 1;
  flat.shape[0] = (uint32_t)n;
  flat.stride[0] = 1;
  const StridedView& wa = va ? *va : flat;
  const StridedView& wb = vb ? *vb : flat;
  if (aligned16(out) && chunkable(a, wa, sizeof(T)) && chunkable(b, wb, sizeof(T))) {
    const uint32_t n_chunks = (uint32_t)(n / (16 / sizeof(T)));
    hipLaunchKernelGGL((binary_rows_kernel<T, OP>), dim3(stream_blocks(n_chunks)), dim3(256), 0, stream, a,
                       wa, b, wb, out, n_chunks);
    return;
  }
  hipLaunchKernelGGL((binary_strided_kernel<T, OP>), dim3(stream_blocks(n)), dim3(256), 0, stream, a, wa,
                     b, wb, out, (uint32_t)n);
}

template <typename T, int... OPS>
bool unary_dispatch(int op, std::integer_sequence<int, OPS...>, const T* x, const StridedView* view,
                    T* out, int64_t n, float p, hipStream_t stream) {
  return ((op == OPS ? (unary_t<T, OPS>(x, view, out, n, p, stream), true) : false) || ...);
}
template <typename T, int... OPS>
bool binary_dispatch(int op, std::integer_sequence<int, OPS...>, const T* a, const StridedView* va,
                     const T* b, const StridedView* vb, T* out, int64_t n, hipStream_t stream) {
  return ((op == OPS ? (binary_t<T, OPS>(a, va, b, vb, out, n, stream), true) : false) || ...);
}

template <typename T, typename R>
void reduce_t(const T* x, T* out, int64_t outer, int64_t rs, hipStream_t stream) {
  if (rs <= 32)
    hipLaunchKernelGGL((reduce_thread_kernel<T, R>), dim3((unsigned)((outer + 255) / 256)), dim3(256), 0,
                       stream, x, out, outer, (int)rs);
  else if (rs < 16384 || outer >= 2048)
    hipLaunchKernelGGL((reduce_wave_kernel<T, R>), dim3((unsigned)((outer + 3) / 4)), dim3(256), 0, stream,
                       x, out, outer, rs);
  else
    hipLaunchKernelGGL((reduce_block_kernel<T, R>), dim3((unsigned)outer), dim3(kRowBlock), 0, stream, x,
                       out, rs);
}
template <typename T>
void lse_t(const T* x, T* out, int64_t outer, int64_t rs, hipStream_t stream) {
  if (rs < 16384 || outer >= 2048)
    hipLaunchKernelGGL((lse_wave_kernel<T>), dim3((unsigned)((outer + 3) / 4)), dim3(256), 0, stream, x,
                       out, outer, rs);
  else
    hipLaunchKernelGGL((lse_block_kernel<T>), dim3((unsigned)outer), dim3(kRowBlock), 0, stream, x, out,
                       rs);
}

}  // namespace

static const char* const kUnaryNames[kUnaryCount] = {
    "unary_neg",  "unary_exp",           "unary_log",        "unary_sin",        "unary_cos",        "unary_tanh",
    "unary_relu", "unary_relu_backward", "unary_scalar_add", "unary_scalar_mul", "unary_scalar_div", "unary_powf"};
static const char* const kBinaryNames[kBinaryCount] = {"binary_add", "binary_sub", "binary_mul",
                                                       "binary_div", "binary_powf", "binary_eq"};

void launch_unary(int dtype_f16, int op, const void* x, const StridedView* view, void* out, int64_t n,
                  double param, hipStream_t stream) {
  LaunchScope scope(kUnaryNames[op], stream);
  const bool scalar_op = op == kUnaryScalarAdd || op == kUnaryScalarMul || op == kUnaryScalarDiv;
  float p = (float)param;
  if (dtype_f16 && scalar_op) p = (float)(half_t)p;
  using Ops = std::make_integer_sequence<int, kUnaryCount>;
  if (dtype_f16)
    unary_dispatch<half_t>(op, Ops{}, (const half_t*)x, view, (half_t*)out, n, p, stream);
  else
    unary_dispatch<float>(op, Ops{}, (const float*)x, view, (float*)out, n, p, stream);
}

void launch_binary(int dtype_f16, int op, const void* a, const StridedView* va, const void* b,
                   const StridedView* vb, void* out, int64_t n, hipStream_t stream) {
  LaunchScope scope(kBinaryNames[op], stream);
  using Ops = std::make_integer_sequence<int, kBinaryCount>;
  if (dtype_f16)
    binary_dispatch<half_t>(op, Ops{}, (const half_t*)a, va, (const half_t*)b, vb, (half_t*)out, n, stream);
  else
    binary_dispatch<float>(op, Ops{}, (const float*)a, va, (const float*)b, vb, (float*)out, n, stream);
}

void launch_reduce(int dtype_f16, int op_max, const void* x, void* out, int64_t outer, int64_t rs,
                   hipStream_t stream) {
  LaunchScope scope(op_max ? "reduce_max" : "reduce_sum", stream);
  if (dtype_f16) {
    if (op_max) reduce_t<half_t, MaxOp>((const half_t*)x, (half_t*)out, outer, rs, stream);
    else reduce_t<half_t, SumOp>((const half_t*)x, (half_t*)out, outer, rs, stream);
  } else {
    if (op_max) reduce_t<float, MaxOp>((const float*)x, (float*)out, outer, rs, stream);
    else reduce_t<float, SumOp>((const float*)x, (float*)out, outer, rs, stream);
  }
}

void launch_log_sum_exp(int dtype_f16, const void* x, void* out, int64_t outer, int64_t rs,
                        hipStream_t stream) {
  LaunchScope scope("log_sum_exp", stream);
  if (dtype_f16) lse_t<half_t>((const half_t*)x, (half_t*)out, outer, rs, stream);
  else lse_t<float>((const float*)x, (float*)out, outer, rs, stream);
}

void launch_gather(int elem_bytes, const void* src, const int64_t* idx, void* out, int64_t left,
                   int64_t src_dim, int64_t index_len, int64_t right, int* error_flag,
                   hipStream_t stream) {
  LaunchScope scope("gather", stream);
  const int64_t n_out = left * index_len * right;
  const dim3 grid(stream_blocks(n_out));
  if (elem_bytes == 2)
    hipLaunchKernelGGL((gather_kernel<uint16_t>), grid, dim3(256), 0, stream, (const uint16_t*)src, idx,
                       (uint16_t*)out, n_out, src_dim, index_len, right, error_flag);
  else if (elem_bytes == 4)
    hipLaunchKernelGGL((gather_kernel<uint32_t>), grid, dim3(256), 0, stream, (const uint32_t*)src, idx,
                       (uint32_t*)out, n_out, src_dim, index_len, right, error_flag);
  else
    hipLaunchKernelGGL((gather_kernel<uint64_t>), grid, dim3(256), 0, stream, (const uint64_t*)src, idx,
                       (uint64_t*)out, n_out, src_dim, index_len, right, error_flag);
}

void launch_scatter_add(int dtype_f16, const void* src, const int64_t* idx, void* dst, int64_t left,
                        int64_t dst_dim, int64_t index_len, int64_t right, int* error_flag,
                        hipStream_t stream) {
  LaunchScope scope("scatter_add", stream);
  const dim3 grid((unsigned)((left * right + 255) / 256));
  if (dtype_f16)
    hipLaunchKernelGGL((scatter_add_kernel<half_t>), grid, dim3(256), 0, stream, (const half_t*)src, idx,
                       (half_t*)dst, left, dst_dim, index_len, right, error_flag);
  else
    hipLaunchKernelGGL((scatter_add_kernel<float>), grid, dim3(256), 0, stream, (const float*)src, idx,
                       (float*)dst, left, dst_dim, index_len, right, error_flag);
}

}  // namespace deers
