// Rotary position embedding fused with the head split / merge around the attention
// core.
//
// The reference applies RoPE to the [B,T,H,D] projections with narrow, four
// element-wise multiplies, two adds and a cat, then permutes to [B,H,T,D]
// (src/models/gpt.rs:49-73, 135-137); the cat leaves q and k with a non-unit
// innermost stride, so every consumer compacts them again.  Here one pass reads the
// projection rows and writes rotated rows straight into compact [B,H,T,D], which
// the attention kernels take as is; the backward applies the inverse rotation to
// dq/dk ([B,H,T,D]) and writes the gradient of the projection in [B,T,H,D].
//   y1 = x1*cos + x2*sin        dx1 = dy1*cos - dy2*sin
//   y2 = x2*cos - x1*sin        dx2 = dy2*cos + dy1*sin
// with x1 = x[..., :D/2], x2 = x[..., D/2:], cos/sin [T, D/2] in the tensor's dtype
// (src/models/gpt.rs:12-47).  Arithmetic is f32 with one rounding to the storage
// type.  One thread moves 16 bytes of each half; a wave covers whole 128-byte+
// rows on both sides.  HBM-bound: 2 x tensor bytes per launch (+ the small tables).
#include "common.h"

namespace deers {

namespace {

template <typename T> struct Vec16;
template <> struct Vec16<half_t> { typedef half8 type; static constexpr int N = 8; };
template <> struct Vec16<float> { typedef floatx4 type; static constexpr int N = 4; };

struct RopeParams {
  const void* src; void* dst;
  const void* cos; const void* sin;
  int64_t s_b, s_t, s_h;   // element strides of the strided side ([B,T,H,D] order for
                           // forward input / backward output; [B,H,T,D] given as b,t,h)
  int64_t d_b, d_t, d_h;   // element strides of the other side, same naming
  int B, T, H, D;
};

// INVERSE = false: src is the projection (strides s_*), dst the rotated heads (d_*).
// INVERSE = true : src is the gradient of the rotated heads, dst the projection grad.
template <typename T, bool INVERSE>
__global__ __launch_bounds__(256) void rope_kernel(RopeParams p) {
  typedef typename Vec16<T>::type V;
  constexpr int N = Vec16<T>::N;
  const int half_chunks = p.D / 2 / N;  // 16-byte chunks in half a row
  const int64_t total = (int64_t)p.B * p.T * p.H * half_chunks;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % half_chunks);
    int64_t r = i / half_chunks;
    const int h = (int)(r % p.H); r /= p.H;
    const int t = (int)(r % p.T);
    const int b = (int)(r / p.T);
    const T* s = (const T*)p.src + b * p.s_b + t * p.s_t + h * p.s_h + c * N;
    T* d = (T*)p.dst + b * p.d_b + t * p.d_t + h * p.d_h + c * N;
    const V a1 = *(const V*)s, a2 = *(const V*)(s + p.D / 2);
    const V cs = *(const V*)((const T*)p.cos + (int64_t)t * (p.D / 2) + c * N);
    const V sn = *(const V*)((const T*)p.sin + (int64_t)t * (p.D / 2) + c * N);
    V o1, o2;
#pragma unroll
    for (int e = 0; e < N; ++e) {
      const float x1 = (float)a1[e], x2 = (float)a2[e], co = (float)cs[e];
      const float si = INVERSE ? -(float)sn[e] : (float)sn[e];
      o1[e] = (T)(x1 * co + x2 * si);
      o2[e] = (T)(x2 * co - x1 * si);
    }
    *(V*)d = o1;
    *(V*)(d + p.D / 2) = o2;
  }
}

// The same rotation one (x1, x2) pair per thread, for head widths whose half row is not a
// whole number of 16-byte chunks (the reference's own GPT test runs head_dim 2,
// tests/gpt.rs:38-49) or rows that are not 16-byte aligned.  Same arithmetic and rounding.
template <typename T, bool INVERSE>
__global__ __launch_bounds__(256) void rope_pair_kernel(RopeParams p) {
  const int half = p.D / 2;
  const int64_t total = (int64_t)p.B * p.T * p.H * half;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % half);
    int64_t r = i / half;
    const int h = (int)(r % p.H); r /= p.H;
    const int t = (int)(r % p.T);
    const int b = (int)(r / p.T);
    const T* s = (const T*)p.src + b * p.s_b + t * p.s_t + h * p.s_h + c;
    T* d = (T*)p.dst + b * p.d_b + t * p.d_t + h * p.d_h + c;
    const float x1 = (float)s[0], x2 = (float)s[half];
    const float co = (float)((const T*)p.cos)[(int64_t)t * half + c];
    const float sn = (float)((const T*)p.sin)[(int64_t)t * half + c];
    const float si = INVERSE ? -sn : sn;
    d[0] = (T)(x1 * co + x2 * si);
    d[half] = (T)(x2 * co - x1 * si);
  }
}

// One generation step's handling of the new token's projections, in one launch: q and k
// rotated at the step's position, q to a compact [B,H,D] tensor, k and the unrotated v to
// row `pos` of their caches.  Inputs are [B,H,D] views by strides {b,h} (thirds of a fused
// [B,3C] projection row); caches [B,H,cap,D] by strides {b,h,t}.
struct DecodeQkvParams {
  const void* q; const void* k; const void* v;
  const void* cos; const void* sin;  // the position's rows: D/2 elements each
  void* q_out; void* k_cache; void* v_cache;
  int64_t in_b, in_h;
  int64_t c_b, c_h, c_t;
  int64_t pos;
  int B, H, D;
};
template <typename T>
__global__ __launch_bounds__(256) void decode_qkv_kernel(DecodeQkvParams p) {
  typedef typename Vec16<T>::type V;
  constexpr int N = Vec16<T>::N;
  const int half_chunks = p.D / 2 / N;
  const int per_tensor = p.B * p.H * half_chunks;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= 3 * per_tensor) return;
  const int which = i / per_tensor;  // 0 q, 1 k, 2 v
  int r = i - which * per_tensor;
  const int c = r % half_chunks; r /= half_chunks;
  const int h = r % p.H;
  const int b = r / p.H;
  const T* src = (const T*)(which == 0 ? p.q : which == 1 ? p.k : p.v) + b * p.in_b + h * p.in_h + c * N;
  T* dst = which == 0 ? (T*)p.q_out + ((int64_t)b * p.H + h) * p.D + c * N
                      : (T*)(which == 1 ? p.k_cache : p.v_cache) + b * p.c_b + h * p.c_h + p.pos * p.c_t + c * N;
  const V a1 = *(const V*)src, a2 = *(const V*)(src + p.D / 2);
  if (which == 2) {
    *(V*)dst = a1;
    *(V*)(dst + p.D / 2) = a2;
    return;
  }
  const V cs = *(const V*)((const T*)p.cos + c * N);
  const V sn = *(const V*)((const T*)p.sin + c * N);
  V o1, o2;
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float x1 = (float)a1[e], x2 = (float)a2[e], co = (float)cs[e], si = (float)sn[e];
    o1[e] = (T)(x1 * co + x2 * si);
    o2[e] = (T)(x2 * co - x1 * si);
  }
  *(V*)dst = o1;
  *(V*)(dst + p.D / 2) = o2;
}

}  // namespace

void launch_decode_qkv(int dtype_f16, const void* q, const void* k, const void* v,
                       const int64_t* in_strides, const void* cos_row, const void* sin_row, void* q_out,
                       void* k_cache, void* v_cache, const int64_t* cache_strides, int64_t pos, int B,
                       int H, int D, hipStream_t stream) {
  DecodeQkvParams p{};
  p.q = q; p.k = k; p.v = v; p.cos = cos_row; p.sin = sin_row;
  p.q_out = q_out; p.k_cache = k_cache; p.v_cache = v_cache;
  p.in_b = in_strides[0]; p.in_h = in_strides[1];
  p.c_b = cache_strides[0]; p.c_h = cache_strides[1]; p.c_t = cache_strides[2];
  p.pos = pos; p.B = B; p.H = H; p.D = D;
  const int n16 = dtype_f16 ? 8 : 4;
  const int total = 3 * B * H * (D / 2 / n16);
  LaunchScope scope("decode_qkv", stream);
  if (dtype_f16)
    hipLaunchKernelGGL((decode_qkv_kernel<half_t>), dim3((total + 255) / 256), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((decode_qkv_kernel<float>), dim3((total + 255) / 256), dim3(256), 0, stream, p);
}

// x: logical [B,T,H,D] with element strides xs = {b,t,h} (D stride 1); y: [B,H,T,D],
// compact or with element strides {b,h,t} (a row range of a KV cache).
// inverse: dy [B,H,T,D] with strides {b,h,t} -> dx compact [B,T,H,D].
// vectorised: every row and half row on both sides is a whole number of aligned 16-byte
// chunks; otherwise one pair per thread.
void launch_rope(int dtype_f16, bool inverse, bool vectorised, const void* src,
                 const int64_t* src_strides, const void* cos, const void* sin, void* dst,
                 const int64_t* dst_strides, int B, int T, int H, int D, hipStream_t stream) {
  RopeParams p{};
  p.src = src; p.dst = dst; p.cos = cos; p.sin = sin;
  p.B = B; p.T = T; p.H = H; p.D = D;
  if (!inverse) {
    p.s_b = src_strides[0]; p.s_t = src_strides[1]; p.s_h = src_strides[2];
    p.d_b = (int64_t)H * T * D; p.d_h = (int64_t)T * D; p.d_t = D;
    if (dst_strides) { p.d_b = dst_strides[0]; p.d_h = dst_strides[1]; p.d_t = dst_strides[2]; }
  } else {
    p.s_b = src_strides[0]; p.s_h = src_strides[1]; p.s_t = src_strides[2];
    p.d_b = (int64_t)T * H * D; p.d_t = (int64_t)H * D; p.d_h = D;
  }
  const int n16 = dtype_f16 ? 8 : 4;
  const int64_t total = vectorised ? (int64_t)B * T * H * (D / 2 / n16) : (int64_t)B * T * H * (D / 2);
  const int64_t blocks = (total + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
  LaunchScope scope(inverse ? "rope_bwd" : "rope_fwd", stream);
  if (!vectorised) {
    if (dtype_f16) {
      if (inverse) hipLaunchKernelGGL((rope_pair_kernel<half_t, true>), dim3(grid), dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((rope_pair_kernel<half_t, false>), dim3(grid), dim3(256), 0, stream, p);
    } else {
      if (inverse) hipLaunchKernelGGL((rope_pair_kernel<float, true>), dim3(grid), dim3(256), 0, stream, p);
      else hipLaunchKernelGGL((rope_pair_kernel<float, false>), dim3(grid), dim3(256), 0, stream, p);
    }
    return;
  }
  if (dtype_f16) {
    if (inverse) hipLaunchKernelGGL((rope_kernel<half_t, true>), dim3(grid), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((rope_kernel<half_t, false>), dim3(grid), dim3(256), 0, stream, p);
  } else {
    if (inverse) hipLaunchKernelGGL((rope_kernel<float, true>), dim3(grid), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((rope_kernel<float, false>), dim3(grid), dim3(256), 0, stream, p);
  }
}

}  // namespace deers
