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

}  // namespace

// x: logical [B,T,H,D] with element strides xs = {b,t,h} (D stride 1); y: [B,H,T,D],
// compact or with element strides {b,h,t} (a row range of a KV cache).
// inverse: dy [B,H,T,D] with strides {b,h,t} -> dx compact [B,T,H,D].
void launch_rope(int dtype_f16, bool inverse, const void* src, const int64_t* src_strides,
                 const void* cos, const void* sin, void* dst, const int64_t* dst_strides, int B,
                 int T, int H, int D, hipStream_t stream) {
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
  const int64_t total = (int64_t)B * T * H * (D / 2 / n16);
  const int64_t blocks = (total + 255) / 256;
  const unsigned grid = (unsigned)(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
  LaunchScope scope(inverse ? "rope_bwd" : "rope_fwd", stream);
  if (dtype_f16) {
    if (inverse) hipLaunchKernelGGL((rope_kernel<half_t, true>), dim3(grid), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((rope_kernel<half_t, false>), dim3(grid), dim3(256), 0, stream, p);
  } else {
    if (inverse) hipLaunchKernelGGL((rope_kernel<float, true>), dim3(grid), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((rope_kernel<float, false>), dim3(grid), dim3(256), 0, stream, p);
  }
}

}  // namespace deers
