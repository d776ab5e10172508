// delta pre-pass of the attention backward, shared by the f16 and f32 paths.
#pragma once

#include "common.h"

namespace deers {

// ---------------------------------------------------------------------------
// delta[b,h,t] = sum_d dO[t,d] * O[t,d]; LPR lanes share one row.
// ---------------------------------------------------------------------------
template <typename E, int D>
__global__ __launch_bounds__(256) void attn_bwd_delta_kernel(BwdParams p, int B) {
  constexpr int VEC = 16 / sizeof(E);
  constexpr int LPR = D / VEC;  // lanes per row
  typedef E vec_t __attribute__((ext_vector_type(VEC)));
  const int64_t rows = (int64_t)B * p.H * p.T;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int part = threadIdx.x % LPR;
  float acc = 0.f;
  if (row < rows) {
    const int t = row % p.T;
    const int bh = row / p.T;
    const int b = bh / p.H, h = bh % p.H;
    const E* o = (const E*)p.o + b * p.so.b + h * p.so.h + (int64_t)t * p.so.t + VEC * part;
    const E* d = (const E*)p.d_o + b * p.sdo.b + h * p.sdo.h + (int64_t)t * p.sdo.t + VEC * part;
    const vec_t ov = *(const vec_t*)o;
    const vec_t dv = *(const vec_t*)d;
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc += (float)ov[e] * (float)dv[e];
  }
#pragma unroll
  for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (row < rows && part == 0) p.delta[row] = acc;
}

}  // namespace deers
