// Decode attention: one query row per (b,h) against a KV cache of L rows, f16.
//
// Same math as the forward with tgt_len = 1 and seqlen_offset = L-1, where the
// causal mask row is all zero (src/nn/functional.rs:26,42).  1 FLOP per byte:
// the kernel is an HBM stream, so the design is about bytes in flight, not
// matrix cores.
//
//   grid = (splits, B*H).  A workgroup streams `chunk` cache rows of one head.
//   A row of D halfs is covered by LPR = D/8 lanes with one 16-byte load each,
//   so a wave reads 1 KiB of K and 1 KiB of V per load instruction, fully
//   coalesced.  ROWS_PER_IT rows are in flight per lane group (K and V loads
//   are issued together: V does not wait for the scores).
//   Each lane group keeps a private online softmax (m, l, o[8] per lane) over
//   the rows it visits; groups are merged once at the end through LDS in a
//   fixed order, and the split partial (m, l, o[D]) goes to the workspace.
//   With one split per head (enough heads to give every CU a workgroup) the
//   workgroup writes the f16 output itself; otherwise a second tiny kernel merges
//   the splits in split order.
//
//   Append form (a generation step): instead of a ready query the kernel takes the new
//   token's q, k, v projections, rotates q and k at the token's position (the
//   arithmetic of decode_qkv_kernel: f32, one rounding to f16), writes k and v to cache
//   row L and attends over rows [0, L] -- rows [0, L) streamed from the cache, row L from
//   the registers that hold it, so nothing written by this launch is read back from
//   memory.  One launch per block and step instead of two.
#include "common.h"

namespace deers {

#ifndef DEERS_DEC_ROWS
#define DEERS_DEC_ROWS 4
#endif
constexpr int kDecRowsPerIt = DEERS_DEC_ROWS;  // cache rows in flight per lane group

// Fewer, longer streams measure faster than many short ones (each workgroup pays a
// start-up and a reduction): split a head only until every CU has a workgroup.
int decode_pick_splits(int64_t BH, int64_t L, int* chunk) {
  int splits = 1;
  while (BH * splits < 256 && L / (splits * 2) >= 256) splits *= 2;
  int64_t c = (L + splits - 1) / splits;
  c = (c + 63) / 64 * 64;
  *chunk = (int)c;
  return splits;
}

// The thread's 8 columns (8*part ..) of rotate_half RoPE applied to one [D] row: columns
// below D/2 are x1*cos + x2*sin, the others x2*cos - x1*sin, with x1 / x2 the lower /
// upper half's elements of the same index (src/models/gpt.rs:49-73).
template <int D>
__device__ __forceinline__ half8 rotate_row(const half_t* row, const half_t* cos_row, const half_t* sin_row,
                                            int part) {
  constexpr int HALF = D / 2;
  const int col = 8 * part;
  const bool upper = col >= HALF;
  const int c = upper ? col - HALF : col;
  const half8 a1 = *(const half8*)(row + c), a2 = *(const half8*)(row + c + HALF);
  const half8 cs = *(const half8*)(cos_row + c), sn = *(const half8*)(sin_row + c);
  half8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float x1 = (float)a1[e], x2 = (float)a2[e], co = (float)cs[e], si = (float)sn[e];
    out[e] = upper ? (half_t)(x2 * co - x1 * si) : (half_t)(x1 * co + x2 * si);
  }
  return out;
}

template <int D, bool APPEND>
__global__ __launch_bounds__(256) void attn_decode_f16_kernel(DecodeParams p) {
  constexpr int LPR = D / 8;        // lanes per cache row
  constexpr int GROUPS = 256 / LPR; // row groups per workgroup
  __shared__ float red_m[GROUPS];
  __shared__ float red_l[GROUPS];
  __shared__ float red_o[GROUPS * D];

  const int tid = threadIdx.x;
  const int part = tid % LPR;
  const int grp = tid / LPR;
  const int split = blockIdx.x;
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh % p.H;

  const half_t* K = (const half_t*)p.k + b * p.skb + h * p.skh + 8 * part;
  const half_t* V = (const half_t*)p.v + b * p.skb + h * p.skh + 8 * part;
  half8 qh;
  half8 k_new = {0, 0, 0, 0, 0, 0, 0, 0}, v_new = {0, 0, 0, 0, 0, 0, 0, 0};
  // the new row is handled by one lane group of the last split
  const bool owns_new_row = APPEND && grp == 0 && split == p.splits - 1;
  if constexpr (APPEND) {
    const int64_t in_off = b * p.in_b + h * p.in_h;
    qh = rotate_row<D>((const half_t*)p.q_in + in_off, (const half_t*)p.cos_row, (const half_t*)p.sin_row, part);
    if (owns_new_row) {
      k_new = rotate_row<D>((const half_t*)p.k_in + in_off, (const half_t*)p.cos_row, (const half_t*)p.sin_row, part);
      v_new = *(const half8*)((const half_t*)p.v_in + in_off + 8 * part);
      *(half8*)(const_cast<half_t*>(K) + (int64_t)p.L * p.skl) = k_new;
      *(half8*)(const_cast<half_t*>(V) + (int64_t)p.L * p.skl) = v_new;
    }
  } else {
    qh = *(const half8*)((const half_t*)p.q + (int64_t)bh * D + 8 * part);
  }
  float qf[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) qf[e] = (float)qh[e] * p.scale_log2;

  const int row_begin = split * p.chunk;
  int row_end = row_begin + p.chunk;
  if (row_end > p.L) row_end = p.L;

  float m = -INFINITY, l = 0.f;
  float o[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = 0.f;

  for (int r0 = row_begin + grp; r0 < row_end; r0 += GROUPS * kDecRowsPerIt) {
    half8 kk[kDecRowsPerIt], vv[kDecRowsPerIt];
#pragma unroll
    for (int u = 0; u < kDecRowsPerIt; ++u) {
      const int row = r0 + u * GROUPS;
      if (row < row_end) {
        // every cache byte is used once: non-temporal loads keep the stream from
        // displacing itself in the caches and measurably raise the achieved HBM rate
        kk[u] = __builtin_nontemporal_load((const half8*)(K + (int64_t)row * p.skl));
        vv[u] = __builtin_nontemporal_load((const half8*)(V + (int64_t)row * p.skl));
      } else {
        kk[u] = half8{0, 0, 0, 0, 0, 0, 0, 0};
        vv[u] = half8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    float s[kDecRowsPerIt];
#pragma unroll
    for (int u = 0; u < kDecRowsPerIt; ++u) {
      float acc = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc += qf[e] * (float)kk[u][e];
#pragma unroll
      for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
      s[u] = (r0 + u * GROUPS < row_end) ? acc : -INFINITY;
    }
    float mloc = s[0];
#pragma unroll
    for (int u = 1; u < kDecRowsPerIt; ++u) mloc = fmaxf(mloc, s[u]);
    const float m_new = fmaxf(m, mloc);  // finite: row r0 itself is always valid
    const float alpha = fast_exp2(m - m_new);
    l *= alpha;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] *= alpha;
#pragma unroll
    for (int u = 0; u < kDecRowsPerIt; ++u) {
      const float pu = fast_exp2(s[u] - m_new);
      l += pu;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] += pu * (float)vv[u][e];
    }
    m = m_new;
  }

  if (owns_new_row) {  // row L from registers (a whole lane group takes this branch)
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += qf[e] * (float)k_new[e];
#pragma unroll
    for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
    const float m_new = fmaxf(m, acc);
    const float alpha = fast_exp2(m - m_new);  // 0 when no cached row was seen (m = -inf)
    const float pu = fast_exp2(acc - m_new);
    l = l * alpha + pu;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = o[e] * alpha + pu * (float)v_new[e];
    m = m_new;
  }

  // ---- merge the row groups of this workgroup (fixed order) ----
  if (part == 0) {
    red_m[grp] = m;
    red_l[grp] = l;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red_o[grp * D + 8 * part + e] = o[e];
  __syncthreads();
  float M = -INFINITY, lsum = 0.f, osum = 0.f;
  if (tid < D) {
    for (int gi = 0; gi < GROUPS; ++gi) M = fmaxf(M, red_m[gi]);
    for (int gi = 0; gi < GROUPS; ++gi) {
      const float mg = red_m[gi];
      const float w = (mg == -INFINITY) ? 0.f : fast_exp2(mg - M);
      lsum += w * red_l[gi];
      osum += w * red_o[gi * D + tid];
    }
  }
  if (p.splits == 1) {  // nothing to merge
    if (tid < D) ((half_t*)p.o)[(int64_t)bh * D + tid] = (half_t)(osum / lsum);
    return;
  }
  if (tid < D) {
    const int64_t slot = (int64_t)bh * p.splits + split;
    p.part_o[slot * D + tid] = osum;
    if (tid == 0) {
      p.part_ml[slot * 2 + 0] = M;
      p.part_ml[slot * 2 + 1] = lsum;
    }
  }
}

// Merges the split partials of a head in split order and writes the f16 output.
// (A merge by the last split to arrive inside the main kernel was tried: the
// device-scope fences it needs cost several times the whole stream.)
template <int D>
__global__ __launch_bounds__(D) void attn_decode_merge_kernel(DecodeParams p) {
  const int bh = blockIdx.x;
  const int d = threadIdx.x;
  float M = -INFINITY;
  for (int s = 0; s < p.splits; ++s) M = fmaxf(M, p.part_ml[((int64_t)bh * p.splits + s) * 2]);
  float lsum = 0.f, osum = 0.f;
  for (int s = 0; s < p.splits; ++s) {
    const int64_t slot = (int64_t)bh * p.splits + s;
    const float ms = p.part_ml[slot * 2];
    const float w = (ms == -INFINITY) ? 0.f : fast_exp2(ms - M);
    lsum += w * p.part_ml[slot * 2 + 1];
    osum += w * p.part_o[slot * D + d];
  }
  ((half_t*)p.o)[(int64_t)bh * D + d] = (half_t)(osum / lsum);
}

void launch_attn_decode_f16(const DecodeParams& p, int B, int D, bool append, hipStream_t stream) {
  dim3 grid(p.splits, B * p.H);
  {
    LaunchScope scope(append ? "attn_decode_append_f16" : "attn_decode_f16", stream);
#define DEERS_DECODE_CASE(DD, APP) \
  if (D == DD && append == APP) hipLaunchKernelGGL((attn_decode_f16_kernel<DD, APP>), grid, dim3(256), 0, stream, p);
    DEERS_DECODE_CASE(32, false)
    DEERS_DECODE_CASE(32, true)
    DEERS_DECODE_CASE(64, false)
    DEERS_DECODE_CASE(64, true)
    DEERS_DECODE_CASE(128, false)
    DEERS_DECODE_CASE(128, true)
#undef DEERS_DECODE_CASE
  }
  if (p.splits > 1) {
    LaunchScope scope("attn_decode_merge", stream);
    if (D == 32)
      hipLaunchKernelGGL(attn_decode_merge_kernel<32>, dim3(B * p.H), dim3(32), 0, stream, p);
    else if (D == 64)
      hipLaunchKernelGGL(attn_decode_merge_kernel<64>, dim3(B * p.H), dim3(64), 0, stream, p);
    else
      hipLaunchKernelGGL(attn_decode_merge_kernel<128>, dim3(B * p.H), dim3(128), 0, stream, p);
  }
}

}  // namespace deers
