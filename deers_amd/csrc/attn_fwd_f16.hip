// Fused causal attention forward, f16 storage / f32 accumulate, gfx950.
//
// Replaces the op chain of src/models/gpt.rs:139-144 (matmul, scalar_mul,
// causal_mask + add, log_sum_exp, sub, exp, matmul) with one kernel that never
// materialises the [T,T] score tensor.
//
// Work decomposition
//   grid  = (ceil(T/128), B*H); 256 threads = 4 waves; wave w owns query rows
//           [q0 + 32w, q0 + 32w + 32) of the workgroup's 128-row tile.
//   loop  over key/value tiles of 64 rows, stopping at the diagonal (tile-level
//           causal skip); only tiles that straddle the diagonal apply the
//           element mask.
//   S^T   = K Q^T on v_mfma_f32_32x32x16_f16 (K tile row-major in LDS as the A
//           operand, the wave's Q rows held in registers as the B operand).  In
//           this orientation every lane owns ONE query column of the 32x32
//           accumulator, so row max / row sum are in-lane reductions plus one
//           exchange with lane+32, and the running rescale of O is a per-lane
//           scalar.
//   O^T  += V^T P^T: P^T is taken straight from the S^T accumulator registers
//           as the B operand; V^T fragments come from the row-major V tile in
//           LDS through ds_read_b64_tr_b16.
//   softmax is the online form in the log2 domain (exp2 of s*scale*log2e - m).
#include "common.h"

namespace deers {

constexpr int kFwdBM = 128;  // query rows per workgroup
constexpr int kFwdBN = 64;   // key/value rows per iteration

template <int D>
__global__ __launch_bounds__(256) void attn_fwd_f16_kernel(FwdParams p) {
  constexpr int LD = D + 8;            // LDS row stride in halfs (16-byte pad)
  constexpr int KS = D / 16;           // contraction steps over D
  constexpr int DB = D / 32;           // 32-wide blocks of D in the output
  constexpr int CH = D / 8;            // 16-byte chunks per row
  constexpr int NLOAD = kFwdBN * CH / 256;  // chunks per thread per tile

  __shared__ __attribute__((aligned(16))) half_t Ks[kFwdBN * LD];
  __shared__ __attribute__((aligned(16))) half_t Vs[kFwdBN * LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int T = p.T;
  const int n_qtiles = gridDim.x;
  const int qtile = n_qtiles - 1 - blockIdx.x;  // longest rows first
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  half_t* O = (half_t*)p.o + b * p.so.b + h * p.so.h;

  const int q0 = qtile * kFwdBM;
  const int qw0 = q0 + 32 * wave;        // first query row of this wave
  const int qrow = qw0 + (lane & 31);    // this lane's query row

  // Q fragments: B operand of S^T = K Q^T, lane holds Q[qrow][16ks + 8g .. +7].
  half8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (qrow < T)
      qf[ks] = *(const half8*)(Q + (int64_t)qrow * p.sq.t + 16 * ks + 8 * g);
    else
      qf[ks] = half8{0, 0, 0, 0, 0, 0, 0, 0};
  }

  floatx16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) oacc[i] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float m = -INFINITY, lsum = 0.f;

  int last_q = q0 + kFwdBM - 1;
  if (last_q > T - 1) last_q = T - 1;
  const int n_tiles = last_q / kFwdBN + 1;

  half8 kreg[NLOAD], vreg[NLOAD];
  auto prefetch = [&](int tile) {
    const int kv0 = tile * kFwdBN;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int kv = kv0 + row;
      if (kv < T) {
        kreg[i] = *(const half8*)(K + (int64_t)kv * p.sk.t + 8 * ch);
        vreg[i] = *(const half8*)(V + (int64_t)kv * p.sv.t + 8 * ch);
      } else {
        kreg[i] = half8{0, 0, 0, 0, 0, 0, 0, 0};
        vreg[i] = half8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      *(half8*)(Ks + row * LD + 8 * ch) = kreg[i];
      *(half8*)(Vs + row * LD + 8 * ch) = vreg[i];
    }
  };

  prefetch(0);
  for (int j = 0; j < n_tiles; ++j) {
    __syncthreads();
    commit();
    __syncthreads();
    if (j + 1 < n_tiles) prefetch(j + 1);

    const int kv0 = j * kFwdBN;
    if (kv0 > qw0 + 31) continue;  // whole tile is in this wave's future

    // ---- S^T[kv, q] for kv in the tile (2 blocks of 32) ----
    floatx16 s[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      s[mb] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        half8 a = *(const half8*)(Ks + (32 * mb + (lane & 31)) * LD + 16 * ks + 8 * g);
        s[mb] = mfma_f16(a, qf[ks], s[mb]);
      }
    }

    // ---- online softmax over this lane's query column ----
    const bool need_mask = (kv0 + kFwdBN - 1 > qw0);
    float mloc = -INFINITY;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float x = s[mb][r] * p.scale_log2;
        if (need_mask) {
          const int kv = kv0 + 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
          if (kv > qrow) x = -INFINITY;
        }
        s[mb][r] = x;
        mloc = fmaxf(mloc, x);
      }
    mloc = fmaxf(mloc, swap32(mloc));
    const float m_new = fmaxf(m, mloc);
    const float alpha = fast_exp2(m - m_new);
    float rsum = 0.f;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = fast_exp2(s[mb][r] - m_new);
        s[mb][r] = e;
        rsum += e;
      }
    rsum += swap32(rsum);
    lsum = lsum * alpha + rsum;
    m = m_new;
#pragma unroll
    for (int db = 0; db < DB; ++db) oacc[db] *= alpha;

    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        const half8 pf = pack_half8(s[mb][8 * st + 0], s[mb][8 * st + 1], s[mb][8 * st + 2],
                                    s[mb][8 * st + 3], s[mb][8 * st + 4], s[mb][8 * st + 5],
                                    s[mb][8 * st + 6], s[mb][8 * st + 7]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const half8 vf = lds_frag_transposed(Vs, LD, 32 * mb + 16 * st, 32 * db, lane);
          oacc[db] = mfma_f16(vf, pf, oacc[db]);
        }
      }
  }

  // ---- epilogue: O = acc / l, LSE = ln(l) + m ln2 ----
  if (qrow < T) {
    const float inv = 1.f / lsum;
    half_t* orow = O + (int64_t)qrow * p.so.t;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        half4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = (half_t)(oacc[db][4 * rq + e] * inv);
        *(half4*)(orow + 32 * db + 8 * rq + 4 * g) = out;
      }
    if (g == 0) p.lse[(int64_t)bh * T + qrow] = (m + fast_log2(lsum)) * kLn2;
  }
}

void launch_attn_fwd_f16(const FwdParams& p, int B, int D, hipStream_t stream) {
  dim3 grid((p.T + kFwdBM - 1) / kFwdBM, B * p.H);
  LaunchScope scope("attn_fwd_f16", stream);
  switch (D) {
    case 32: hipLaunchKernelGGL(attn_fwd_f16_kernel<32>, grid, dim3(256), 0, stream, p); break;
    case 64: hipLaunchKernelGGL(attn_fwd_f16_kernel<64>, grid, dim3(256), 0, stream, p); break;
    case 128: hipLaunchKernelGGL(attn_fwd_f16_kernel<128>, grid, dim3(256), 0, stream, p); break;
  }
}

}  // namespace deers
