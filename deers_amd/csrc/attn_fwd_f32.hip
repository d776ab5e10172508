// Fused causal attention forward, f32 storage and arithmetic, gfx950.
//
// Same decomposition as the f16 kernel (one query column per lane, S^T = K Q^T,
// O^T += V^T P^T, online softmax in the log2 domain) on v_mfma_f32_32x32x2_f32.
// With one contraction element per lane per MFMA there is no transposed-operand
// problem: V^T fragments are plain 4-byte LDS reads of the row-major V tile, and
// P^T accumulator registers are used as B operands without conversion.
// Contraction over D assigns lane group g the contiguous half [g*D/2, (g+1)*D/2)
// so K fragments are 16-byte LDS reads.
#include "common.h"

namespace deers {

constexpr int kFwd32BM = 128;

template <int D, int BN>
__global__ __launch_bounds__(256) void attn_fwd_f32_kernel(FwdParams p, int BH, int n_qtiles,
                                                           int heads_per_xcd) {
  constexpr int LD = D + 4;   // LDS row stride in floats
  constexpr int KH = D / 2;   // contraction steps (2 elements of D per MFMA)
  constexpr int DB = D / 32;
  constexpr int MB = BN / 32;
  constexpr int CH = D / 4;   // 16-byte chunks per row
  constexpr int NLOAD = BN * CH / 256;

  __shared__ __attribute__((aligned(16))) float Ks[BN * LD];
  __shared__ __attribute__((aligned(16))) float Vs[BN * LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int T = p.T;
  // every tile of a head on one XCD, each XCD's list longest first
  int bh, rank;
  if (!map_block(blockIdx.x, n_qtiles, heads_per_xcd, BH, &bh, &rank)) return;
  const int qtile = n_qtiles - 1 - rank;
  const int b = bh / p.H, h = bh % p.H;

  const float* Q = (const float*)p.q + b * p.sq.b + h * p.sq.h;
  const float* K = (const float*)p.k + b * p.sk.b + h * p.sk.h;
  const float* V = (const float*)p.v + b * p.sv.b + h * p.sv.h;
  float* O = (float*)p.o + b * p.so.b + h * p.so.h;

  const int q0 = qtile * kFwd32BM;
  const int qw0 = q0 + 32 * wave;
  const int qrow = qw0 + (lane & 31);

  float qf[KH];
#pragma unroll
  for (int c = 0; c < KH / 4; ++c) {
    floatx4 t = floatx4{0, 0, 0, 0};
    if (qrow < T) t = *(const floatx4*)(Q + (int64_t)qrow * p.sq.t + g * KH + 4 * c);
#pragma unroll
    for (int e = 0; e < 4; ++e) qf[4 * c + e] = t[e];
  }

  floatx16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) oacc[i] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float m = -INFINITY, lsum = 0.f;

  int last_q = q0 + kFwd32BM - 1;
  if (last_q > T - 1) last_q = T - 1;
  const int n_tiles = last_q / BN + 1;

  floatx4 kreg[NLOAD], vreg[NLOAD];
  auto prefetch = [&](int tile) {
    const int kv0 = tile * BN;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int kv = kv0 + row;
      if (kv < T) {
        kreg[i] = *(const floatx4*)(K + (int64_t)kv * p.sk.t + 4 * ch);
        vreg[i] = *(const floatx4*)(V + (int64_t)kv * p.sv.t + 4 * ch);
      } else {
        kreg[i] = floatx4{0, 0, 0, 0};
        vreg[i] = floatx4{0, 0, 0, 0};
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      *(floatx4*)(Ks + row * LD + 4 * ch) = kreg[i];
      *(floatx4*)(Vs + row * LD + 4 * ch) = vreg[i];
    }
  };

  prefetch(0);
  for (int j = 0; j < n_tiles; ++j) {
    __syncthreads();
    commit();
    __syncthreads();
    if (j + 1 < n_tiles) prefetch(j + 1);

    const int kv0 = j * BN;
    if (kv0 > qw0 + 31) continue;

    floatx16 s[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      s[mb] = floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
      const float* krow = Ks + (32 * mb + (lane & 31)) * LD + g * KH;
#pragma unroll
      for (int c = 0; c < KH / 4; ++c) {
        const floatx4 a = *(const floatx4*)(krow + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) s[mb] = mfma_f32(a[e], qf[4 * c + e], s[mb]);
      }
    }

    const bool need_mask = (kv0 + BN - 1 > qw0);
    float mloc = -INFINITY;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
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
    for (int mb = 0; mb < MB; ++mb)
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

#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const float a = Vs[row * LD + 32 * db + (lane & 31)];
          oacc[db] = mfma_f32(a, s[mb][r], oacc[db]);
        }
      }
  }

  if (qrow < T) {
    const float inv = 1.f / lsum;
    float* orow = O + (int64_t)qrow * p.so.t;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        floatx4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = oacc[db][4 * rq + e] * inv;
        *(floatx4*)(orow + 32 * db + 8 * rq + 4 * g) = out;
      }
    if (g == 0) p.lse[(int64_t)bh * T + qrow] = (m + fast_log2(lsum)) * kLn2;
  }
}

void launch_attn_fwd_f32(const FwdParams& p, int B, int D, hipStream_t stream) {
  const int BH = B * p.H;
  const int n_qtiles = (p.T + kFwd32BM - 1) / kFwd32BM;
  const int heads_per_xcd = (BH + 7) / 8;
  const dim3 grid(8 * n_qtiles * heads_per_xcd);
  LaunchScope scope("attn_fwd_f32", stream);
  switch (D) {
    case 32:
      hipLaunchKernelGGL((attn_fwd_f32_kernel<32, 64>), grid, dim3(256), 0, stream, p, BH, n_qtiles,
                         heads_per_xcd);
      break;
    case 64:
      hipLaunchKernelGGL((attn_fwd_f32_kernel<64, 64>), grid, dim3(256), 0, stream, p, BH, n_qtiles,
                         heads_per_xcd);
      break;
    case 128:
      hipLaunchKernelGGL((attn_fwd_f32_kernel<128, 32>), grid, dim3(256), 0, stream, p, BH, n_qtiles,
                         heads_per_xcd);
      break;
  }
}

}  // namespace deers
