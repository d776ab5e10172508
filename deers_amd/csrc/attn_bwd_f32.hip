// Fused causal attention backward, f32 storage and arithmetic, gfx950.
//
// Same three launches and orientations as the f16 backward (delta, dK/dV with
// one key column per lane, dQ with one query column per lane) on
// v_mfma_f32_32x32x2_f32.  One contraction element per lane per MFMA means the
// accumulator registers of P / dS are B operands as they are, and the
// "transposed" A fragments are ordinary 4-byte reads of the row-major LDS tiles.
// Contraction over D gives lane group g the contiguous half [g*D/2, (g+1)*D/2).
#include "common.h"
#include "bwd_delta.h"

namespace deers {

constexpr int kBwd32Blk = 128;

#define ZERO16 floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#define ZEROF4 floatx4{0, 0, 0, 0}

template <int D, int STEP>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_f32_kernel(BwdParams p, int BH, int n_blocks,
                                                                int heads_per_xcd) {
  constexpr int LD = D + 4;
  constexpr int KH = D / 2;
  constexpr int DB = D / 32;
  constexpr int MB = STEP / 32;
  constexpr int CH = D / 4;
  constexpr int NLOAD = STEP * CH / 256;

  __shared__ __attribute__((aligned(16))) float Qs[STEP * LD];
  __shared__ __attribute__((aligned(16))) float dOs[STEP * LD];
  __shared__ __attribute__((aligned(16))) float lse2s[STEP];
  __shared__ __attribute__((aligned(16))) float deltas[STEP];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int T = p.T;
  // every block of a head on one XCD, each XCD's list longest first: the first key
  // block is seen by every query block
  int bh, rank;
  if (!map_block(blockIdx.x, n_blocks, heads_per_xcd, BH, &bh, &rank)) return;
  const int kvblk = rank;
  const int b = bh / p.H, h = bh % p.H;

  const float* Q = (const float*)p.q + b * p.sq.b + h * p.sq.h;
  const float* K = (const float*)p.k + b * p.sk.b + h * p.sk.h;
  const float* V = (const float*)p.v + b * p.sv.b + h * p.sv.h;
  const float* dO = (const float*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  float* dK = (float*)p.dk + b * p.sdk.b + h * p.sdk.h;
  float* dV = (float*)p.dv + b * p.sdv.b + h * p.sdv.h;
  const float* lse = p.lse + (int64_t)bh * T;
  const float* delta = p.delta + (int64_t)bh * T;

  const int kv0 = kvblk * kBwd32Blk;
  const int kvw0 = kv0 + 32 * wave;
  const int kvrow = kvw0 + (lane & 31);

  float kf[KH], vf[KH];
#pragma unroll
  for (int c = 0; c < KH / 4; ++c) {
    floatx4 tk = ZEROF4, tv = ZEROF4;
    if (kvrow < T) {
      tk = *(const floatx4*)(K + (int64_t)kvrow * p.sk.t + g * KH + 4 * c);
      tv = *(const floatx4*)(V + (int64_t)kvrow * p.sv.t + g * KH + 4 * c);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      kf[4 * c + e] = tk[e];
      vf[4 * c + e] = tv[e];
    }
  }

  floatx16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    dkacc[i] = ZERO16;
    dvacc[i] = ZERO16;
  }

  const int first_tile = kv0 / STEP;
  const int n_tiles = (T + STEP - 1) / STEP;

  floatx4 qreg[NLOAD], doreg[NLOAD];
  float lreg = 0.f, dreg = 0.f;
  auto prefetch = [&](int tile) {
    const int q0 = tile * STEP;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int qr = q0 + row;
      if (qr < T) {
        qreg[i] = *(const floatx4*)(Q + (int64_t)qr * p.sq.t + 4 * ch);
        doreg[i] = *(const floatx4*)(dO + (int64_t)qr * p.sdo.t + 4 * ch);
      } else {
        qreg[i] = ZEROF4;
        doreg[i] = ZEROF4;
      }
    }
    if (tid < STEP) {
      const int qr = q0 + tid;
      lreg = qr < T ? lse[qr] * kLog2e : 0.f;
      dreg = qr < T ? delta[qr] : 0.f;
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      *(floatx4*)(Qs + row * LD + 4 * ch) = qreg[i];
      *(floatx4*)(dOs + row * LD + 4 * ch) = doreg[i];
    }
    if (tid < STEP) {
      lse2s[tid] = lreg;
      deltas[tid] = dreg;
    }
  };

  if (first_tile < n_tiles) prefetch(first_tile);
  for (int j = first_tile; j < n_tiles; ++j) {
    __syncthreads();
    commit();
    __syncthreads();
    if (j + 1 < n_tiles) prefetch(j + 1);

    const int q0 = j * STEP;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int qb0 = q0 + 32 * mb;
      if (qb0 + 31 < kvw0) continue;

      floatx16 s = ZERO16, dp = ZERO16;
      const float* qrow_p = Qs + (32 * mb + (lane & 31)) * LD + g * KH;
      const float* dorow_p = dOs + (32 * mb + (lane & 31)) * LD + g * KH;
#pragma unroll
      for (int c = 0; c < KH / 4; ++c) {
        const floatx4 a = *(const floatx4*)(qrow_p + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) s = mfma_f32(a[e], kf[4 * c + e], s);
      }
#pragma unroll
      for (int c = 0; c < KH / 4; ++c) {
        const floatx4 a = *(const floatx4*)(dorow_p + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) dp = mfma_f32(a[e], vf[4 * c + e], dp);
      }

      const bool need_mask = (qb0 < kvw0 + 31);
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const floatx4 l4 = *(const floatx4*)(lse2s + 32 * mb + 8 * rq + 4 * g);
        const floatx4 d4 = *(const floatx4*)(deltas + 32 * mb + 8 * rq + 4 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * rq + e;
          float pv = fast_exp2(s[r] * p.scale_log2 - l4[e]);
          if (need_mask) {
            const int qr = qb0 + 8 * rq + 4 * g + e;
            if (kvrow > qr) pv = 0.f;
          }
          s[r] = pv;
          dp[r] = pv * (dp[r] - d4[e]);
        }
      }

#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const float ado = dOs[row * LD + 32 * db + (lane & 31)];
          dvacc[db] = mfma_f32(ado, s[r], dvacc[db]);
          const float aq = Qs[row * LD + 32 * db + (lane & 31)];
          dkacc[db] = mfma_f32(aq, dp[r], dkacc[db]);
        }
      }
    }
  }

  if (kvrow < T) {
    float* dkrow = dK + (int64_t)kvrow * p.sdk.t;
    float* dvrow = dV + (int64_t)kvrow * p.sdv.t;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        floatx4 ok, ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ok[e] = dkacc[db][4 * rq + e] * p.scale;
          ov[e] = dvacc[db][4 * rq + e];
        }
        *(floatx4*)(dkrow + 32 * db + 8 * rq + 4 * g) = ok;
        *(floatx4*)(dvrow + 32 * db + 8 * rq + 4 * g) = ov;
      }
  }
}

template <int D, int STEP>
__global__ __launch_bounds__(256) void attn_bwd_dq_f32_kernel(BwdParams p, int BH, int n_blocks,
                                                              int heads_per_xcd) {
  constexpr int LD = D + 4;
  constexpr int KH = D / 2;
  constexpr int DB = D / 32;
  constexpr int MB = STEP / 32;
  constexpr int CH = D / 4;
  constexpr int NLOAD = STEP * CH / 256;

  __shared__ __attribute__((aligned(16))) float Ks[STEP * LD];
  __shared__ __attribute__((aligned(16))) float Vs[STEP * LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int T = p.T;
  int bh, rank;
  if (!map_block(blockIdx.x, n_blocks, heads_per_xcd, BH, &bh, &rank)) return;
  const int qtile = n_blocks - 1 - rank;  // the last query block sees every key block
  const int b = bh / p.H, h = bh % p.H;

  const float* Q = (const float*)p.q + b * p.sq.b + h * p.sq.h;
  const float* K = (const float*)p.k + b * p.sk.b + h * p.sk.h;
  const float* V = (const float*)p.v + b * p.sv.b + h * p.sv.h;
  const float* dO = (const float*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  float* dQ = (float*)p.dq + b * p.sdq.b + h * p.sdq.h;

  const int q0 = qtile * kBwd32Blk;
  const int qw0 = q0 + 32 * wave;
  const int qrow = qw0 + (lane & 31);

  float qf[KH], dof[KH];
#pragma unroll
  for (int c = 0; c < KH / 4; ++c) {
    floatx4 tq = ZEROF4, td = ZEROF4;
    if (qrow < T) {
      tq = *(const floatx4*)(Q + (int64_t)qrow * p.sq.t + g * KH + 4 * c);
      td = *(const floatx4*)(dO + (int64_t)qrow * p.sdo.t + g * KH + 4 * c);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      qf[4 * c + e] = tq[e];
      dof[4 * c + e] = td[e];
    }
  }
  const float lse2 = qrow < T ? p.lse[(int64_t)bh * T + qrow] * kLog2e : 0.f;
  const float dlt = qrow < T ? p.delta[(int64_t)bh * T + qrow] : 0.f;

  floatx16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) dqacc[i] = ZERO16;

  int last_q = q0 + kBwd32Blk - 1;
  if (last_q > T - 1) last_q = T - 1;
  const int n_tiles = last_q / STEP + 1;

  floatx4 kreg[NLOAD], vreg[NLOAD];
  auto prefetch = [&](int tile) {
    const int kv0 = tile * STEP;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int kv = kv0 + row;
      if (kv < T) {
        kreg[i] = *(const floatx4*)(K + (int64_t)kv * p.sk.t + 4 * ch);
        vreg[i] = *(const floatx4*)(V + (int64_t)kv * p.sv.t + 4 * ch);
      } else {
        kreg[i] = ZEROF4;
        vreg[i] = ZEROF4;
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

    const int kv0 = j * STEP;
    if (kv0 > qw0 + 31) continue;

#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int kvb0 = kv0 + 32 * mb;
      if (kvb0 > qw0 + 31) continue;

      floatx16 s = ZERO16, dp = ZERO16;
      const float* krow_p = Ks + (32 * mb + (lane & 31)) * LD + g * KH;
      const float* vrow_p = Vs + (32 * mb + (lane & 31)) * LD + g * KH;
#pragma unroll
      for (int c = 0; c < KH / 4; ++c) {
        const floatx4 a = *(const floatx4*)(krow_p + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) s = mfma_f32(a[e], qf[4 * c + e], s);
      }
#pragma unroll
      for (int c = 0; c < KH / 4; ++c) {
        const floatx4 a = *(const floatx4*)(vrow_p + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) dp = mfma_f32(a[e], dof[4 * c + e], dp);
      }

      const bool need_mask = (kvb0 + 31 > qw0);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float pv = fast_exp2(s[r] * p.scale_log2 - lse2);
        if (need_mask) {
          const int kv = kvb0 + 8 * (r >> 2) + 4 * g + (r & 3);
          if (kv > qrow) pv = 0.f;
        }
        dp[r] = pv * (dp[r] - dlt);
      }

#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 32 * mb + 8 * (r >> 2) + 4 * g + (r & 3);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const float ak = Ks[row * LD + 32 * db + (lane & 31)];
          dqacc[db] = mfma_f32(ak, dp[r], dqacc[db]);
        }
      }
    }
  }

  if (qrow < T) {
    float* dqrow = dQ + (int64_t)qrow * p.sdq.t;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        floatx4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = dqacc[db][4 * rq + e] * p.scale;
        *(floatx4*)(dqrow + 32 * db + 8 * rq + 4 * g) = out;
      }
  }
}

template <int D, int STEP>
static void launch_bwd_f32_d(const BwdParams& p, int B, hipStream_t stream) {
  const int64_t rows = (int64_t)B * p.H * p.T;
  constexpr int LPR = D / 4;
  const int64_t threads = rows * LPR;
  {
    LaunchScope scope("attn_bwd_delta", stream);
    hipLaunchKernelGGL((attn_bwd_delta_kernel<float, D>), dim3((threads + 255) / 256), dim3(256),
                       0, stream, p, B);
  }
  const int BH = B * p.H;
  const int n_blocks = (p.T + kBwd32Blk - 1) / kBwd32Blk;
  const int heads_per_xcd = (BH + 7) / 8;
  const dim3 grid(8 * n_blocks * heads_per_xcd);
  {
    LaunchScope scope("attn_bwd_dkdv_f32", stream);
    hipLaunchKernelGGL((attn_bwd_dkdv_f32_kernel<D, STEP>), grid, dim3(256), 0, stream, p, BH,
                       n_blocks, heads_per_xcd);
  }
  {
    LaunchScope scope("attn_bwd_dq_f32", stream);
    hipLaunchKernelGGL((attn_bwd_dq_f32_kernel<D, STEP>), grid, dim3(256), 0, stream, p, BH,
                       n_blocks, heads_per_xcd);
  }
}

void launch_attn_bwd_f32(const BwdParams& p, int B, int D, hipStream_t stream) {
  switch (D) {
    case 32: launch_bwd_f32_d<32, 64>(p, B, stream); break;
    case 64: launch_bwd_f32_d<64, 64>(p, B, stream); break;
    case 128: launch_bwd_f32_d<128, 32>(p, B, stream); break;
  }
}

}  // namespace deers
