// Fused causal attention backward, f16 storage / f32 accumulate, gfx950.
//
// Replaces the reference's op-by-op autograd sweep over the attention core
// (src/backprop.rs:52-66 through src/ops.rs:1089-1101, 422-425, 210-214,
// 777-799, 1162-1175, 638-643) by recomputation from (Q, K, V, O, LSE, dO):
//     P  = exp(S*scale + mask - LSE)        dV = P^T dO
//     dP = dO V^T                           dS = P o (dP - delta),  delta = rowsum(dO o O)
//     dQ = scale dS K                       dK = scale dS^T Q
//
// Three launches, no atomics, bit-reproducible:
//   1. delta   : delta[b,h,t] = sum_d dO*O (f32).
//   2. dK/dV   : a workgroup owns 128 key rows (32 per wave, K^T and V^T held in
//                registers as B operands) and walks the query tiles at or below
//                the diagonal.  Orientation S[q,kv] (one key column per lane) so P
//                and dS leave the accumulators directly as B operands of
//                dV^T += dO^T P and dK^T += Q^T dS; dO^T / Q^T fragments come
//                from the row-major LDS tiles via ds_read_b64_tr_b16.
//   3. dQ      : a workgroup owns 128 query rows (32 per wave, Q and dO in
//                registers) and walks key tiles up to the diagonal.  Orientation
//                S^T[kv,q] (one query column per lane, LSE and delta are per-lane
//                scalars); dS^T leaves the accumulators as the B operand of
//                dQ^T += K^T dS^T with K^T fragments read transposed from LDS.
// Recomputing S and dP in both 2 and 3 costs 7 tile GEMMs instead of 5 but
// keeps every product in registers and needs no dQ accumulation buffer.
#include "common.h"
#include "bwd_delta.h"

namespace deers {

constexpr int kBwdBlk = 128;  // rows owned by a workgroup (keys in dK/dV, queries in dQ)
constexpr int kBwdStep = 64;  // rows of the streamed operand per iteration

#define ZERO16 floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#define ZEROH8 half8{0, 0, 0, 0, 0, 0, 0, 0}

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dkdv_f16_kernel(BwdParams p) {
  constexpr int LD = D + 8;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int CH = D / 8;
  constexpr int NLOAD = kBwdStep * CH / 256;

  __shared__ __attribute__((aligned(16))) half_t Qs[kBwdStep * LD];
  __shared__ __attribute__((aligned(16))) half_t dOs[kBwdStep * LD];
  __shared__ __attribute__((aligned(16))) float lse2s[kBwdStep];
  __shared__ __attribute__((aligned(16))) float deltas[kBwdStep];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int T = p.T;
  const int kvblk = blockIdx.x;  // block 0 walks the most query tiles: it goes first
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  const half_t* dO = (const half_t*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  half_t* dK = (half_t*)p.dk + b * p.sdk.b + h * p.sdk.h;
  half_t* dV = (half_t*)p.dv + b * p.sdv.b + h * p.sdv.h;
  const float* lse = p.lse + (int64_t)bh * T;
  const float* delta = p.delta + (int64_t)bh * T;

  const int kv0 = kvblk * kBwdBlk;
  const int kvw0 = kv0 + 32 * wave;
  const int kvrow = kvw0 + (lane & 31);

  // K^T and V^T as B operands: lane holds row kvrow, halfs 16ks+8g .. +7.
  half8 kf[KS], vf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (kvrow < T) {
      kf[ks] = *(const half8*)(K + (int64_t)kvrow * p.sk.t + 16 * ks + 8 * g);
      vf[ks] = *(const half8*)(V + (int64_t)kvrow * p.sv.t + 16 * ks + 8 * g);
    } else {
      kf[ks] = ZEROH8;
      vf[ks] = ZEROH8;
    }
  }

  floatx16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    dkacc[i] = ZERO16;
    dvacc[i] = ZERO16;
  }

  const int first_tile = kv0 / kBwdStep;
  const int n_tiles = (T + kBwdStep - 1) / kBwdStep;

  half8 qreg[NLOAD], doreg[NLOAD];
  float lreg = 0.f, dreg = 0.f;
  auto prefetch = [&](int tile) {
    const int q0 = tile * kBwdStep;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int qr = q0 + row;
      if (qr < T) {
        qreg[i] = *(const half8*)(Q + (int64_t)qr * p.sq.t + 8 * ch);
        doreg[i] = *(const half8*)(dO + (int64_t)qr * p.sdo.t + 8 * ch);
      } else {
        qreg[i] = ZEROH8;
        doreg[i] = ZEROH8;
      }
    }
    if (tid < kBwdStep) {
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
      *(half8*)(Qs + row * LD + 8 * ch) = qreg[i];
      *(half8*)(dOs + row * LD + 8 * ch) = doreg[i];
    }
    if (tid < kBwdStep) {
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

    const int q0 = j * kBwdStep;
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int qb0 = q0 + 32 * mb;        // first query row of this 32-block
      if (qb0 + 31 < kvw0) continue;       // every query here precedes the wave's keys

      // S[q, kv] and dP[q, kv]
      floatx16 s = ZERO16, dp = ZERO16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8 aq = *(const half8*)(Qs + (32 * mb + (lane & 31)) * LD + 16 * ks + 8 * g);
        s = mfma_f16(aq, kf[ks], s);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8 ad = *(const half8*)(dOs + (32 * mb + (lane & 31)) * LD + 16 * ks + 8 * g);
        dp = mfma_f16(ad, vf[ks], dp);
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
      for (int st = 0; st < 2; ++st) {
        const half8 pf = pack_half8(s[8 * st + 0], s[8 * st + 1], s[8 * st + 2], s[8 * st + 3],
                                    s[8 * st + 4], s[8 * st + 5], s[8 * st + 6], s[8 * st + 7]);
        const half8 dsf =
            pack_half8(dp[8 * st + 0], dp[8 * st + 1], dp[8 * st + 2], dp[8 * st + 3],
                       dp[8 * st + 4], dp[8 * st + 5], dp[8 * st + 6], dp[8 * st + 7]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const half8 dot = lds_frag_transposed(dOs, LD, 32 * mb + 16 * st, 32 * db, lane);
          dvacc[db] = mfma_f16(dot, pf, dvacc[db]);
          const half8 qt = lds_frag_transposed(Qs, LD, 32 * mb + 16 * st, 32 * db, lane);
          dkacc[db] = mfma_f16(qt, dsf, dkacc[db]);
        }
      }
    }
  }

  if (kvrow < T) {
    half_t* dkrow = dK + (int64_t)kvrow * p.sdk.t;
    half_t* dvrow = dV + (int64_t)kvrow * p.sdv.t;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        half4 ok, ov;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ok[e] = (half_t)(dkacc[db][4 * rq + e] * p.scale);
          ov[e] = (half_t)(dvacc[db][4 * rq + e]);
        }
        *(half4*)(dkrow + 32 * db + 8 * rq + 4 * g) = ok;
        *(half4*)(dvrow + 32 * db + 8 * rq + 4 * g) = ov;
      }
  }
}

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
template <int D>
__global__ __launch_bounds__(256) void attn_bwd_dq_f16_kernel(BwdParams p) {
  constexpr int LD = D + 8;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int CH = D / 8;
  constexpr int NLOAD = kBwdStep * CH / 256;

  __shared__ __attribute__((aligned(16))) half_t Ks[kBwdStep * LD];
  __shared__ __attribute__((aligned(16))) half_t Vs[kBwdStep * LD];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 5;
  const int T = p.T;
  const int qtile = gridDim.x - 1 - blockIdx.x;  // longest rows first
  const int bh = blockIdx.y;
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  const half_t* dO = (const half_t*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  half_t* dQ = (half_t*)p.dq + b * p.sdq.b + h * p.sdq.h;

  const int q0 = qtile * kBwdBlk;
  const int qw0 = q0 + 32 * wave;
  const int qrow = qw0 + (lane & 31);

  half8 qf[KS], dof[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (qrow < T) {
      qf[ks] = *(const half8*)(Q + (int64_t)qrow * p.sq.t + 16 * ks + 8 * g);
      dof[ks] = *(const half8*)(dO + (int64_t)qrow * p.sdo.t + 16 * ks + 8 * g);
    } else {
      qf[ks] = ZEROH8;
      dof[ks] = ZEROH8;
    }
  }
  const float lse2 = qrow < T ? p.lse[(int64_t)bh * T + qrow] * kLog2e : 0.f;
  const float dlt = qrow < T ? p.delta[(int64_t)bh * T + qrow] : 0.f;

  floatx16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) dqacc[i] = ZERO16;

  int last_q = q0 + kBwdBlk - 1;
  if (last_q > T - 1) last_q = T - 1;
  const int n_tiles = last_q / kBwdStep + 1;

  half8 kreg[NLOAD], vreg[NLOAD];
  auto prefetch = [&](int tile) {
    const int kv0 = tile * kBwdStep;
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      const int idx = tid + 256 * i;
      const int row = idx / CH, ch = idx % CH;
      const int kv = kv0 + row;
      if (kv < T) {
        kreg[i] = *(const half8*)(K + (int64_t)kv * p.sk.t + 8 * ch);
        vreg[i] = *(const half8*)(V + (int64_t)kv * p.sv.t + 8 * ch);
      } else {
        kreg[i] = ZEROH8;
        vreg[i] = ZEROH8;
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

    const int kv0 = j * kBwdStep;
    if (kv0 > qw0 + 31) continue;

#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
      const int kvb0 = kv0 + 32 * mb;
      if (kvb0 > qw0 + 31) continue;

      floatx16 s = ZERO16, dp = ZERO16;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8 ak = *(const half8*)(Ks + (32 * mb + (lane & 31)) * LD + 16 * ks + 8 * g);
        s = mfma_f16(ak, qf[ks], s);
      }
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8 av = *(const half8*)(Vs + (32 * mb + (lane & 31)) * LD + 16 * ks + 8 * g);
        dp = mfma_f16(av, dof[ks], dp);
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
      for (int st = 0; st < 2; ++st) {
        const half8 dsf =
            pack_half8(dp[8 * st + 0], dp[8 * st + 1], dp[8 * st + 2], dp[8 * st + 3],
                       dp[8 * st + 4], dp[8 * st + 5], dp[8 * st + 6], dp[8 * st + 7]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const half8 kt = lds_frag_transposed(Ks, LD, 32 * mb + 16 * st, 32 * db, lane);
          dqacc[db] = mfma_f16(kt, dsf, dqacc[db]);
        }
      }
    }
  }

  if (qrow < T) {
    half_t* dqrow = dQ + (int64_t)qrow * p.sdq.t;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        half4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = (half_t)(dqacc[db][4 * rq + e] * p.scale);
        *(half4*)(dqrow + 32 * db + 8 * rq + 4 * g) = out;
      }
  }
}

template <int D>
static void launch_bwd_f16_d(const BwdParams& p, int B, hipStream_t stream) {
  const int64_t rows = (int64_t)B * p.H * p.T;
  constexpr int LPR = D / 8;
  const int64_t threads = rows * LPR;
  {
    LaunchScope scope("attn_bwd_delta", stream);
    hipLaunchKernelGGL((attn_bwd_delta_kernel<half_t, D>), dim3((threads + 255) / 256),
                       dim3(256), 0, stream, p, B);
  }
  dim3 grid((p.T + kBwdBlk - 1) / kBwdBlk, B * p.H);
  {
    LaunchScope scope("attn_bwd_dkdv_f16", stream);
    hipLaunchKernelGGL(attn_bwd_dkdv_f16_kernel<D>, grid, dim3(256), 0, stream, p);
  }
  {
    LaunchScope scope("attn_bwd_dq_f16", stream);
    hipLaunchKernelGGL(attn_bwd_dq_f16_kernel<D>, grid, dim3(256), 0, stream, p);
  }
}

void launch_attn_bwd_f16(const BwdParams& p, int B, int D, hipStream_t stream) {
  switch (D) {
    case 32: launch_bwd_f16_d<32>(p, B, stream); break;
    case 64: launch_bwd_f16_d<64>(p, B, stream); break;
    case 128: launch_bwd_f16_d<128>(p, B, stream); break;
  }
}

}  // namespace deers
