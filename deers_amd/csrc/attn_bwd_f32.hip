// Fused causal attention backward, f32 storage and arithmetic, gfx950.
//
// v_mfma_f32_32x32x2_f32 runs at 1/16 of the f16 matrix rate, so these kernels are bound
// by the matrix pipe alone (a 32x32 score block costs 160 MFMAs = ~10 k cycles with 5 tile
// GEMMs; its softmax a few hundred).  Head widths 32 and 64 therefore take the ONE-PASS
// form, 5 tile GEMMs per block instead of the 7 of a dQ pass plus a dK/dV pass:
//   1. prep : delta = rowsum(dO o O) per query row, and dQ cleared.
//   2. main : a workgroup owns 128 keys (32 per wave, K and V rows in registers as B
//             operands) and walks the 32-row query tiles at or below the diagonal:
//             S = Q K^T, dP = dO V^T, P = exp2(S*scale*log2e - lse2), dS = P o (dP - delta),
//             dV^T += dO^T P, dK^T += Q^T dS; scale*dS goes to LDS as [128 keys][32
//             queries], and after a barrier the waves share out
//             dQ[q,d] += (scale dS)[q, 128 keys] K[128 keys, d]
//             (K block resident in LDS) and add their blocks to dQ with no-return f32
//             atomics: 2 k adds per 10 k cycles of MFMA work, far below what the L2
//             atomic units sustain.  (For the f16 kernels, 16x faster per block, the same
//             scheme lost to the atomics.)
//           dQ sums the contributions of up to T/128 key blocks in arrival order: it is
//           reproducible to f32 rounding (~1e-7 relative), not bit for bit; dK and dV are
//           bit-reproducible.
// One contraction element per lane per MFMA means the accumulator registers of P / dS are B
// operands as they are, and the "transposed" A fragments are ordinary 4-byte reads of the
// row-major LDS tiles.  Contraction over D gives lane group g the contiguous half
// [g*D/2, (g+1)*D/2).
// Head width 128 keeps the earlier three launches (delta, dK/dV with one key column per
// lane, dQ with one query column per lane): its K block and exchange tile do not fit LDS
// beside the streamed tiles.
#include <algorithm>
#include <map>
#include <utility>
#include <vector>

#include "common.h"
#include "bwd_delta.h"

// Hooks for a timing harness that includes this file (phase stamps of the one-pass kernel);
// empty in the library.
#ifndef DEERS_PHASE
#define DEERS_PHASE(k)
#define DEERS_PHASE_STATE
#endif

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

// ---------------------------------------------------------------------------
// one-pass form (D = 32, 64)
// ---------------------------------------------------------------------------
// delta[b,h,t] = sum_d dO*O, and what the main kernel adds to with atomics cleared: the dQ
// row, and the dK and dV rows of the key blocks that two work items share (rows < split_rows).
template <int D>
__global__ __launch_bounds__(256) void attn_bwd_prep_f32_kernel(BwdParams p, int B, int split_rows) {
  constexpr int LPR = D / 4;  // lanes per row, 16 bytes each
  const int64_t rows = (int64_t)B * p.H * p.T;
  const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) / LPR;
  const int part = threadIdx.x % LPR;
  float acc = 0.f;
  if (row < rows) {
    const int t = row % p.T;
    const int bh = row / p.T;
    const int b = bh / p.H, h = bh % p.H;
    const float* o = (const float*)p.o + b * p.so.b + h * p.so.h + (int64_t)t * p.so.t + 4 * part;
    const float* d = (const float*)p.d_o + b * p.sdo.b + h * p.sdo.h + (int64_t)t * p.sdo.t + 4 * part;
    const floatx4 ov = *(const floatx4*)o, dv = *(const floatx4*)d;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc += ov[e] * dv[e];
    *(floatx4*)((float*)p.dq + b * p.sdq.b + h * p.sdq.h + (int64_t)t * p.sdq.t + 4 * part) = ZEROF4;
    if (t < split_rows) {
      *(floatx4*)((float*)p.dk + b * p.sdk.b + h * p.sdk.h + (int64_t)t * p.sdk.t + 4 * part) = ZEROF4;
      *(floatx4*)((float*)p.dv + b * p.sdv.b + h * p.sdv.h + (int64_t)t * p.sdv.t + 4 * part) = ZEROF4;
    }
  }
#pragma unroll
  for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (row < rows && part == 0) p.delta[row] = acc;
}

// One workgroup's work in the one-pass kernel: the query tiles [tile_begin, tile_end) (32 rows
// each) of key block kvblk.  `shared`: the block has a second item and both add to dK / dV.
struct Bwd32Item {
  int kvblk, tile_begin, tile_end, shared;
};

template <int D>
struct Fused32Cfg {
  static constexpr int STEP = 32;        // query rows per iteration
  static constexpr int LD = D + 4;       // row pitch of the Q, dO, K tiles (floats)
  static constexpr int LDS_DS = STEP + 4;  // row pitch of the dS^T exchange tile
  static constexpr int kFloats = 2 * STEP * LD + 2 * STEP + kBwd32Blk * LD + kBwd32Blk * LDS_DS;
  static constexpr size_t kLds = kFloats * sizeof(float);
};

// Two workgroups per CU, so that one's barriers, softmax and atomics run under the other's
// MFMAs (414 -> 354 us at 8x12x1024x64; three at D = 32 were slower than two, 234 against
// 218 us).  The bound is needed at D = 64: left free, the compiler spreads into 80
// accumulation registers it has no use for and a CU holds a single workgroup.
template <int D>
__global__ __launch_bounds__(256, 2) void attn_bwd_fused_f32_kernel(
    BwdParams p, int BH, int n_items, int heads_per_xcd, const Bwd32Item* items) {
  using Cfg = Fused32Cfg<D>;
  constexpr int STEP = Cfg::STEP, LD = Cfg::LD, LDS_DS = Cfg::LDS_DS;
  constexpr int KH = D / 2;
  constexpr int DB = D / 32;
  constexpr int CH = D / 4;
  constexpr int NLOAD = STEP * CH / 256;       // 16-byte loads per thread per streamed tile
  constexpr int NKLOAD = kBwd32Blk * CH / 256;  // ... for the resident K block
  // dQ tile of an iteration: 32 queries x D = DB blocks of 32x32, shared out over the four
  // waves: wave w takes block w % DB over the keys [KPW * (w / DB), + KPW)
  constexpr int KV_SPLIT = 4 / DB;
  constexpr int KPW = kBwd32Blk / KV_SPLIT;
  static_assert(NLOAD >= 1 && DB >= 1 && DB <= 2, "head width 32 or 64");

  extern __shared__ __attribute__((aligned(16))) float smem32[];
  float* Qs = smem32;
  float* dOs = Qs + STEP * LD;
  float* lse2s = dOs + STEP * LD;
  float* deltas = lse2s + STEP;
  float* Ks = deltas + STEP;           // the workgroup's 128 K rows, for dQ = dS K
  float* dSs = Ks + kBwd32Blk * LD;    // scale * dS^T of the current tile: [128 keys][32 queries]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;
  int bh, rank;
  if (!map_block(blockIdx.x, n_items, heads_per_xcd, BH, &bh, &rank)) return;
  // items are listed longest first; the fields are the same in every lane: held in scalar
  // registers, so that what derives from them (trip counts, the causal tests) is scalar too
  Bwd32Item it = items[rank];
  it.kvblk = __builtin_amdgcn_readfirstlane(it.kvblk);
  it.tile_begin = __builtin_amdgcn_readfirstlane(it.tile_begin);
  it.tile_end = __builtin_amdgcn_readfirstlane(it.tile_end);
  it.shared = __builtin_amdgcn_readfirstlane(it.shared);
  const int kvblk = it.kvblk;
  const int b = bh / p.H, h = bh % p.H;

  const float* Q = (const float*)p.q + b * p.sq.b + h * p.sq.h;
  const float* K = (const float*)p.k + b * p.sk.b + h * p.sk.h;
  const float* V = (const float*)p.v + b * p.sv.b + h * p.sv.h;
  const float* dO = (const float*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  float* dQ = (float*)p.dq + b * p.sdq.b + h * p.sdq.h;
  float* dK = (float*)p.dk + b * p.sdk.b + h * p.sdk.h;
  float* dV = (float*)p.dv + b * p.sdv.b + h * p.sdv.h;
  const float* lse = p.lse + (int64_t)bh * T;
  const float* delta = p.delta + (int64_t)bh * T;

  const int kv0 = kvblk * kBwd32Blk;
  const int kvw0 = kv0 + 32 * wave;
  const int kvrow = kvw0 + (lane & 31);

  // K block -> LDS (rows past T-1 as zeros: their dS is zero anyway)
#pragma unroll
  for (int i = 0; i < NKLOAD; ++i) {
    const int idx = tid + 256 * i;
    const int row = idx / CH, ch = idx % CH;
    floatx4 t = ZEROF4;
    if (kv0 + row < T) t = *(const floatx4*)(K + (int64_t)(kv0 + row) * p.sk.t + 4 * ch);
    *(floatx4*)(Ks + row * LD + 4 * ch) = t;
  }

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

  const int first_tile = it.tile_begin;  // this item's share of the block's query tiles
  const int n_tiles = it.tile_end;

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

  const int my_db = wave % DB;
  const int my_kv = KPW * (wave / DB);  // first key (within the block) of this wave's dQ share

  prefetch(first_tile);
  DEERS_PHASE_STATE;
  DEERS_PHASE(9);
  for (int j = first_tile; j < n_tiles; ++j) {
    __syncthreads();  // the previous tile's readers (Qs, dOs, dSs) are done
    DEERS_PHASE(0);
    commit();
    DEERS_PHASE(1);
    __syncthreads();
    DEERS_PHASE(2);
    if (j + 1 < n_tiles) prefetch(j + 1);

    const int qb0 = j * STEP;
    if (qb0 + 31 >= kvw0) {  // else every query here precedes the wave's keys
      floatx16 s = ZERO16, dp = ZERO16;
      const float* qrow_p = Qs + (lane & 31) * LD + g * KH;
      const float* dorow_p = dOs + (lane & 31) * LD + g * KH;
#pragma unroll
      for (int c = 0; c < KH / 4; ++c) {
        const floatx4 a = *(const floatx4*)(qrow_p + 4 * c);
        const floatx4 a2 = *(const floatx4*)(dorow_p + 4 * c);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          s = mfma_f32(a[e], kf[4 * c + e], s);
          dp = mfma_f32(a2[e], vf[4 * c + e], dp);
        }
      }

      DEERS_PHASE(3);
      const bool need_mask = (qb0 < kvw0 + 31);
      float* ds_row = dSs + (32 * wave + (lane & 31)) * LDS_DS + 4 * g;
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const floatx4 l4 = *(const floatx4*)(lse2s + 8 * rq + 4 * g);
        const floatx4 d4 = *(const floatx4*)(deltas + 8 * rq + 4 * g);
        floatx4 out;
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
          out[e] = dp[r] * p.scale;
        }
        *(floatx4*)(ds_row + 8 * rq) = out;
      }
      DEERS_PHASE(4);

#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * g + (r & 3);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const float ado = dOs[row * LD + 32 * db + (lane & 31)];
          dvacc[db] = mfma_f32(ado, s[r], dvacc[db]);
          const float aq = Qs[row * LD + 32 * db + (lane & 31)];
          dkacc[db] = mfma_f32(aq, dp[r], dkacc[db]);
        }
      }
    }
    DEERS_PHASE(5);
    __syncthreads();  // scale * dS^T of this tile is complete
    DEERS_PHASE(6);

    // dQ[q, d-block] += sum over this wave's keys of dS[q, kv] K[kv, d]; key sub-blocks
    // whose wave skipped the tile hold no data: only the first live_kv keys do
    {
      // live keys come in whole 32-key sub-blocks: the products go in runs of 16, each
      // run's operand reads issued ahead of its MFMAs
      const int live_kv = min(kBwd32Blk, qb0 + 32 - kv0);
      const int n_runs = max(0, min(KPW, live_kv - my_kv)) / 32;
      floatx16 acc = ZERO16;
      const float* a_p = dSs + (my_kv + g) * LDS_DS + (lane & 31);
      const float* b_p = Ks + (my_kv + g) * LD + 32 * my_db + (lane & 31);
      for (int run = 0; run < n_runs; ++run) {
#pragma unroll
        for (int t = 0; t < 16; ++t)
          acc = mfma_f32(a_p[(32 * run + 2 * t) * LDS_DS], b_p[(32 * run + 2 * t) * LD], acc);
      }
      DEERS_PHASE(7);
      if (n_runs > 0 && qb0 + 32 <= T) {
        float* dst = dQ + (int64_t)(qb0 + 4 * g) * p.sdq.t + 32 * my_db + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int qo = 8 * (r >> 2) + (r & 3);
          unsafeAtomicAdd(dst + (int64_t)qo * p.sdq.t, acc[r]);
        }
      } else if (n_runs > 0) {
        float* dst = dQ + (int64_t)(qb0 + 4 * g) * p.sdq.t + 32 * my_db + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int qo = 8 * (r >> 2) + (r & 3);
          if (qb0 + 4 * g + qo < T) unsafeAtomicAdd(dst + (int64_t)qo * p.sdq.t, acc[r]);
        }
      }
    }
    DEERS_PHASE(8);
  }

  if (it.shared) {
    // The block's other item adds its half too (the prep kernel cleared the rows).  In the
    // accumulator layout a lane owns a key row, so an atomic instruction would touch 64
    // cache lines; staged through LDS (the K block's space) each one covers one row's
    // contiguous floats instead.
    constexpr int NOUT = kBwd32Blk * D / 256;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      __syncthreads();  // Ks free: dQ products of the last tile / the previous staging are done
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          floatx4 o4;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            o4[e] = which == 0 ? dkacc[db][4 * rq + e] * p.scale : dvacc[db][4 * rq + e];
          *(floatx4*)(Ks + (32 * wave + (lane & 31)) * LD + 32 * db + 8 * rq + 4 * g) = o4;
        }
      __syncthreads();
      float* dst = which == 0 ? dK : dV;
      const int64_t pitch = which == 0 ? p.sdk.t : p.sdv.t;
#pragma unroll 4
      for (int i = 0; i < NOUT; ++i) {
        const int idx = tid + 256 * i;
        const int row = idx / D, col = idx % D;
        if (kv0 + row < T) unsafeAtomicAdd(dst + (int64_t)(kv0 + row) * pitch + col, Ks[row * LD + col]);
      }
    }
  } else if (kvrow < T) {
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

// Work items of a launch at sequence length T, longest first, in device memory (built once
// per (T, split) and kept for the life of the process).  A key block walks the query tiles
// from its diagonal to the end, so block 0 has twice the mean number of iterations.  When
// the launch has fewer workgroups than the device holds, blocks with more than half of block
// 0's iterations are cut into two items of half the range, which add their dK / dV halves
// with atomics onto cleared rows (a sum of exactly two terms, so dK and dV stay
// bit-reproducible): 42 -> 29 us at 4x6x256x32, 145 -> 81 us at 3x5x640x64.  A launch that
// fills the device is bound by CU throughput, not by its longest chain, and the extra
// prologues and write-outs only cost (354 -> 386 us at 8x12x1024x64): it is not split.
// split_rows: key rows [0, split_rows) of every head are shared.
struct Bwd32Items {
  const Bwd32Item* dev = nullptr;
  int n_items = 0;
  int split_rows = 0;
};
static Bwd32Items bwd32_items(int T, bool split) {
  static std::map<std::pair<int, bool>, Bwd32Items> cache;  // launches are serialised by the caller
  auto it = cache.find({T, split});
  if (it != cache.end()) return it->second;
  constexpr int kStep = 32, kTilesPerBlock = kBwd32Blk / kStep;
  const int n_blocks = (T + kBwd32Blk - 1) / kBwd32Blk;
  const int n_tiles = (T + kStep - 1) / kStep;
  std::vector<Bwd32Item> items;
  Bwd32Items out;
  for (int kb = 0; kb < n_blocks; ++kb) {
    const int first = kb * kTilesPerBlock;
    const int n = n_tiles - first;
    if (split && 2 * n > n_tiles && n >= 2) {
      const int mid = first + (n + 1) / 2;
      items.push_back({kb, first, mid, 1});
      items.push_back({kb, mid, n_tiles, 1});
      out.split_rows = std::min(T, (kb + 1) * kBwd32Blk);
    } else {
      items.push_back({kb, first, n_tiles, 0});
    }
  }
  std::stable_sort(items.begin(), items.end(), [](const Bwd32Item& a, const Bwd32Item& b) {
    return a.tile_end - a.tile_begin > b.tile_end - b.tile_begin;
  });
  Bwd32Item* dev = nullptr;
  if (hipMalloc(&dev, items.size() * sizeof(Bwd32Item)) != hipSuccess) return Bwd32Items{};
  if (hipMemcpy(dev, items.data(), items.size() * sizeof(Bwd32Item), hipMemcpyHostToDevice) !=
      hipSuccess) {
    (void)hipFree(dev);
    return Bwd32Items{};
  }
  out.dev = dev;
  out.n_items = (int)items.size();
  cache.emplace(std::make_pair(T, split), out);
  return out;
}

template <int D>
static bool launch_bwd_fused_f32_d(const BwdParams& p, int B, hipStream_t stream) {
  constexpr size_t lds = Fused32Cfg<D>::kLds;
  static bool attr_set = false;  // launches are serialised by the caller
  static int capacity = 0;       // workgroups of the main kernel the device holds at once
  if (!attr_set) {
    if (lds > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_bwd_fused_f32_kernel<D>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    int dev = 0, per_cu = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_bwd_fused_f32_kernel<D>, 256, lds) ==
            hipSuccess)
      capacity = per_cu * prop.multiProcessorCount;
    attr_set = true;
  }
  const int n_blocks = (p.T + kBwd32Blk - 1) / kBwd32Blk;
  const Bwd32Items items = bwd32_items(p.T, (int64_t)n_blocks * B * p.H < capacity);
  if (!items.dev) {
    (void)hipGetLastError();  // the two-pass form stands in: leave no error behind for the caller's check
    return false;
  }
  const int64_t rows = (int64_t)B * p.H * p.T;
  constexpr int LPR = D / 4;
  const int64_t threads = rows * LPR;
  {
    LaunchScope scope("attn_bwd_prep_f32", stream);
    hipLaunchKernelGGL((attn_bwd_prep_f32_kernel<D>), dim3((threads + 255) / 256), dim3(256), 0, stream,
                       p, B, items.split_rows);
  }
  const int BH = B * p.H;
  const int heads_per_xcd = (BH + 7) / 8;
  LaunchScope scope("attn_bwd_f32", stream);
  hipLaunchKernelGGL((attn_bwd_fused_f32_kernel<D>), dim3(8 * items.n_items * heads_per_xcd), dim3(256),
                     lds, stream, p, BH, items.n_items, heads_per_xcd, items.dev);
  return true;
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
    // the two-pass form stands in if the one-pass kernel's item table cannot be allocated
    case 32:
      if (!launch_bwd_fused_f32_d<32>(p, B, stream)) launch_bwd_f32_d<32, 64>(p, B, stream);
      break;
    case 64:
      if (!launch_bwd_fused_f32_d<64>(p, B, stream)) launch_bwd_f32_d<64, 64>(p, B, stream);
      break;
    case 128: launch_bwd_f32_d<128, 32>(p, B, stream); break;
  }
}

}  // namespace deers
