// Fused causal attention backward, f16 storage / f32 accumulate, gfx950.
//
// Replaces the reference's op-by-op autograd sweep over the attention core
// (src/backprop.rs:52-66 through src/ops.rs:1089-1101, 422-425, 210-214,
// 777-799, 1162-1175, 638-643) by recomputation from (Q, K, V, O, LSE, dO):
//     P  = exp(S*scale + mask - LSE)        dV = P^T dO
//     dP = dO V^T                           dS = P o (dP - delta),  delta = rowsum(dO o O)
//     dQ = scale dS K                       dK = scale dS^T Q
//
// One launch with two roles, no atomics on data, bit-reproducible (the dQ role
// publishes, for the rows it owns, negdelta[b,h,t] = -sum_d dO*O and
// lse2 = LSE*log2(e) as f32 in a workspace whose rows are padded to a multiple of 64
// per head, with lse2 = +inf and negdelta = 0 in the padding so padded query rows
// get probability exactly 0; the dK/dV role waits for a block's rows through a flag,
// see attn_bwd_f16_kernel):
//   2. dK/dV   : a workgroup owns 128 key rows (32 per wave, K^T and V^T held in
//                registers as B operands) and walks the 64-row query tiles at or
//                below the diagonal.  Orientation S[q,kv] (one key column per lane)
//                so P and dS leave the accumulators directly as B operands of
//                dV^T += dO^T P and dK^T += Q^T dS; dO^T / Q^T fragments come
//                from the row-major LDS tiles via ds_read_b64_tr_b16.
//   1. dQ      : a workgroup owns 128 query rows (32 per wave, Q and dO in
//                registers) and walks 64-row key tiles up to the diagonal.
//                Orientation S^T[kv,q] (one query column per lane, LSE and delta are
//                per-lane scalars); dS^T leaves the accumulators as the B operand of
//                dQ^T += K^T dS^T with K^T fragments read transposed from LDS.
// Recomputing S and dP in both roles costs 7 tile GEMMs instead of 5 but
// keeps every product in registers and needs no dQ accumulation buffer.
//
// The "- delta" of dS is folded into the dP accumulator's initial value, so the
// vector pipe spends per score one fma + one exp2 (P), one multiply (dS) and the
// f16 packing.  Streamed tiles go global -> LDS asynchronously
// (global_load_lds_dwordx4), unpadded and XOR-swizzled, into a ring of P+1 slots
// requested P iterations ahead; one barrier per iteration.
#include <type_traits>


#include "attn_bwd_f16_bp.h"
#include "common.h"

namespace deers {

constexpr int kBwdBlk = 128;  // rows owned by a workgroup (keys in dK/dV, queries in dQ)
constexpr int kBwdStep = 64;  // rows of the streamed operand per iteration

#define ZEROH8 half8{0, 0, 0, 0, 0, 0, 0, 0}

template <int D>
struct BwdCfg {
  static constexpr int P = (D == 128) ? 1 : 2;   // prefetch distance in iterations
  static constexpr int NS = P + 1;               // ring slots
  static constexpr int RB = D * 2;               // row bytes
  static constexpr int TILE_B = kBwdStep * RB;   // bytes of one streamed tile
  static constexpr int VEC_B = kBwdStep * 4;     // bytes of one per-row f32 vector
  static constexpr int SLOT_B = 2 * TILE_B + 2 * VEC_B;  // dK/dV: Q, dO, lse2, negdelta
  static constexpr size_t kLdsDkdv = NS * SLOT_B;
  static constexpr size_t kLdsDq = NS * 2 * TILE_B;      // dQ: K, V
};

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void bwd_dkdv_f16_body(const BwdParams& p, int BH, int n_blocks,
                                                  int heads_per_xcd, int block_id) {
  using Cfg = BwdCfg<D>;
  constexpr int P = Cfg::P, NS = Cfg::NS, RB = Cfg::RB, TILE_B = Cfg::TILE_B;
  constexpr int VEC_B = Cfg::VEC_B, SLOT_B = Cfg::SLOT_B;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int CH = D / 8;
  constexpr int RPW = 1024 / RB;       // tile rows covered by one wave-wide 1 KiB load
  constexpr int NWLW = TILE_B / 4096;  // 1 KiB loads per wave per tile
  // every wave issues the same number of loads per iteration (vmcnt bookkeeping):
  // Q and dO slabs plus one 256-byte vector (even waves: lse2, odd waves: negdelta)
  constexpr int LPI = 2 * NWLW + 1;

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;

  int bh, rank;
  if (!map_block(block_id, n_blocks, heads_per_xcd, BH, &bh, &rank)) return;
  const int kvblk = rank;  // key block 0 walks the most query tiles
  set_block_priority(rank, n_blocks);
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  const half_t* dO = (const half_t*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  half_t* dK = (half_t*)p.dk + b * p.sdk.b + h * p.sdk.h;
  half_t* dV = (half_t*)p.dv + b * p.sdv.b + h * p.sdv.h;
  const float* lse2 = p.lse2 + (int64_t)bh * p.t_pad;
  const float* negdelta = p.negdelta + (int64_t)bh * p.t_pad;
  const int kv0 = kvblk * kBwdBlk;
  const int kvw0 = kv0 + 32 * wave;
  const int kvrow = kvw0 + (lane & 31);

  const int first_tile = kv0 / kBwdStep;
  const int n_tiles = (T + kBwdStep - 1) / kBwdStep;  // query tiles first_tile .. n_tiles-1

  // ---- asynchronous loads of query tile t into ring slot t % NS ----
  const uint32_t lds0 = lds_address(smem);
  const int sqt = (int)p.sq.t, sdot = (int)p.sdo.t;
  const int tail_tile = (T - 1) / kBwdStep;
  uint32_t ld_q[NWLW], ld_do[NWLW], ld_q_tail[NWLW], ld_do_tail[NWLW];
#pragma unroll
  for (int i = 0; i < NWLW; ++i) {
    const int row = (wave * NWLW + i) * RPW + lane / CH;
    const int col = 16 * ((lane % CH) ^ lds_swizzle<CH>(row));
    const int row_tail = min(row, T - 1 - tail_tile * kBwdStep);
    ld_q[i] = (uint32_t)(row * sqt * 2 + col);
    ld_do[i] = (uint32_t)(row * sdot * 2 + col);
    ld_q_tail[i] = (uint32_t)(row_tail * sqt * 2 + col);
    ld_do_tail[i] = (uint32_t)(row_tail * sdot * 2 + col);
  }
  // The row statistics of query block qb come from the dQ workgroup that owns it, which
  // runs in the same launch on the same XCD (see the launch kernel below).  This block needs
  // those of query blocks kvblk .. n_blocks-1: before its first request it polls all their
  // flags at once, one per lane, so the loop itself never waits for a flag (a poll there
  // drains the wave's whole ring of tile loads, every other iteration).
  // Bounded: a producer cannot be held up by this workgroup (it was dispatched earlier and
  // waits for nothing), so the bound is not reached in practice; it guarantees that every
  // wave leaves the loop.  A wait that does run out raises the error word in front of the
  // flags (the statistics it then reads are not valid and this call's dK / dV are wrong):
  // the host reports it at the next synchronisation.
  auto wait_published = [&]() {
    if (p.epoch == 0) return;  // the statistics were published by an earlier launch
    for (int base = kvblk; base < n_blocks; base += 64) {
      const int qb = base + lane;
      const int* flag = p.ready + (int64_t)bh * n_blocks + min(qb, n_blocks - 1);
      int spins = 0;
      for (;;) {
        const int seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__all(seen == p.epoch)) break;
        if (++spins >= p.spin_limit) {
          __hip_atomic_store(p.error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(8);
      }
    }
  };
  auto request = [&](int t) {
    const int tc = min(t, n_tiles - 1);  // clamped repeats are never consumed
    const uint32_t slot = lds0 + (t % NS) * SLOT_B;
    const half_t* qbase = Q + (uint32_t)(tc * kBwdStep * sqt);
    const half_t* dobase = dO + (uint32_t)(tc * kBwdStep * sdot);
#pragma unroll
    for (int i = 0; i < NWLW; ++i) {
      const uint32_t dst = slot + (wave * NWLW + i) * 1024;
      async_load16_to_lds(qbase, tc == tail_tile ? ld_q_tail[i] : ld_q[i], dst);
      async_load16_to_lds(dobase, tc == tail_tile ? ld_do_tail[i] : ld_do[i], dst + TILE_B);
    }
    // per-row vectors (the workspace rows are padded, no clamp needed)
    const float* vec = ((wave & 1) ? negdelta : lse2) + tc * kBwdStep;
    async_load4_to_lds(vec, lane * 4, slot + 2 * TILE_B + (wave & 1) * VEC_B);
  };

  // K^T and V^T as B operands: lane holds row kvrow, halfs 16ks+8g .. +7.
  // Rows past T-1 read row T-1 instead: their keys are masked for every valid query
  // and their dK/dV rows are not stored, and without a branch the loads issue as one
  // batch with a single wait.  Issued before the flag poll, which is a round trip to L2 of
  // its own: the two latencies overlap.
  half8 kf[KS], vf[KS];
  {
    const int krow = min(kvrow, T - 1);
    const half_t* kp = K + (int64_t)krow * p.sk.t + 8 * g;
    const half_t* vp = V + (int64_t)krow * p.sv.t + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      kf[ks] = *(const half8*)(kp + 16 * ks);
      vf[ks] = *(const half8*)(vp + 16 * ks);
    }
  }

  wait_published();
#pragma unroll
  for (int i = 0; i < P; ++i) request(first_tile + i);

  // ---- per-lane swizzled read offsets (bytes within a tile) ----
  int aoff[KS];  // row-major A operand: row lane%32 (+32 for the second block), chunk 2ks+g
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    aoff[ks] = (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  int toff_lo[DB], toff_hi[DB];  // transposed A operand (see lds_read_tr16)
  {
    const int lrow = 4 * g + ((lane & 15) >> 2);
    const int c4 = lane & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      toff_lo[db] = lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      toff_hi[db] = (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }

  floatx16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    dkacc[i] = ZERO16;
    dvacc[i] = ZERO16;
  }
  // kept in a vector register: v_fma_f32 with a scalar-register operand issues at 4.4 clocks
  // per SIMD against 2.6 with three vector registers, and every score passes through one
  float c = p.scale_log2;
  asm volatile("" : "+v"(c));

  // Per-iteration LDS read addresses: slot base + per-lane offset, one add each; everything
  // else (second 32-row block, dO tile, contraction step) is an instruction offset.
  uint32_t a_at[KS], t_lo_at[DB], t_hi_at[DB], vec_at;
  auto set_slot = [&](uint32_t slot) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a_at[ks] = opaque(slot + aoff[ks]);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      t_lo_at[db] = opaque(slot + toff_lo[db]);
      t_hi_at[db] = opaque(slot + toff_hi[db]);
    }
    vec_at = opaque(slot + 2 * TILE_B + 16 * g);
  };

  // One 32-query block of the current slot: MASKED applies the causal element mask.
  auto block = [&](auto masked, auto mb_c, int qb0) {
    constexpr bool MASKED = decltype(masked)::value;
    constexpr int MB = decltype(mb_c)::value;
    constexpr uint32_t QT = 32 * MB * RB;            // Q rows of this block
    constexpr uint32_t DOT = TILE_B + 32 * MB * RB;  // dO rows of this block
    // dP starts from -delta[q] (row value of every accumulator register)
    floatx16 s = ZERO16, dp;
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      const floatx4 nd = lds_read_float4_at(vec_at + VEC_B + 128 * MB + 32 * rq);
#pragma unroll
      for (int e = 0; e < 4; ++e) dp[4 * rq + e] = nd[e];
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      s = mfma_f16(lds_read_half8_at(a_at[ks] + QT), kf[ks], s);
      dp = mfma_f16(lds_read_half8_at(a_at[ks] + DOT), vf[ks], dp);
    }
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      const floatx4 l4 = lds_read_float4_at(vec_at + 128 * MB + 32 * rq);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int r = 4 * rq + e;
        float pv = fast_exp2(__builtin_fmaf(s[r], c, -l4[e]));
        if constexpr (MASKED) {
          if (kvrow > qb0 + 8 * rq + 4 * g + e) pv = 0.f;
        }
        s[r] = pv;
        dp[r] = pv * dp[r];
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
        const half4 lo = lds_read_tr16_at(t_lo_at[db] + DOT + 16 * st * RB);
        const half4 hi = lds_read_tr16_at(t_hi_at[db] + DOT + 16 * st * RB);
        dvacc[db] = mfma_f16(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7), pf,
                             dvacc[db]);
        const half4 qlo = lds_read_tr16_at(t_lo_at[db] + QT + 16 * st * RB);
        const half4 qhi = lds_read_tr16_at(t_hi_at[db] + QT + 16 * st * RB);
        dkacc[db] = mfma_f16(__builtin_shufflevector(qlo, qhi, 0, 1, 2, 3, 4, 5, 6, 7), dsf,
                             dkacc[db]);
      }
    }
  };

  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  wait_all_vmem();  // K/V fragments are in registers; see wait_all_vmem
  for (int j = first_tile; j < n_tiles; ++j) {
    // tile j was requested P iterations ago; at most the P-1 younger groups may
    // still be in flight.  The barrier also retires all reads of the slot that the
    // next request overwrites (tile j-1's).
    wait_vmcnt<(P - 1) * LPI>();
    __syncthreads();
    request(j + P);
    set_slot(lds0 + (j % NS) * SLOT_B);
    const int q0 = j * kBwdStep;
    auto one = [&](auto mb_c) {
      const int qb0 = q0 + 32 * decltype(mb_c)::value;  // first query row of this 32-block
      if (qb0 + 31 < kvw0) return;                       // every query here precedes the wave's keys
      if (qb0 < kvw0 + 31)
        block(yes, mb_c, qb0);
      else
        block(no, mb_c, qb0);
    };
    one(std::integral_constant<int, 0>{});
    one(std::integral_constant<int, 1>{});
  }

  if (kvrow < T) {
    half_t* dkrow = dK + (int64_t)kvrow * p.sdk.t;
    half_t* dvrow = dV + (int64_t)kvrow * p.sdv.t;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      store_block_f16(dkrow + 32 * db, dkacc[db], p.scale, g);
      store_block_f16(dvrow + 32 * db, dvacc[db], 1.f, g);
    }
  }
}

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void bwd_dq_f16_body(const BwdParams& p, int BH, int n_blocks,
                                                int heads_per_xcd, int block_id) {
  using Cfg = BwdCfg<D>;
  constexpr int P = Cfg::P, NS = Cfg::NS, RB = Cfg::RB, TILE_B = Cfg::TILE_B;
  constexpr int KS = D / 16;
  constexpr int DB = D / 32;
  constexpr int CH = D / 8;
  constexpr int RPW = 1024 / RB;
  constexpr int NWLW = TILE_B / 4096;
  constexpr int LPI = 2 * NWLW;

  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;

  int bh, rank;
  if (!map_block(block_id, n_blocks, heads_per_xcd, BH, &bh, &rank)) return;
  const int qtile = n_blocks - 1 - rank;  // the last query block walks the most key tiles
  set_block_priority(rank, n_blocks);
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  const half_t* dO = (const half_t*)p.d_o + b * p.sdo.b + h * p.sdo.h;
  half_t* dQ = (half_t*)p.dq + b * p.sdq.b + h * p.sdq.h;
  const int q0 = qtile * kBwdBlk;
  const int qw0 = q0 + 32 * wave;
  const int qrow = qw0 + (lane & 31);

  int last_q = q0 + kBwdBlk - 1;
  if (last_q > T - 1) last_q = T - 1;
  const int n_tiles = last_q / kBwdStep + 1;

  // ---- asynchronous loads of key/value tile t into ring slot t % NS ----
  const uint32_t lds0 = lds_address(smem);
  const int skt = (int)p.sk.t, svt = (int)p.sv.t;
  const int tail_tile = (T - 1) / kBwdStep;
  uint32_t ld_k[NWLW], ld_v[NWLW], ld_k_tail[NWLW], ld_v_tail[NWLW];
#pragma unroll
  for (int i = 0; i < NWLW; ++i) {
    const int row = (wave * NWLW + i) * RPW + lane / CH;
    const int col = 16 * ((lane % CH) ^ lds_swizzle<CH>(row));
    const int row_tail = min(row, T - 1 - tail_tile * kBwdStep);
    ld_k[i] = (uint32_t)(row * skt * 2 + col);
    ld_v[i] = (uint32_t)(row * svt * 2 + col);
    ld_k_tail[i] = (uint32_t)(row_tail * skt * 2 + col);
    ld_v_tail[i] = (uint32_t)(row_tail * svt * 2 + col);
  }
  auto request = [&](int t) {
    const int tc = min(t, n_tiles - 1);
    const uint32_t slot = lds0 + (t % NS) * 2 * TILE_B;
    const half_t* kbase = K + (uint32_t)(tc * kBwdStep * skt);
    const half_t* vbase = V + (uint32_t)(tc * kBwdStep * svt);
#pragma unroll
    for (int i = 0; i < NWLW; ++i) {
      const uint32_t dst = slot + (wave * NWLW + i) * 1024;
      async_load16_to_lds(kbase, tc == tail_tile ? ld_k_tail[i] : ld_k[i], dst);
      async_load16_to_lds(vbase, tc == tail_tile ? ld_v_tail[i] : ld_v[i], dst + TILE_B);
    }
  };
#pragma unroll
  for (int i = 0; i < P; ++i) request(i);

  half8 qf[KS], dof[KS];
  float dsum = 0.f;  // this lane's half of rowsum(dO o O)
  float lse_clamped;
  const half_t* O = (const half_t*)p.o + b * p.so.b + h * p.so.h;
  // Rows past T-1 read row T-1 instead (their dQ rows are not stored and a query owns
  // its accumulator column, so nothing leaks into valid rows): without a branch all
  // loads issue as one batch with a single wait.
  {
    const int lrow = min(qrow, T - 1);
    const half_t* qp = Q + (int64_t)lrow * p.sq.t + 8 * g;
    const half_t* dop = dO + (int64_t)lrow * p.sdo.t + 8 * g;
    const half_t* op = O + (int64_t)lrow * p.so.t + 8 * g;
    half8 of[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = *(const half8*)(qp + 16 * ks);
      dof[ks] = *(const half8*)(dop + 16 * ks);
      of[ks] = *(const half8*)(op + 16 * ks);
    }
    const float lse_row = p.lse[(int64_t)bh * T + lrow];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) dsum += (float)dof[ks][e] * (float)of[ks][e];
    if (qrow >= T) dsum = 0.f;
    lse_clamped = lse_row;
  }
  // Per-row statistics, also published for the dK/dV kernel that runs next: rows in
  // the padding [T, t_pad) get lse2 = +inf and negdelta = 0, i.e. probability 0.
  const float nd = -pair_sum(dsum);
  const float l2 = qrow < T ? lse_clamped * kLog2e : INFINITY;
  if (g == 0 && qrow < p.t_pad) {
    p.lse2[(int64_t)bh * p.t_pad + qrow] = l2;
    p.negdelta[(int64_t)bh * p.t_pad + qrow] = nd;
  }
  floatx16 nd16;  // initial value of every dP^T accumulator: -delta of this lane's query
#pragma unroll
  for (int r = 0; r < 16; ++r) nd16[r] = nd;

  int aoff[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    aoff[ks] = (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  int toff_lo[DB], toff_hi[DB];
  {
    const int lrow = 4 * g + ((lane & 15) >> 2);
    const int c4 = lane & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      toff_lo[db] = lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      toff_hi[db] = (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }

  floatx16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) dqacc[i] = ZERO16;
  // kept in a vector register: v_fma_f32 with a scalar-register operand issues at 4.4 clocks
  // per SIMD against 2.6 with three vector registers, and every score passes through one
  float c = p.scale_log2;
  asm volatile("" : "+v"(c));

  uint32_t a_at[KS], t_lo_at[DB], t_hi_at[DB];  // per-iteration LDS read addresses (see dK/dV)
  auto set_slot = [&](uint32_t slot) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a_at[ks] = opaque(slot + aoff[ks]);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      t_lo_at[db] = opaque(slot + toff_lo[db]);
      t_hi_at[db] = opaque(slot + toff_hi[db]);
    }
  };

  auto block = [&](auto masked, auto mb_c, int kvb0) {
    constexpr bool MASKED = decltype(masked)::value;
    constexpr int MB = decltype(mb_c)::value;
    constexpr uint32_t KT = 32 * MB * RB;           // K rows of this block
    constexpr uint32_t VT = TILE_B + 32 * MB * RB;  // V rows of this block
    floatx16 s = ZERO16, dp = nd16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      s = mfma_f16(lds_read_half8_at(a_at[ks] + KT), qf[ks], s);
      dp = mfma_f16(lds_read_half8_at(a_at[ks] + VT), dof[ks], dp);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float pv = fast_exp2(__builtin_fmaf(s[r], c, -l2));
      if constexpr (MASKED) {
        if (kvb0 + 8 * (r >> 2) + 4 * g + (r & 3) > qrow) pv = 0.f;
      }
      dp[r] = pv * dp[r];
    }
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const half8 dsf =
          pack_half8(dp[8 * st + 0], dp[8 * st + 1], dp[8 * st + 2], dp[8 * st + 3],
                     dp[8 * st + 4], dp[8 * st + 5], dp[8 * st + 6], dp[8 * st + 7]);
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const half4 lo = lds_read_tr16_at(t_lo_at[db] + KT + 16 * st * RB);
        const half4 hi = lds_read_tr16_at(t_hi_at[db] + KT + 16 * st * RB);
        dqacc[db] = mfma_f16(__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7), dsf,
                             dqacc[db]);
      }
    }
  };

  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  wait_all_vmem();  // Q/dO fragments are in registers; see wait_all_vmem
  for (int j = 0; j < n_tiles; ++j) {
    wait_vmcnt<(P - 1) * LPI>();
    __syncthreads();
    if (j == 0 && tid == 0) {
      // every wave drained its stores of lse2 / negdelta (wait_all_vmem above) before
      // this barrier: the rows are in the XCD's L2, tell the dK/dV workgroups
      __hip_atomic_store(p.ready + (int64_t)bh * n_blocks + qtile, p.epoch, __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
    request(j + P);
    set_slot(lds0 + (j % NS) * 2 * TILE_B);
    const int kv0 = j * kBwdStep;
    auto one = [&](auto mb_c) {
      const int kvb0 = kv0 + 32 * decltype(mb_c)::value;
      if (kvb0 > qw0 + 31) return;  // block lies entirely in this wave's future
      if (kvb0 + 31 > qw0)
        block(yes, mb_c, kvb0);
      else
        block(no, mb_c, kvb0);
    };
    one(std::integral_constant<int, 0>{});
    one(std::integral_constant<int, 1>{});
  }

  if (qrow < T) {
    half_t* dqrow = dQ + (int64_t)qrow * p.sdq.t;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_block_f16(dqrow + 32 * db, dqacc[db], p.scale, g);
  }
}

// One launch for the whole backward: the first half of the grid runs the dQ role, the
// second half the dK/dV role.  Each half is cut into groups of 8 * heads_per_xcd workgroups,
// one block length over all heads per group, and block ids inside a group map to heads the
// same way in both halves (a half is a multiple of 8 long), so the dK/dV workgroups of a
// head share an XCD, and its L2, with the dQ workgroups that publish the head's row
// statistics; they are dispatched after them and poll a per-block flag before they first
// touch a query block's statistics.  Against two launches this saves a dispatch and lets
// the heavy dK/dV blocks start while dQ blocks are still running.
//
// The dK/dV groups run longest first, so the launch ends on its shortest blocks.  The dQ
// groups run longest first too unless `dq_short_first`: then the shortest come first, publish
// their rows' statistics within microseconds and leave, and dK/dV work starts early instead
// of after the longest dQ blocks, which otherwise fill the device alone, have drained.  The
// host asks for that when a group is a sizeable part of what the device holds at once (see
// launch_bwd_f16_d).  Either way every dQ workgroup precedes every dK/dV workgroup in
// dispatch order, and dQ workgroups wait for nothing.
//
// `first_id` is added to blockIdx.x: 0 with a grid of both halves is the single launch;
// a grid of one half with first_id = 0, then one with first_id = the half's length, runs
// the two roles as two launches in stream order (the flags are then already set when the
// second launch starts).  The hand-over inside one launch stores the statistics, drains
// the stores (vmcnt 0) and sets the flag with relaxed atomics and no cache write-back,
// which is only enough when producer and consumer share one L2, i.e. one XCD: the host
// takes the single launch only on a device where workgroup id % 8 is known to be the XCD.
//
// The flags hold epochs (one per backward call, passed by the host) and are never cleared.
// Epoch 0 means that the flags are not used: the dK/dV role does not wait.  The host passes it
// with the two-launch form while the stream is being captured into a graph, whose replays
// could not be given a fresh epoch each.
template <int D>
__global__ __launch_bounds__(256, (D == 128 ? 1 : 2)) void attn_bwd_f16_kernel(BwdParams p, int BH, int n_blocks,
                                                                               int heads_per_xcd, int first_id,
                                                                               int dq_short_first) {
  const int group_wgs = 8 * heads_per_xcd;
  const int per_role = n_blocks * group_wgs;
  const int id = (int)blockIdx.x + first_id;
  if (id < per_role) {
    const int group = id / group_wgs;
    const int rank = dq_short_first ? n_blocks - 1 - group : group;
    bwd_dq_f16_body<D>(p, BH, n_blocks, heads_per_xcd, rank * group_wgs + id % group_wgs);
  } else {
    bwd_dkdv_f16_body<D>(p, BH, n_blocks, heads_per_xcd, id - per_role);
  }
}

// The same grid with the block-pipelined role bodies (head widths 32 and 64).
template <int D>
__global__ __launch_bounds__(256, 2) void attn_bwd_f16_bp_kernel(BwdParams p, int BH, int n_blocks, int heads_per_xcd,
                                                                  int first_id, int dq_short_first) {
  const int group_wgs = 8 * heads_per_xcd;
  const int per_role = n_blocks * group_wgs;
  const int id = (int)blockIdx.x + first_id;
  int bh, rank;
  if (id < per_role) {
    const int group = id / group_wgs;
    const int r = dq_short_first ? n_blocks - 1 - group : group;
    if (map_block(r * group_wgs + id % group_wgs, n_blocks, heads_per_xcd, BH, &bh, &rank))
      bwd_dq_f16_bp_body<D>(p, __builtin_amdgcn_readfirstlane(bh), n_blocks - 1 - __builtin_amdgcn_readfirstlane(rank),
                            n_blocks, blockIdx.x);
  } else {
    if (map_block(id - per_role, n_blocks, heads_per_xcd, BH, &bh, &rank))
      bwd_dkdv_f16_bp_body<D>(p, __builtin_amdgcn_readfirstlane(bh), __builtin_amdgcn_readfirstlane(rank), n_blocks,
                              blockIdx.x);
  }
}

template <int D>
static void launch_bwd_f16_d(const BwdParams& p, int B, int mode, hipStream_t stream) {
  const int BH = B * p.H;
  const int n_blocks = (p.T + kBwdBlk - 1) / kBwdBlk;
  const int heads_per_xcd = (BH + 7) / 8;
  const int per_role = 8 * n_blocks * heads_per_xcd;
  typedef void (*Kernel)(BwdParams, int, int, int, int, int);
  Kernel kernel = attn_bwd_f16_kernel<D>;
  size_t lds = BwdCfg<D>::kLdsDkdv > BwdCfg<D>::kLdsDq ? BwdCfg<D>::kLdsDkdv : BwdCfg<D>::kLdsDq;
  if constexpr (D <= 64) {  // head widths 32 and 64 take the block-pipelined bodies
    kernel = attn_bwd_f16_bp_kernel<D>;
    lds = BwdBpCfg<D>::kLds;
  }
  static bool attr_set = false;  // launches are serialised by the caller
  if (!attr_set) {
    if (lds > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    attr_set = true;
  }
  if (mode == 2) {  // test hook: consumers only, so that their bounded wait runs out
    LaunchScope scope("attn_bwd_f16_dkdv", stream);
    hipLaunchKernelGGL(kernel, dim3(per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, per_role, 0);
    return;
  }
  if (mode == 1) {
    // Device capacity in workgroups of this kernel, found once (launches are serialised by
    // the caller).  The shortest-first dQ order pays when the longest dQ groups would
    // otherwise hold the device to themselves.
    static int capacity = 0;
    if (capacity == 0) {
      int dev = 0, per_cu = 0;
      hipDeviceProp_t prop;
      if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
          hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, lds) == hipSuccess && per_cu > 0)
        capacity = per_cu * prop.multiProcessorCount;
      else
        capacity = -1;
    }
    const int dq_short_first = capacity > 0 && bwd_dq_short_first(8 * heads_per_xcd, capacity);
    LaunchScope scope("attn_bwd_f16", stream);
    hipLaunchKernelGGL(kernel, dim3(2 * per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, 0,
                       dq_short_first);
    return;
  }
  {
    LaunchScope scope("attn_bwd_f16_dq", stream);
    hipLaunchKernelGGL(kernel, dim3(per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, 0, 0);
  }
  {
    LaunchScope scope("attn_bwd_f16_dkdv", stream);
    hipLaunchKernelGGL(kernel, dim3(per_role), dim3(256), lds, stream, p, BH, n_blocks, heads_per_xcd, per_role, 0);
  }
}

// mode 1: both roles in one grid with the flag hand-over (needs workgroup id % 8 == XCD);
// mode 0: two launches in stream order; mode 2: only the dK/dV half of the single launch
// (host-side test of the bounded wait: nobody publishes, every wait runs out).
void launch_attn_bwd_f16(const BwdParams& p, int B, int D, int mode, hipStream_t stream) {
  switch (D) {
    case 32: launch_bwd_f16_d<32>(p, B, mode, stream); break;
    case 64: launch_bwd_f16_d<64>(p, B, mode, stream); break;
    case 128: launch_bwd_f16_d<128>(p, B, mode, stream); break;
  }
}

}  // namespace deers
