// Block-pipelined causal attention backward (f16 storage, f32 accumulate, gfx950): the two role
// bodies of the single-launch backward (attn_bwd_f16.hip) for head widths 32, 64 and 128.
//
//     P  = exp(S*scale + mask - LSE)        dV = P^T dO
//     dP = dO V^T                           dS = P o (dP - delta),  delta = rowsum(dO o O)
//     dQ = scale dS K                       dK = scale dS^T Q
// (the reference's backward bodies: src/ops.rs:1089-1101, 422-425, 210-214, 777-799, 1162-1175,
// 638-643, walked by src/backprop.rs:52-66).
//
// A dQ workgroup owns 128 queries and walks the keys up to the diagonal, a dK/dV workgroup owns
// 128 keys and walks the queries from the diagonal on; the dQ role publishes the row statistics
// the dK/dV role needs.  The loops follow what the SIMD rewards (see attn_fwd_f16_bp.h): the unit is a 32-row block of
// the streamed operand, and in stage n a wave issues the MFMAs that consume block n-1's
// probabilities (dV, dK, or dQ) and those that produce block n+1's scores (S, dP) between the
// vector ops of block n, one MFMA per score register: exponential, multiply and the f16 packing
// ride in the MFMA's shadow.  Nothing else is left on the vector pipe:
//   * scale*log2(e) is folded into the f16 queries, once, by the dQ role, which keeps them in
//     registers and also writes them to the workspace; the dK/dV role streams these scaled
//     queries (its dK sum is rescaled by ln 2 at the end).  The forward folds the scale into its
//     queries the same way, so all three kernels exponentiate bit-identical scores: with the
//     scale folded into K in the dK/dV role instead, its scores differed from the forward's by up
//     to |S| * 2^-11, a dominant probability by 0.2 %, and dK of a peaked row by 6e-3;
//   * the S accumulator starts from -LSE*log2(e) and the dP accumulator from -delta (row values
//     read from LDS straight into the accumulator registers in the dK/dV role, 16-register
//     constants in the dQ role), so P = exp2(S) and dS = P * dP;
//   * the causal mask of a diagonal block is applied to the packed f16 pairs.
// Streamed blocks travel global -> LDS asynchronously into a ring of 6 slots, three stages
// ahead, one bare barrier per stage; the stage loop is unrolled over the ring so every LDS
// address is a fixed register plus an instruction offset.
#pragma once
#include <type_traits>

#include "common.h"

namespace deers {

#ifndef ZERO16
#define ZERO16 floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#endif

// Hook for a timestamp-tracing build of these bodies; expands to nothing in the library.
#ifndef DEERS_TRACE_POINT
#define DEERS_TRACE_POINT(slot)
#endif

constexpr int kBwdBpBlk = 32;   // rows of the streamed operand per stage
constexpr int kBwdBpOwn = 128;  // rows owned by a workgroup (keys in dK/dV, queries in dQ)

template <int D>
struct BwdBpCfg {
  static constexpr int R = 6;                    // ring slots (blocks)
  static constexpr int F = 3;                    // stages between a block's request and its barrier
  static constexpr int RB = D * 2;               // row bytes
  static constexpr int TB = kBwdBpBlk * RB;      // bytes of one operand's block
  static constexpr int VEC_B = 256;              // one per-row f32 vector as loaded (64 floats, 32 used)
  // dK/dV slot: Q block, dO block, then per wave its own copy of (-lse2, -delta)
  static constexpr int SLOT_DKDV = 2 * TB + 4 * 2 * VEC_B;
  static constexpr int SLOT_DQ = 2 * TB;         // dQ slot: K block, V block
  static constexpr size_t kLdsDkdv = (size_t)R * SLOT_DKDV;
  static constexpr size_t kLdsDq = (size_t)R * SLOT_DQ;
  static constexpr size_t kLds = kLdsDkdv > kLdsDq ? kLdsDkdv : kLdsDq;
};

// A ring slot is either a value or, in the unrolled turns of the ring, a compile-time constant.
template <uint32_t N>
using SlotC = std::integral_constant<uint32_t, N>;
template <class S>
constexpr bool kConstSlot = !std::is_integral_v<S>;
template <int R, int K, class S>
__device__ __forceinline__ auto slot_plus(S s) {
  if constexpr (kConstSlot<S>)
    return SlotC<(S::value + K) % R>{};
  else
    return (uint32_t)((s + K) % R);
}

// Packs two f32 into an f16 pair (round to nearest even).
__device__ __forceinline__ uint32_t pack_pair_f16(float a, float b) {
  return __builtin_bit_cast(uint32_t, half2v{(half_t)a, (half_t)b});
}

// ---------------------------------------------------------------------------
// dK / dV
// ---------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void bwd_dkdv_f16_bp_body(const BwdParams& p, int bh, int kvblk, int n_own,
                                                     [[maybe_unused]] int trace_row) {
  using Cfg = BwdBpCfg<D>;
  constexpr int R = Cfg::R, F = Cfg::F, RB = Cfg::RB, TB = Cfg::TB, VEC_B = Cfg::VEC_B, SLOT_B = Cfg::SLOT_DKDV;
  constexpr int KS = D / 16, DB = D / 32, CH = D / 8;
  constexpr int RPW = 1024 / RB;            // block rows covered by one 1 KiB wave load
  constexpr int NLT = 2 * TB / 1024 / 4;    // tile loads per wave per stage (Q then dO)
  constexpr int LPI = NLT + 2;              // + the wave's two row vectors
  constexpr int NM2 = 4 * DB;               // MFMAs that consume a block: (dV, dK) x 2 steps x DB
  constexpr int NM1 = 2 * KS;               // MFMAs that produce a block: (S, dP) x KS
  constexpr int W = 4;                      // operand fragments in flight ahead of their MFMA
  static_assert(D == 128 || D == 64 || D == 32, "head widths 32, 64 and 128");
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;
  DEERS_TRACE_POINT(0);  // key block 0 walks the most queries
  const int b_ = bh / p.H, h_ = bh % p.H;
  // the queries as the dQ role scaled them (f16(Q * scale * log2(e)), compact rows)
  const half_t* Q = (const half_t*)p.qs + (int64_t)bh * p.t_pad * D;
  const half_t* K = (const half_t*)p.k + b_ * p.sk.b + h_ * p.sk.h;
  const half_t* V = (const half_t*)p.v + b_ * p.sv.b + h_ * p.sv.h;
  const half_t* dO = (const half_t*)p.d_o + b_ * p.sdo.b + h_ * p.sdo.h;
  half_t* dK = (half_t*)p.dk + b_ * p.sdk.b + h_ * p.sdk.h;
  half_t* dV = (half_t*)p.dv + b_ * p.sdv.b + h_ * p.sdv.h;
  const float* neglse2 = p.lse2 + (int64_t)bh * p.t_pad;    // -LSE*log2(e); -inf in the padding
  const float* negdelta = p.negdelta + (int64_t)bh * p.t_pad;
  const int kv0 = kvblk * kBwdBpOwn;
  const int kvw0 = kv0 + 32 * wave;
  const int kvrow = kvw0 + (lane & 31);
  const int blk0 = kv0 / kBwdBpBlk;                       // first query block (the diagonal of wave 0)
  const int last_blk = (T - 1) / kBwdBpBlk;               // holds row T-1: its rows are clamped
  const int n_blk = last_blk - blk0 + 1;                  // query blocks blk0 .. last_blk
  const unsigned edge_span = (unsigned)max(n_blk - wave - 1, 0);  // stages wave+1 .. n_blk-1 need no mask
  const uint32_t lds0 = lds_address(smem);
  const int sqt = D, sdot = (int)p.sdo.t;

  // ---- this wave's loads of a stage: NLT of the 2 * TB / 1024 tile loads (waves 0 and 1 fetch
  // the Q block, waves 2 and 3 the dO block; a load covers RPW rows) and its two row vectors.
  // Lane offsets are fixed; rows past T-1 of a last, partial block read row T-1 (their
  // statistics give probability 0). ----
  constexpr int NLH = TB / 1024;
  const bool w_do = wave * NLT >= NLH;  // wave-uniform
  const half_t* tbase = w_do ? dO : Q;
  const int tstride = w_do ? sdot : sqt;
  const bool partial = (T & (kBwdBpBlk - 1)) != 0;
  uint32_t ld_off[NLT], ld_off_last[NLT], ld_dst[NLT];
#pragma unroll
  for (int i = 0; i < NLT; ++i) {
    const int n = (wave * NLT + i) % NLH;
    const int row = n * RPW + lane / CH;
    const int col = 16 * ((lane % CH) ^ lds_swizzle<CH>(row));
    ld_off[i] = (uint32_t)(row * tstride * 2 + col);
    ld_off_last[i] = (uint32_t)(min(row, T - 1 - last_blk * kBwdBpBlk) * tstride * 2 + col);
    ld_dst[i] = lds0 + (w_do ? TB : 0) + n * 1024;
  }
  const uint32_t vec_dst = lds0 + 2 * TB + wave * 2 * VEC_B;
  // The loads of relative block nb into ring slot `slot`, one instruction per part (tile loads,
  // then the two row vectors: the block's 32 floats, twice, since a wave load writes 64;
  // nothing outside the block is read, so no line of rows that are not published yet enters
  // this CU's L1).
  auto request_part = [&](int part, int nb, uint32_t slot) {
    const int blk = min(blk0 + min(max(nb, 0), n_blk - 1), last_blk);
    if (part < NLT) {
      const uint32_t off = partial && blk == last_blk ? ld_off_last[part] : ld_off[part];
      async_load16_to_lds(tbase + (uint32_t)(blk * kBwdBpBlk * tstride), off, ld_dst[part] + slot * SLOT_B);
    } else if (part == NLT) {
      async_load4_to_lds(neglse2 + blk * kBwdBpBlk, (lane & 31) * 4, vec_dst + slot * SLOT_B);
    } else {
      async_load4_to_lds(negdelta + blk * kBwdBpBlk, (lane & 31) * 4, vec_dst + VEC_B + slot * SLOT_B);
    }
  };
  auto request = [&](int nb, uint32_t slot) {
#pragma unroll
    for (int part = 0; part < LPI; ++part) request_part(part, nb, slot);
  };

  // K^T and V^T as B operands: lane holds row kvrow, halfs 16ks+8g .. +7.  Rows past
  // T-1 read row T-1: their keys are masked for every valid query and their rows are not stored.
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
  // The row statistics of query block qb come from the dQ workgroup that owns it (same launch,
  // same XCD).  Poll the flags of all the 128-row query blocks this workgroup will walk, one
  // per lane, before the first request; bounded, and a wait that runs out raises the error word.
  if (p.epoch != 0) {  // epoch 0: the statistics were published by an earlier launch
    for (int base = kvblk; base < n_own; base += 64) {
      const int qb = base + lane;
      const int* flag = p.ready + (int64_t)bh * n_own + min(qb, n_own - 1);
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
  }
  DEERS_TRACE_POINT(1);
#pragma unroll
  for (int nb = 0; nb <= F; ++nb) request(nb, nb % R);

  // ---- LDS read addresses of ring slot 0 (fixed; slots, the dO half and the 16-row steps are
  // instruction offsets) ----
  uint32_t aa[KS], ta_lo[DB], ta_hi[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    aa[ks] = lds0 + (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  {
    const int lrow = 4 * g + ((lane & 15) >> 2);
    const int c4 = lane & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      ta_lo[db] = lds0 + lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      ta_hi[db] = lds0 + (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }
  const uint32_t va = vec_dst + 16 * g;  // this wave's vectors: rows 4g .. (+32 rq)
  // A ring of more than 64 KB does not fit the 16-bit offset of an LDS instruction: the upper
  // half of its slots is addressed from a second set of base registers (where the slot is a
  // constant of the unrolled ring; a slot held in a register is added to the base).
  constexpr bool SPLIT = (size_t)R * SLOT_B > 65536;
  constexpr uint32_t HALF_B = (R / 2) * SLOT_B;
  uint32_t aa_hi[SPLIT ? KS : 1], ta_lo_hi[SPLIT ? DB : 1], ta_hi_hi[SPLIT ? DB : 1];
  if constexpr (SPLIT) {  // (opaque, or the compiler recomputes each of them at every use)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      aa_hi[ks] = aa[ks] + HALF_B;
      asm volatile("" : "+v"(aa_hi[ks]));
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      ta_lo_hi[db] = ta_lo[db] + HALF_B;
      ta_hi_hi[db] = ta_hi[db] + HALF_B;
      asm volatile("" : "+v"(ta_lo_hi[db]), "+v"(ta_hi_hi[db]));
    }
  }
  uint32_t va_lo[1] = {va}, va_hi[1] = {va + HALF_B};
  if constexpr (SPLIT) asm volatile("" : "+v"(va_hi[0]));
  auto slot_addr = [&](const uint32_t* lo, [[maybe_unused]] const uint32_t* hi, int idx, auto slot) -> uint32_t {
    if constexpr (SPLIT && kConstSlot<decltype(slot)>) {
      if constexpr (decltype(slot)::value >= (uint32_t)(R / 2))
        return hi[idx] + (decltype(slot)::value - R / 2) * SLOT_B;
      else
        return lo[idx] + decltype(slot)::value * SLOT_B;
    } else {
      return lo[idx] + (uint32_t)slot * SLOT_B;
    }
  };

  floatx16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) {
    dkacc[i] = ZERO16;
    dvacc[i] = ZERO16;
  }
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  half8 pf[2], dsf[2];  // P and dS of the previous block as B operands (rows 0-15, 16-31)
  half8 fr[W];          // operand fragments on their way from LDS
  wait_all_vmem();
  __syncthreads();

  // fragment mi of the MFMAs that consume the block in `slot`: (step st, output block db, dV|dK)
  // = (mi / (2 DB), (mi / 2) % DB, mi % 2); dV reads dO^T, dK reads Q^T
  auto fetch2 = [&](int mi, auto slot) -> half8 {
    const int st = mi / (2 * DB), db = (mi >> 1) % DB;
    const uint32_t off = ((mi & 1) ? 0 : TB) + 16 * st * RB;
    const half4 lo = lds_read_tr16_at(slot_addr(ta_lo, ta_lo_hi, db, slot) + off);
    const half4 hi = lds_read_tr16_at(slot_addr(ta_hi, ta_hi_hi, db, slot) + off);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // fragment mi of the MFMAs that produce the block in `slot`: (contraction step, S|dP) = (mi / 2, mi % 2)
  auto fetch1 = [&](int mi, auto slot) -> half8 {
    return lds_read_half8_at(slot_addr(aa, aa_hi, mi >> 1, slot) + ((mi & 1) ? TB : 0));
  };
  // accumulator seeds of the block in `slot`: S from -lse2, dP from -delta (row values)
  // One eighth of the accumulator seeds of the block in `slot`: part 2 rq gives S rows from
  // -lse2, part 2 rq + 1 gives dP rows from -delta (row values, the same for every lane of a half)
  auto seed_part = [&](int part, floatx16& s, floatx16& dp, auto slot) {
    const int rq = part >> 1;
    const floatx4 a = lds_read_float4_at(slot_addr(va_lo, va_hi, 0, slot) + ((part & 1) ? VEC_B : 0) + 32 * rq);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (part & 1)
        dp[4 * rq + e] = a[e];
      else
        s[4 * rq + e] = a[e];
    }
  };

  // One stage (relative block n in ring slot SLOT = n % R), entered right after its barrier.
  // (s, dp) = S and dP of block n; (sn, dpn) = those of block n+1, produced here.  FIRST: n == 0,
  // no block n-1.  A wave issues one instruction every four clocks at best, and only what
  // follows an MFMA within its 32 clocks costs nothing: so everything a stage does is spread
  // over its 16 chunks, one MFMA each: the consumers of block n-1 first (their first W fragments
  // were fetched by the previous stage), then the producers of block n+1, each followed by the
  // fetch of a fragment W MFMAs ahead (rolling into the next stage's consumers, which read
  // block n), by one of the eight seed reads, by one of the loads that refill the slot of
  // block n-2 with block n+1+F, and by the exponential, product and packing of block n.
  auto stage = [&](auto first_c, auto produce_c, auto PSLOT, auto SLOT, auto NSLOT, int n, floatx16& s,
                   floatx16& dp, floatx16& sn, floatx16& dpn) {
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr bool PRODUCE = decltype(produce_c)::value;  // false: block n+1 lies past the end
    constexpr int N2 = FIRST ? 0 : NM2, NMS = N2 + (PRODUCE ? NM1 : 0);
    constexpr int NPRE = NM2 < W ? NM2 : W;  // fragments a stage finds fetched
    // whether the fetches can roll on into the next stage (a fragment must land in the register
    // its MFMA names, which is the one just freed only if the counts are multiples of W)
    constexpr bool ROLL = (NM2 + NM1) % W == 0 && NM1 % W == 0 && NMS % W == 0;
    const uint32_t RSLOT = ((uint32_t)SLOT + 1 + F) % R;
    auto fetch = [&](int mi) -> half8 { return mi < N2 ? fetch2(mi, PSLOT) : fetch1(mi - N2, NSLOT); };
    if constexpr (FIRST) {
#pragma unroll
      for (int mi = 0; mi < W && mi < NMS; ++mi) fr[mi] = fetch(mi);
#pragma unroll
      for (int part = 0; part < 8; ++part) seed_part(part, sn, dpn, NSLOT);
    } else {
#pragma unroll
      for (int mi = NPRE; mi < W && mi < NMS; ++mi) fr[mi] = fetch(mi);
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t pw[8], dw[8];
    auto finish_pair = [&](int i) {  // f16 packing of the pair finished in chunk 2i+1
      pw[i] = pack_pair_f16(s[2 * i], s[2 * i + 1]);
      dw[i] = pack_pair_f16(dp[2 * i], dp[2 * i + 1]);
      asm volatile("" : "+v"(pw[i]), "+v"(dw[i]));
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
      for (int mi = (i * NMS + 15) / 16; mi < ((i + 1) * NMS + 15) / 16; ++mi) {  // an MFMA leads every run of chunks
        if (mi < N2) {
          const int st = mi / (2 * DB), db = (mi >> 1) % DB;
          if (mi & 1)
            dkacc[db] = mfma_f16(fr[mi % W], dsf[st], dkacc[db]);
          else
            dvacc[db] = mfma_f16(fr[mi % W], pf[st], dvacc[db]);
        } else {
          const int ks = (mi - N2) >> 1;
          if ((mi - N2) & 1)
            dpn = mfma_f16(fr[mi % W], vf[ks], dpn);
          else
            sn = mfma_f16(fr[mi % W], kf[ks], sn);
        }
        if (mi + W < NMS)
          fr[mi % W] = fetch(mi + W);
        else if (ROLL && mi + W - NMS < NPRE)
          fr[mi % W] = fetch2(mi + W - NMS, SLOT);
      }
      if (!FIRST && PRODUCE && i < 8) seed_part(i, sn, dpn, NSLOT);
      if (i >= 1 && i <= LPI) request_part(i - 1, n + 1 + F, RSLOT);
      s[i] = fast_exp2(s[i]);
      if (i > 0) dp[i - 1] = s[i - 1] * dp[i - 1];
      if (i > 2 && (i & 1)) finish_pair((i - 3) >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    dp[15] = s[15] * dp[15];
    if constexpr (!ROLL) {
#pragma unroll
      for (int mi = 0; mi < NPRE; ++mi) fr[mi] = fetch2(mi, SLOT);
    }
    finish_pair(7);
    // Causal mask, on the packed pairs: query row 32 (blk0 + n) + 8 (r/4) + 4g + r%4 of register r
    // against this lane's key.  Only the wave's first blocks have masked entries.
    // Blocks past the end (the closing stages only consume) are cleared entirely: their slots
    // hold the last block a second time.
    if ((unsigned)(n - wave - 1) >= edge_span) {  // n <= wave or n >= n_blk, one compare
      const int dist = n >= n_blk ? 64 : kvrow - 32 * (blk0 + n) - 4 * g;  // rows below dist are masked
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int qr = 8 * (i >> 1) + 2 * (i & 1);  // row offset of the pair's first register
        const uint32_t keep = (qr < dist ? 0u : 0xffffu) | (qr + 1 < dist ? 0u : 0xffff0000u);
        pw[i] &= keep;
        dw[i] &= keep;
      }
    }
    pf[0] = __builtin_bit_cast(half8, u32x4{pw[0], pw[1], pw[2], pw[3]});
    pf[1] = __builtin_bit_cast(half8, u32x4{pw[4], pw[5], pw[6], pw[7]});
    dsf[0] = __builtin_bit_cast(half8, u32x4{dw[0], dw[1], dw[2], dw[3]});
    dsf[1] = __builtin_bit_cast(half8, u32x4{dw[4], dw[5], dw[6], dw[7]});
#pragma unroll
    for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(pf[i]), "+v"(dsf[i]));
  };

  // Waves 2 and 3 have nothing in blocks 0 and 1 (every query of those lies before their keys):
  // they start their pipeline at block 2 and only keep the loads and barriers of stages 0 and 1.
  const int n0 = wave & 2;
  // ---- S, dP of block n0 (blocks 0 .. F are in LDS) ----
  floatx16 sa, dpa, sb, dpb;
#pragma unroll
  for (int part = 0; part < 8; ++part) seed_part(part, sa, dpa, n0);
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    sa = mfma_f16(fetch1(2 * ks, n0), kf[ks], sa);
    dpa = mfma_f16(fetch1(2 * ks + 1, n0), vf[ks], dpa);
  }
  // ---- stage n: barrier n retires the reads of block n-2, whose slot request(n) refills with
  // block n+1+F, and makes block n+1 (requested F stages ago) visible ----
  auto open_stage = [&]() {
    wait_vmcnt<(F - 1) * LPI>();
    // bare barrier: the LDS reads in flight (next stage's first fragments) touch slots that are
    // not refilled for two more stages
    __builtin_amdgcn_s_barrier();
  };
  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  DEERS_TRACE_POINT(2);
  for (int i = 0; i < n0; ++i) {  // stages without work: their loads and barrier
    open_stage();
    request(i + 1 + F, (uint32_t)(i + 1 + F) % R);
  }
  open_stage();
  stage(yes, yes, (uint32_t)(n0 + R - 1) % R, (uint32_t)n0, (uint32_t)n0 + 1, n0, sa, dpa, sb, dpb);
  DEERS_TRACE_POINT(3);
  auto two_stages = [&](auto slot, int n) {  // stages n (odd, ring slot `slot`) and n + 1
    const auto s1 = slot_plus<R, 1>(slot);
    const auto s2 = slot_plus<R, 2>(slot);
    open_stage();
    stage(no, yes, slot_plus<R, R - 1>(slot), slot, s1, n, sb, dpb, sa, dpa);
    open_stage();
    stage(no, yes, slot, s1, s2, n + 1, sa, dpa, sb, dpb);
  };
  auto last_two_stages = [&](uint32_t slot, int n) {  // the same without the products of blocks n+1, n+2
    const uint32_t s1 = (slot + 1) % R, s2 = (slot + 2) % R;
    open_stage();
    stage(no, no, (slot + R - 1) % R, slot, s1, n, sb, dpb, sa, dpa);
    open_stage();
    stage(no, no, slot, s1, s2, n + 1, sa, dpa, sb, dpb);
  };
  // Stages 1 .. n_blk, rounded up to an even count (the closing stages only consume: their own
  // blocks lie past the end and are cleared).  Whole turns of the ring run with every LDS
  // address a fixed register plus an instruction offset; the remaining pairs take the slot as
  // a value.  (Leaving the unrolled loop from its middle instead made the register allocator
  // copy whole accumulators at every exit: 168 spilled values.)
  const int n_total = (n_blk + 1) & ~1;
  // The last pair produces nothing: the blocks after it lie past the end.
  int n = n0 + 1;
  for (; n % R != 1 && n + 2 <= n_total; n += 2) two_stages((uint32_t)n % R, n);  // up to the ring's start
  for (; n + R + 1 <= n_total; n += R) {
    two_stages(SlotC<1>{}, n);
    two_stages(SlotC<3>{}, n + 2);
    two_stages(SlotC<5>{}, n + 4);
  }
  for (; n + 2 <= n_total; n += 2) two_stages((uint32_t)n % R, n);
  if (n <= n_total) last_two_stages((uint32_t)n % R, n);
  DEERS_TRACE_POINT(4);

  if (kvrow < T) {
    half_t* dkrow = dK + (int64_t)kvrow * p.sdk.t;
    half_t* dvrow = dV + (int64_t)kvrow * p.sdv.t;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      store_block_f16(dkrow + 32 * db, dkacc[db], kLn2, g);  // sum of dS * Q * scale * log2(e)
      store_block_f16(dvrow + 32 * db, dvacc[db], 1.f, g);
    }
  }
  DEERS_TRACE_POINT(5);
}

// ---------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void bwd_dq_f16_bp_body(const BwdParams& p, int bh, int qtile, int n_own,
                                                   [[maybe_unused]] int trace_row) {
  using Cfg = BwdBpCfg<D>;
  constexpr int R = Cfg::R, F = Cfg::F, RB = Cfg::RB, TB = Cfg::TB, SLOT_B = Cfg::SLOT_DQ;
  constexpr int KS = D / 16, DB = D / 32, CH = D / 8;
  constexpr int RPW = 1024 / RB;
  constexpr int LPI = 2 * TB / 1024 / 4;    // tile loads per wave per stage (K then V)
  constexpr int NM2 = 2 * DB;               // MFMAs that consume a block: dQ, 2 steps x DB
  constexpr int NM1 = 2 * KS;               // MFMAs that produce a block: (S, dP) x KS
  constexpr int W = 4;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;
  DEERS_TRACE_POINT(0);  // the last query block walks the most keys
  const int b_ = bh / p.H, h_ = bh % p.H;
  const half_t* Q = (const half_t*)p.q + b_ * p.sq.b + h_ * p.sq.h;
  const half_t* K = (const half_t*)p.k + b_ * p.sk.b + h_ * p.sk.h;
  const half_t* V = (const half_t*)p.v + b_ * p.sv.b + h_ * p.sv.h;
  const half_t* dO = (const half_t*)p.d_o + b_ * p.sdo.b + h_ * p.sdo.h;
  half_t* dQ = (half_t*)p.dq + b_ * p.sdq.b + h_ * p.sdq.h;
  const int q0 = qtile * kBwdBpOwn, qw0 = q0 + 32 * wave, qrow = qw0 + (lane & 31);
  const int n_blk = (min(q0 + kBwdBpOwn - 1, T - 1) >> 5) + 1;  // key blocks 0 .. n_blk-1
  const int bd = min(qw0, T - 1) >> 5;                           // this wave's diagonal block
  const int last_blk = (T - 1) >> 5;
  const uint32_t lds0 = lds_address(smem);
  const int skt = (int)p.sk.t, svt = (int)p.sv.t;
  // This wave's LPI tile loads of a stage (waves 0 and 1 fetch the K block, waves 2 and 3 the
  // V block); rows past T-1 of a last, partial block read row T-1 (masked for every query).
  constexpr int NLH = TB / 1024;
  const bool w_v = wave * LPI >= NLH;  // wave-uniform
  const half_t* tbase = w_v ? V : K;
  const int tstride = w_v ? svt : skt;
  const bool partial = (T & (kBwdBpBlk - 1)) != 0;
  uint32_t ld_off[LPI], ld_off_last[LPI], ld_dst[LPI];
#pragma unroll
  for (int i = 0; i < LPI; ++i) {
    const int n = (wave * LPI + i) % NLH;
    const int row = n * RPW + lane / CH;
    const int col = 16 * ((lane % CH) ^ lds_swizzle<CH>(row));
    ld_off[i] = (uint32_t)(row * tstride * 2 + col);
    ld_off_last[i] = (uint32_t)(min(row, T - 1 - last_blk * kBwdBpBlk) * tstride * 2 + col);
    ld_dst[i] = lds0 + (w_v ? TB : 0) + n * 1024;
  }
  auto request_part = [&](int part, int nb, uint32_t slot) {
    const int blk = min(max(nb, 0), n_blk - 1);
    const uint32_t off = partial && blk == last_blk ? ld_off_last[part] : ld_off[part];
    async_load16_to_lds(tbase + (uint32_t)(blk * kBwdBpBlk * tstride), off, ld_dst[part] + slot * SLOT_B);
  };
  auto request = [&](int nb, uint32_t slot) {
#pragma unroll
    for (int part = 0; part < LPI; ++part) request_part(part, nb, slot);
  };

  // Q (scaled) and dO as B operands.  Rows past T-1 read row T-1: their dQ rows are not stored
  // and a query owns its accumulator column.
  half8 qf[KS], dof[KS];
  {
    const int lrow = min(qrow, T - 1);
    const half_t* qp = Q + (int64_t)lrow * p.sq.t + 8 * g;
    const half_t* dop = dO + (int64_t)lrow * p.sdo.t + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[ks] = *(const half8*)(qp + 16 * ks);
      dof[ks] = *(const half8*)(dop + 16 * ks);
    }
  }
#pragma unroll
  for (int nb = 0; nb <= F; ++nb) request(nb, nb % R);
  // This row's statistics, published for the dK/dV role: rows in the padding [T, t_pad) get
  // -lse2 = -inf and -delta = 0, i.e. probability 0.
  float nl2, nd;
  {
    const int lrow = min(qrow, T - 1);
    const half_t* op = (const half_t*)p.o + b_ * p.so.b + h_ * p.so.h + (int64_t)lrow * p.so.t + 8 * g;
    half8 of[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) of[ks] = *(const half8*)(op + 16 * ks);
    const float lse_row = p.lse[(int64_t)bh * T + lrow];
    float dsum = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) dsum += (float)dof[ks][e] * (float)of[ks][e];
    if (qrow >= T) dsum = 0.f;
    nd = -pair_sum(dsum);
    nl2 = qrow < T ? -lse_row * kLog2e : -INFINITY;
    if (g == 0 && qrow < p.t_pad) {
      p.lse2[(int64_t)bh * p.t_pad + qrow] = nl2;
      p.negdelta[(int64_t)bh * p.t_pad + qrow] = nd;
    }
  }
  floatx16 nl16, nd16;  // initial values of the S^T and dP^T accumulators (this lane's query)
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    nl16[r] = nl2;
    nd16[r] = nd;
  }
  uint32_t aa[KS], ta_lo[DB], ta_hi[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    aa[ks] = lds0 + (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  {
    const int lrow = 4 * g + ((lane & 15) >> 2);
    const int c4 = lane & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      ta_lo[db] = lds0 + lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      ta_hi[db] = lds0 + (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }
  // (as in the dK/dV role: a second set of base registers for the upper half of a ring over 64 KB)
  constexpr bool SPLIT = (size_t)R * SLOT_B > 65536;
  constexpr uint32_t HALF_B = (R / 2) * SLOT_B;
  uint32_t aa_hi[SPLIT ? KS : 1], ta_lo_hi[SPLIT ? DB : 1], ta_hi_hi[SPLIT ? DB : 1];
  if constexpr (SPLIT) {  // (opaque, or the compiler recomputes each of them at every use)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      aa_hi[ks] = aa[ks] + HALF_B;
      asm volatile("" : "+v"(aa_hi[ks]));
    }
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      ta_lo_hi[db] = ta_lo[db] + HALF_B;
      ta_hi_hi[db] = ta_hi[db] + HALF_B;
      asm volatile("" : "+v"(ta_lo_hi[db]), "+v"(ta_hi_hi[db]));
    }
  }
  auto slot_addr = [&](const uint32_t* lo, [[maybe_unused]] const uint32_t* hi, int idx, auto slot) -> uint32_t {
    if constexpr (SPLIT && kConstSlot<decltype(slot)>) {
      if constexpr (decltype(slot)::value >= (uint32_t)(R / 2))
        return hi[idx] + (decltype(slot)::value - R / 2) * SLOT_B;
      else
        return lo[idx] + decltype(slot)::value * SLOT_B;
    } else {
      return lo[idx] + (uint32_t)slot * SLOT_B;
    }
  };
  floatx16 dqacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) dqacc[i] = ZERO16;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  half8 dsf[2];
  half8 fr[W];
  wait_all_vmem();
  {
    const float c = p.scale_log2;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[ks][e] = (half_t)((float)qf[ks][e] * c);
  }
  // The scaled queries go to the workspace: the dK/dV role forms its scores from these very
  // values, as the forward did, so that all three exponentiate identical scores (with the
  // scale folded into K there instead, scores differed by up to |S| * 2^-11 and a dominant
  // probability by 0.2 %).
  if (qrow < T) {
    half_t* qs = (half_t*)p.qs + ((int64_t)bh * p.t_pad + qrow) * D + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) *(half8*)(qs + 16 * ks) = qf[ks];
  }
  __syncthreads();  // every wave's first blocks have landed (the stores drain under the first products)

  auto fetch2 = [&](int mi, auto slot) -> half8 {  // dQ: (step, output block) = (mi / DB, mi % DB), K^T
    const int st = mi / DB, db = mi % DB;
    const uint32_t off = 16 * st * RB;
    const half4 lo = lds_read_tr16_at(slot_addr(ta_lo, ta_lo_hi, db, slot) + off);
    const half4 hi = lds_read_tr16_at(slot_addr(ta_hi, ta_hi_hi, db, slot) + off);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto fetch1 = [&](int mi, auto slot) -> half8 {  // (contraction step, S|dP) = (mi / 2, mi % 2): K rows | V rows
    return lds_read_half8_at(slot_addr(aa, aa_hi, mi >> 1, slot) + ((mi & 1) ? TB : 0));
  };

  // One stage, spread over 16 chunks as in the dK/dV role: the consumers of block n-1 (dQ), the
  // producers of block n+1 (S^T, dP^T), the rolling fragment fetches, the loads that refill the
  // slot of block n-2, and the vector ops of block n.
  auto stage = [&](auto first_c, auto produce_c, auto PSLOT, auto SLOT, auto NSLOT, int n, floatx16& s,
                   floatx16& dp, floatx16& sn, floatx16& dpn) {
    constexpr bool FIRST = decltype(first_c)::value;
    constexpr bool PRODUCE = decltype(produce_c)::value;  // false: block n+1 lies past the wave's diagonal
    constexpr int N2 = FIRST ? 0 : NM2, NMS = N2 + (PRODUCE ? NM1 : 0);
    constexpr int NPRE = NM2 < W ? NM2 : W;
    constexpr bool ROLL = (NM2 + NM1) % W == 0 && NM1 % W == 0 && NMS % W == 0;
    const uint32_t RSLOT = ((uint32_t)SLOT + 1 + F) % R;
    auto fetch = [&](int mi) -> half8 { return mi < N2 ? fetch2(mi, PSLOT) : fetch1(mi - N2, NSLOT); };
#pragma unroll
    for (int mi = FIRST ? 0 : NPRE; mi < W && mi < NMS; ++mi) fr[mi] = fetch(mi);
    __builtin_amdgcn_sched_barrier(0);
    uint32_t dw[8];
    auto finish_pair = [&](int i) {
      dw[i] = pack_pair_f16(dp[2 * i], dp[2 * i + 1]);
      asm volatile("" : "+v"(dw[i]));
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
      for (int mi = (i * NMS + 15) / 16; mi < ((i + 1) * NMS + 15) / 16; ++mi) {  // an MFMA leads every run of chunks
        if (mi < N2) {
          const int st = mi / DB, db = mi % DB;
          dqacc[db] = mfma_f16(fr[mi % W], dsf[st], dqacc[db]);
        } else {
          const int ks = (mi - N2) >> 1;
          if ((mi - N2) & 1)
            dpn = mfma_f16(fr[mi % W], dof[ks], ks == 0 ? nd16 : dpn);
          else
            sn = mfma_f16(fr[mi % W], qf[ks], ks == 0 ? nl16 : sn);
        }
        if (mi + W < NMS)
          fr[mi % W] = fetch(mi + W);
        else if (ROLL && mi + W - NMS < NPRE)
          fr[mi % W] = fetch2(mi + W - NMS, SLOT);
      }
      if (i >= 1 && i <= LPI) request_part(i - 1, n + 1 + F, RSLOT);
      s[i] = fast_exp2(s[i]);
      if (i > 0) dp[i - 1] = s[i - 1] * dp[i - 1];
      if (i > 2 && (i & 1)) finish_pair((i - 3) >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    dp[15] = s[15] * dp[15];
    if constexpr (!ROLL) {
#pragma unroll
      for (int mi = 0; mi < NPRE; ++mi) fr[mi] = fetch2(mi, SLOT);
    }
    finish_pair(7);
    // Causal mask on the packed pairs: key 32 n + 8 (r/4) + 4g + r%4 of register r against this
    // lane's query; from the wave's diagonal block on (blocks beyond it are masked entirely).
    if (n >= bd) {
      const int dist = qrow - 4 * g - 32 * n;  // keys above dist are masked
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int kr = 8 * (i >> 1) + 2 * (i & 1);
        const uint32_t keep = (kr > dist ? 0u : 0xffffu) | (kr + 1 > dist ? 0u : 0xffff0000u);
        dw[i] &= keep;
      }
    }
    dsf[0] = __builtin_bit_cast(half8, u32x4{dw[0], dw[1], dw[2], dw[3]});
    dsf[1] = __builtin_bit_cast(half8, u32x4{dw[4], dw[5], dw[6], dw[7]});
#pragma unroll
    for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(dsf[i]));
  };

  floatx16 sa, dpa, sb, dpb;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    sa = mfma_f16(fetch1(2 * ks, 0), qf[ks], ks == 0 ? nl16 : sa);
    dpa = mfma_f16(fetch1(2 * ks + 1, 0), dof[ks], ks == 0 ? nd16 : dpa);
  }
  auto open_stage = [&]() {
    wait_vmcnt<(F - 1) * LPI>();
    __builtin_amdgcn_s_barrier();
  };
  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  DEERS_TRACE_POINT(2);
  // The first stage's barrier doubles as the hand-over: every wave has drained its stores of the
  // statistics and of the scaled queries before it, the rows are in the XCD's L2, tell the
  // dK/dV workgroups.
  wait_all_vmem();
  __builtin_amdgcn_s_barrier();
  if (tid == 0)
    __hip_atomic_store(p.ready + (int64_t)bh * n_own + qtile, p.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  stage(yes, yes, R - 1, 0, 1, 0, sa, dpa, sb, dpb);
  DEERS_TRACE_POINT(3);
  auto two_stages = [&](auto slot, int n) {  // stages n (odd, ring slot `slot`) and n + 1
    const auto s1 = slot_plus<R, 1>(slot);
    const auto s2 = slot_plus<R, 2>(slot);
    open_stage();
    stage(no, yes, slot_plus<R, R - 1>(slot), slot, s1, n, sb, dpb, sa, dpa);
    open_stage();
    stage(no, yes, slot, s1, s2, n + 1, sa, dpa, sb, dpb);
  };
  auto last_two_stages = [&](uint32_t slot, int n) {  // the same without the products of blocks n+1, n+2
    const uint32_t s1 = (slot + 1) % R, s2 = (slot + 2) % R;
    open_stage();
    stage(no, no, (slot + R - 1) % R, slot, s1, n, sb, dpb, sa, dpa);
    open_stage();
    stage(no, no, slot, s1, s2, n + 1, sa, dpa, sb, dpb);
  };
  // Stages 1 .. n_blk, rounded up to an even count (the closing stages only consume: their own
  // blocks lie past the end and are cleared).  Whole turns of the ring run with every LDS
  // address a fixed register plus an instruction offset; the remaining pairs take the slot as
  // a value.  (Leaving the unrolled loop from its middle instead made the register allocator
  // copy whole accumulators at every exit: 168 spilled values.)
  const int n_total = (n_blk + 1) & ~1;
  // A wave's last block is its diagonal block bd, consumed in stage bd + 1: the pairs after that
  // stage have nothing for it but the barriers (the loads of those stages are never consumed).
  const int n_live = min(n_total, (bd + 2) & ~1);
  // Its last live pair produces nothing: the blocks after it lie past its diagonal.
  int n = 1;
  for (; n + R + 1 <= n_live; n += R) {
    two_stages(SlotC<1>{}, n);
    two_stages(SlotC<3>{}, n + 2);
    two_stages(SlotC<5>{}, n + 4);
  }
  for (; n + 2 <= n_live; n += 2) two_stages((uint32_t)n % R, n);
  if (n <= n_live) {
    last_two_stages((uint32_t)n % R, n);
    n += 2;
  }
  for (; n <= n_total; n += 2) {
    open_stage();
    open_stage();
  }
  DEERS_TRACE_POINT(4);

  if (qrow < T) {
    half_t* dqrow = dQ + (int64_t)qrow * p.sdq.t;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_block_f16(dqrow + 32 * db, dqacc[db], p.scale, g);
  }
  DEERS_TRACE_POINT(5);
}

}  // namespace deers
