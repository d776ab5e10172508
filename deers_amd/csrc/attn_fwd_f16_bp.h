// Block-pipelined causal attention forward (f16 storage, f32 accumulate, gfx950): the device
// body, shared by the library kernel (attn_fwd_f16.hip) and by the micro-benchmark that times
// its steady-state loop (microbench/simd_mfma_valu.hip).
#pragma once
#include <type_traits>

#include "common.h"

namespace deers {

constexpr int kFwdBM = 128;  // query rows per workgroup
constexpr int kFwdBN = 64;   // key/value rows per tile

#ifndef ZERO16
#define ZERO16 floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#endif

template <int D>
struct FwdCfg {
  // prefetch distance in tiles; D = 128 keeps one tile less in flight so that two
  // workgroups' rings (2 x 64 KB) share a CU
  static constexpr int P = D == 128 ? 1 : 2;
  static constexpr int NS = P + 1;              // ring slots per tensor
  static constexpr int RB = D * 2;              // row bytes
  static constexpr int TILE_B = kFwdBN * RB;    // tile bytes
  static constexpr size_t kLds = 2 * NS * TILE_B;
};

// Position -> tile table of a launch whose workgroups are all resident at once, passed in
// the kernel arguments: entry p = (head index within the XCD) << 16 | query tile for the
// workgroup at position p = blockIdx.x / 8 of its XCD.
constexpr int kMaxResidentTiles = 128;  // per XCD: 32 CUs x at most 4 workgroups
struct TileOrder {
  int32_t code[kMaxResidentTiles];
};

// ---- block-pipelined kernel: matrix and vector work interleaved inside every wave ----
// What one SIMD does with this loop's instructions (measured, see microbench/simd_mfma_valu.hip):
// an MFMA that has to wait for the matrix pipe holds the vector issue port, so a wave that
// issues MFMAs back to back stalls every other wave's vector work, and two waves in different
// phases do not overlap; but the vector ops that FOLLOW an MFMA in the same wave issue while it
// executes, about four of them per MFMA for free (two of which may be exponentials), and
// v_dot2_f32_f16 costs 16 clocks beside an MFMA where an add costs 3.  So the loop is cut into
// chunks of one MFMA and the softmax of two scores, and everything that is not the exponential,
// the f16 packing and the row sum is taken off the vector pipe:
//   * scale * log2(e) is folded into the f16 Q fragments once per workgroup;
//   * the score accumulator starts from -m (the row's reference maximum), so the MFMA result is
//     already the exponent; -m is kept in LDS, four copies per lane, and four 16-byte reads fill
//     the accumulator with it (no vector-pipe work, no 16 registers set aside);
//   * the reference maximum is the maximum of the row's first 32 keys and is only replaced when a
//     block's probabilities approach the f16 range (sum of a lane's 16 values > 6e4; then that
//     block is recomputed from global memory against its true maximum, a cold path); between
//     those events no maxima are formed at all;
//   * row sums are plain f32 adds of the exponentials.
// The unit of the pipeline is a 32-key block: in stage b the wave issues the MFMAs of
// O += V(b-1) P(b-1) and of S(b+1) between the exponentials of S(b).  K and V blocks travel
// global -> LDS asynchronously into rings, F stages ahead, one barrier per stage; a block has
// landed one barrier before its first use, so the first V fragments of a stage leave LDS at the
// end of the stage before it, across the barrier, and the K fragments (needed in the stage's
// second half) right after it.  Inside a stage nothing is conditional (a branch around a single
// MFMA costs a lone wave more than the MFMA: eight such branches per stage were 23 % of the
// stage); what a wave leaves out it leaves out in whole stages at the end of its walk: the
// pair of stages at its diagonal block forms no further scores, and after it the wave only
// keeps the workgroup's barriers and its share of the loads.
// Hook for a timestamp-tracing build of this kernel; expands to nothing in the library.
#ifndef DEERS_TRACE_POINT
#define DEERS_TRACE_POINT(slot)
#endif
constexpr float kF16SumGuard = 60000.f;
constexpr int kBpBlk = 32;  // keys per block / stage
#ifndef BP_OCC
#define BP_OCC 3
#endif

template <int D>
struct BpCfg {
  static constexpr int R = D == 128 ? 4 : 6;     // ring slots (blocks) per tensor
  static constexpr int F = R - 2;                // stages between a block's request and its barrier
  static constexpr int RB = D * 2;               // row bytes
  static constexpr int TB = kBpBlk * RB;         // block bytes
  static constexpr int NL = 2 * TB / 1024;       // 1 KiB wave loads per stage (K then V)
  static constexpr int LPI = NL / 4;             // per wave
  static constexpr size_t kRings = (size_t)(2 * R) * TB;
  static constexpr size_t kLds = kRings + 4 * 1024;  // + per wave: -m of each lane's row, four times over
};

// BENCH (micro-benchmark build of the same body): the loop runs `bench_stages` stages of a long
// row with no diagonal in reach and the wave's clocks around the loop go to `bench_clk`.
template <int D, bool BENCH>
__device__ __forceinline__ void attn_fwd_f16_bp_body(const FwdParams& p, int BH, int n_qtiles, int heads_per_xcd,
                                                     const TileOrder& order, int bench_stages, long long* bench_clk) {
  using Cfg = BpCfg<D>;
  constexpr int R = Cfg::R, F = Cfg::F, RB = Cfg::RB, TB = Cfg::TB, LPI = Cfg::LPI;
  constexpr int KS = D / 16, DB = D / 32, CH = D / 8;
  constexpr int RPW = 1024 / RB;                    // block rows covered by one 1 KiB wave load
  constexpr int W = 4;                              // operand fragments in flight ahead of their MFMA
  constexpr int NPF = 2 * DB < W ? 2 * DB : W;      // V fragments fetched ahead of a stage
  extern __shared__ __attribute__((aligned(1024))) char smem[];  // K ring, V ring, seeds
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;
  int bh, qtile;
  if (order.code[0] >= 0) {
    const int code = order.code[blockIdx.x >> 3];
    bh = (code >> 16) * 8 + (blockIdx.x & 7);
    qtile = code & 0xffff;
    if (bh >= BH) return;
  } else {
    int rank;
    if (!map_block(blockIdx.x, n_qtiles, heads_per_xcd, BH, &bh, &rank)) return;
    qtile = n_qtiles - 1 - rank;
  }
  qtile = __builtin_amdgcn_readfirstlane(qtile);
  bh = __builtin_amdgcn_readfirstlane(bh);
  [[maybe_unused]] const int trace_row = blockIdx.x;
  DEERS_TRACE_POINT(0);
  const int b_ = bh / p.H, h_ = bh % p.H;
  const half_t* Q = (const half_t*)p.q + b_ * p.sq.b + h_ * p.sq.h;
  const half_t* K = (const half_t*)p.k + b_ * p.sk.b + h_ * p.sk.h;
  const half_t* V = (const half_t*)p.v + b_ * p.sv.b + h_ * p.sv.h;
  half_t* O = (half_t*)p.o + b_ * p.so.b + h_ * p.so.h;
  const int q0 = qtile * kFwdBM, qw0 = q0 + 32 * wave, qrow = qw0 + (lane & 31);
  // blocks the workgroup reads (the last wave's diagonal block is the last one) and this wave's
  // own diagonal block
  const int n_blk = BENCH ? bench_stages : (min(q0 + kFwdBM - 1, T - 1) >> 5) + 1;
  const int bd = BENCH ? (1 << 28) : min(qw0, T - 1) >> 5;
  const uint32_t lds0 = lds_address(smem);
  const int last_blk = (T - 1) >> 5;  // the block that holds row T-1: its rows are clamped
  const int skt = (int)p.sk.t, svt = (int)p.sv.t;
  // This wave's LPI loads of a stage (waves 0 and 1 fetch the K block, waves 2 and 3 the V
  // block; a load covers RPW rows).  lane -> (row, 16-byte chunk), chunk swizzled; rows past T-1
  // of a last, partial block read row T-1.
  constexpr int NLH = Cfg::NL / 2;
  const bool w_v = wave * LPI >= NLH;  // wave-uniform
  const half_t* tbase = w_v ? V : K;
  const int tstride = w_v ? svt : skt;
  const bool partial = (T & (kBpBlk - 1)) != 0;
  uint32_t ld_off[LPI], ld_off_last[LPI], ld_dst[LPI];
#pragma unroll
  for (int i = 0; i < LPI; ++i) {
    const int n = (wave * LPI + i) % NLH;
    const int row = n * RPW + lane / CH;
    const int col = 16 * ((lane % CH) ^ lds_swizzle<CH>(row));
    ld_off[i] = (uint32_t)(row * tstride * 2 + col);
    ld_off_last[i] = (uint32_t)(min(row, T - 1 - last_blk * kBpBlk) * tstride * 2 + col);
    ld_dst[i] = lds0 + (w_v ? R * TB : 0) + n * 1024;
  }
  // Load `part` of the request of K block kb into ring slot kslot and V block vb into vslot.
  // Blocks outside [0, n_blk) are clamped: they are never consumed.
  auto request_part = [&](int part, int kb, int vb, uint32_t kslot, uint32_t vslot) {
    const int want = w_v ? vb : kb;
    const int blk = BENCH ? (want & 15) : min(max(want, 0), n_blk - 1);
    const uint32_t off = partial && blk == last_blk ? ld_off_last[part] : ld_off[part];
    async_load16_to_lds(tbase + (uint32_t)(blk * kBpBlk * tstride), off, ld_dst[part] + (w_v ? vslot : kslot) * TB);
  };
  auto request = [&](int kb, int vb, uint32_t kslot, uint32_t vslot) {
#pragma unroll
    for (int part = 0; part < LPI; ++part) request_part(part, kb, vb, kslot, vslot);
  };
  // Q fragments first (ordinary loads), then K(0) .. K(F), V(0) .. V(F-1)
  half8 qf[KS];
  {
    const half_t* qp = Q + (int64_t)min(qrow, T - 1) * p.sq.t + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const half8*)(qp + 16 * ks);
  }
#pragma unroll
  for (int s = -F - 1; s < 0; ++s) request(s + 1 + F, s + F, (s + 1 + F) % R, (s + F + R) % R);

  // LDS read addresses of ring slot 0, fixed: K rows as row-major A fragments (row lane%32,
  // chunk 2ks+g), V as transposed fragments (see lds_read_tr16).  Slots and the 16-key steps of
  // a block are instruction offsets: the stage loop is unrolled over the ring.
  uint32_t ka[KS], va_lo[DB], va_hi[DB];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    ka[ks] = lds0 + (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  {
    const int lrow = 4 * g + ((lane & 15) >> 2);
    const int c4 = lane & 3;
    const uint32_t base = lds0 + R * TB;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      va_lo[db] = base + lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      va_hi[db] = base + (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }
  floatx16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) oacc[i] = ZERO16;
  float m = -INFINITY, lsum = 0.f;  // m in units of the scaled scores (log2 domain)
  half8 pf[2];                      // P of the previous block as B operands (keys 0-15, 16-31)
  half8 fr[W];                      // operand fragments on their way from LDS
  wait_all_vmem();
  DEERS_TRACE_POINT(1);
  {  // fold scale * log2(e) into Q (one rounding to f16)
    const float c = p.scale_log2;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[ks][e] = (half_t)((float)qf[ks][e] * c);
  }
  __syncthreads();

  // Causal mask of a 32-key block starting at key kb0, in place (tied operands: a select
  // written in C++ left the choice of registers to the allocator, which copied the whole
  // accumulator in every stage, masked or not).
  auto mask_block = [&](floatx16& s, int kb0) {
    const int dist = qrow - 4 * g - kb0;
    const float ninf = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      asm volatile("v_cmp_gt_i32_e32 vcc, %2, %1\n\tv_cndmask_b32_e32 %0, %0, %3, vcc"
                   : "+v"(s[r])
                   : "v"(dist), "n"(8 * (r >> 2) + (r & 3)), "v"(ninf)
                   : "vcc");
  };
  auto row_max = [&](const floatx16& s) {
    float mx4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) mx4[i] = s[i];
#pragma unroll
    for (int r = 4; r < 16; r += 2) mx4[(r >> 1) & 3] = fmaxf(fmaxf(mx4[(r >> 1) & 3], s[r]), s[r + 1]);
    return pair_max(fmaxf(fmaxf(mx4[0], mx4[1]), fmaxf(mx4[2], mx4[3])));
  };
  // -m of this lane's row, four copies: lane l of wave w owns 16 bytes at seed_at
  const uint32_t seed_at = lds0 + (uint32_t)Cfg::kRings + wave * 1024 + lane * 16;
  auto set_negm = [&]() { *(DEERS_LDS floatx4*)(uintptr_t)seed_at = floatx4{-m, -m, -m, -m}; };
  auto seed_part = [&](int j, floatx16& s) {  // registers 4j .. 4j+3 of s = -m
    // volatile: four separate reads (one read and twelve register moves otherwise)
    const floatx4 x = *(volatile DEERS_LDS const floatx4*)(uintptr_t)seed_at;
#pragma unroll
    for (int e = 0; e < 4; ++e) s[4 * j + e] = x[e];
  };
  // V fragment j of the block in ring slot `slot` (16-key step j / DB, output rows 32 (j % DB) ..)
  // and K fragment ks of the block in `slot`
  auto fetch_v = [&](int j, uint32_t slot) -> half8 {
    const int ms = j / DB, db = j % DB;
    const half4 lo = lds_read_tr16_at(va_lo[db] + slot * TB + 16 * ms * RB);
    const half4 hi = lds_read_tr16_at(va_hi[db] + slot * TB + 16 * ms * RB);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto fetch_k = [&](int ks, uint32_t slot) -> half8 { return lds_read_half8_at(ka[ks] + slot * TB); };

  // One stage (block b, ring slot SLOT = b % R), entered right after its barrier.  cur = S(b)
  // (already -m unless FIRST), nxt = S(b+1) to be produced (only while b is before the wave's
  // diagonal block; from there on the wave sees masked blocks).  FIRST: b == 0, cur is the raw
  // product and fixes m, and there is no block b-1; otherwise the first NPF V fragments of
  // block b-1 are in fr.  MFMA order: PV, then S.  A wave issues one instruction every four
  // clocks at best and only what follows an MFMA within its 32 clocks costs nothing, so the
  // stage's other work is spread over its eight chunks: the fetch of a fragment W MFMAs ahead
  // (rolling into the next stage's first V fragments), the four seed reads, the loads that
  // refill the slots of K(b) and V(b-2), and the exponentials, sums and packing of block b.
  // One body serves every position of a wave: variants per position made the register
  // allocator spill hundreds of values.
  auto stage = [&](auto first_c, auto produce_c, auto slot_c, int b, floatx16& cur, floatx16& nxt) {
    constexpr bool FIRST = decltype(first_c)::value, HAS_PV = !FIRST;
    constexpr bool PRODUCE = decltype(produce_c)::value;  // false: block b + 1 lies past the wave's diagonal
    const uint32_t SLOT = (uint32_t)slot_c;  // a constant in the unrolled ring, a value in the last pair
    const uint32_t KSLOT = (SLOT + 1) % R, VSLOT = (SLOT + R - 1) % R;
    constexpr int NPV = HAS_PV ? 2 * DB : 0, NMS = PRODUCE ? KS : 0, NM = NPV + NMS;
    constexpr int NPRE = HAS_PV ? NPF : 0;  // fragments already in fr
    constexpr bool ROLL = NM % W == 0;      // a fetched fragment lands in the register its MFMA names
    const bool masked = b >= bd;  // block b is the wave's diagonal block, or lies beyond it
    auto fetch = [&](int mi) -> half8 { return mi < NPV ? fetch_v(mi, VSLOT) : fetch_k(mi - NPV, KSLOT); };
#pragma unroll
    for (int mi = NPRE; mi < W && mi < NM; ++mi) fr[mi] = fetch(mi);
    if constexpr (FIRST) {
      if (masked) mask_block(cur, 32 * b);
      m = row_max(cur);
      set_negm();
    }
    if constexpr (FIRST) {
#pragma unroll
      for (int j = 0; j < 4; ++j) seed_part(j, nxt);
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t pw[8];
    float bs0, bs1;
    auto finish_pair = [&](int i) {  // f16 packing and row sum of the pair exponentiated in chunk i
      pw[i] = __builtin_bit_cast(uint32_t, half2v{(half_t)cur[2 * i], (half_t)cur[2 * i + 1]});
      if (i == 0) {
        bs0 = cur[0];
        bs1 = cur[1];
      } else {
        bs0 += cur[2 * i];
        bs1 += cur[2 * i + 1];
      }
      asm volatile("" : "+v"(pw[i]), "+v"(bs0), "+v"(bs1));
    };
#pragma unroll
    for (int i = 0; i < 8; ++i) {
#pragma unroll
      for (int mi = i * NM / 8; mi < (i + 1) * NM / 8; ++mi) {
        if (mi < NPV) {
          const int ms = mi / DB, db = mi % DB;
          oacc[db] = mfma_f16(fr[mi % W], pf[ms], oacc[db]);
        } else {
          const int ks = mi - NPV;
          nxt = mfma_f16(fr[mi % W], qf[ks], nxt);
        }
        if (mi + W < NM)
          fr[mi % W] = fetch(mi + W);
        else if (ROLL && mi + W - NM < NPF)
          fr[mi % W] = fetch_v(mi + W - NM, SLOT);  // the next stage multiplies V(b) by P(b)
      }
      if (!FIRST && PRODUCE && i < 4) seed_part(i, nxt);
      if (i >= 1 && i <= LPI) request_part(i - 1, b + 1 + F, b + F, (SLOT + 1 + F) % R, (SLOT + F) % R);
      if constexpr (FIRST) {
        cur[2 * i] = fast_exp2(cur[2 * i] - m);
        cur[2 * i + 1] = fast_exp2(cur[2 * i + 1] - m);
      } else {
        cur[2 * i] = fast_exp2(cur[2 * i]);
        cur[2 * i + 1] = fast_exp2(cur[2 * i + 1]);
      }
      if (i > 0) finish_pair(i - 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (!ROLL) {
#pragma unroll
      for (int j = 0; j < NPF; ++j) fr[j] = fetch_v(j, SLOT);
    }
    finish_pair(7);
    float bsum = bs0 + bs1;
    if constexpr (!FIRST) {
      if (masked) {
        // Diagonal block (or a block beyond it, whose scores were never formed): the masked
        // entries went through the exponential as they were; clear them in the packed pairs and
        // take the row sum from what is left.  (Masking the scores themselves, a conditional
        // change of a whole accumulator, cost sixteen register moves in EVERY stage.)
        const int dist = qrow - 4 * g - 32 * b;
        bsum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int kr = 8 * (i >> 1) + 2 * (i & 1);  // key of the pair's first score; the second is kr + 1
          const uint32_t keep = (kr > dist ? 0u : 0xffffu) | (kr + 1 > dist ? 0u : 0xffff0000u);
          pw[i] &= keep;
          bsum = add_half2(__builtin_bit_cast(half2v, pw[i]), bsum);
        }
      }
    }
    if (__builtin_expect(__any(bsum > kF16SumGuard), 0)) {
      // Cold path: some probability of this block may not fit f16 against the reference maximum
      // in use.  Recompute the block's scores from global memory, move the reference to the
      // true maximum, rescale what has been accumulated and redo the block against it.
      floatx16 s = ZERO16;
      {
        const half_t* kp = K + (int64_t)min(32 * b + (lane & 31), T - 1) * p.sk.t + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = mfma_f16(*(const half8*)(kp + 16 * ks), qf[ks], s);
      }
      // The compiler's wait states between an MFMA and a read of its result follow the program
      // text, not the branches: with the mask skipped, the row maximum below read the result
      // one instruction after the last MFMA (seen on the device as sporadic infinities).
      asm volatile("s_nop 15\n\ts_nop 15" : "+v"(s));  // tied to s: after its MFMAs, before its readers
      if (masked) mask_block(s, 32 * b);
      const float m_new = fmaxf(m, row_max(s));
      const float shift = m - m_new;  // <= 0
      const float alpha = fast_exp2(shift);
      m = m_new;
      lsum *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
#pragma unroll
      for (int r = 0; r < 16; ++r) nxt[r] += shift;
      set_negm();
      bsum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float e0 = fast_exp2(s[2 * i] - m), e1 = fast_exp2(s[2 * i + 1] - m);
        bsum += e0 + e1;
        pw[i] = __builtin_bit_cast(uint32_t, half2v{(half_t)e0, (half_t)e1});
      }
    }
    lsum += bsum;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    pf[0] = __builtin_bit_cast(half8, u32x4{pw[0], pw[1], pw[2], pw[3]});
    pf[1] = __builtin_bit_cast(half8, u32x4{pw[4], pw[5], pw[6], pw[7]});
#pragma unroll
    for (int i = 0; i < 2; ++i) asm volatile("" : "+v"(pf[i]));
    asm volatile("" : "+v"(lsum));
  };

  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  // ---- S(0) ----
  floatx16 sa, sb;
  sa = ZERO16;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) sa = mfma_f16(fetch_k(ks, 0), qf[ks], sa);

  // ---- stage b: barrier b retires the reads of K(b) and V(b-2), whose slots request(b) refills
  // (with K(b+1+F) and V(b+F); both rings have F + 2 slots), and makes K(b+1) and V(b), requested
  // F stages ago, visible ----
  auto open_stage = [&]() {
    wait_vmcnt<(F - 1) * LPI>();
    // A bare barrier: no wait for the LDS reads in flight.  Those are the next stage's first V
    // fragments and the seed, whose slots are not refilled for another stage; every read of the
    // two slots the request refills has been consumed by an MFMA this wave issued already.
    __builtin_amdgcn_s_barrier();
  };
  open_stage();
  stage(yes, yes, std::integral_constant<int, 0>{}, 0, sa, sb);
  DEERS_TRACE_POINT(2);
  [[maybe_unused]] const long long bench_t0 = BENCH ? clock64() : 0;
  // Stages come two at a time (an odd count runs one more, fully masked stage).  A wave's last
  // block is its diagonal block bd, consumed in stage bd + 1: after the pair that holds that
  // stage the wave only keeps the workgroup's barriers and its share of the loads.  (Any path
  // AROUND a stage body inside the walk made the register allocator spill 100-700 values; leaving
  // the walk early does not.)  The loop body is one turn of the ring, so that every LDS address
  // is a fixed register plus an instruction offset.
  auto two_stages = [&](auto produce_c, auto slot_c, int b) {  // stages b (odd) and b + 1
    const uint32_t slot = (uint32_t)slot_c;
    open_stage();
    stage(no, produce_c, slot_c, b, sb, sa);
    open_stage();
    if constexpr (std::is_integral_v<decltype(slot_c)>)
      stage(no, produce_c, (slot + 1) % R, b + 1, sa, sb);
    else
      stage(no, produce_c, std::integral_constant<int, (decltype(slot_c)::value + 1) % R>{}, b + 1, sa, sb);
    DEERS_TRACE_POINT(3 + (b >> 1));
  };
  const int n_total = (n_blk + 1) & ~1;                              // the workgroup's last stage
  const int n_live = BENCH ? n_total : min(n_total, (bd + 2) & ~1);  // this wave's last stage with work
  // The wave's last pair of stages, (n_live - 1, n_live), lies at or past its diagonal block:
  // it forms no further scores.
  const int b_last = BENCH ? n_live + 1 : n_live - 1;
  // Whole turns of the ring run with constant slots; the remaining pairs take the slot as a
  // value.  (Leaving the unrolled turn from its middle made the register allocator spill.)
  int b = 1;
  for (; b + R <= b_last; b += R) {
    two_stages(yes, std::integral_constant<int, 1>{}, b);
    two_stages(yes, std::integral_constant<int, 3 % R>{}, b + 2);
    if constexpr (R == 6) two_stages(yes, std::integral_constant<int, 5>{}, b + 4);
  }
  for (; b < b_last; b += 2) two_stages(yes, (uint32_t)b % R, b);
  if constexpr (!BENCH) two_stages(no, (uint32_t)b_last % R, b_last);
  for (b = n_live + 1; b <= n_total; ++b) {  // stages without work: the barrier and the loads
    open_stage();
    request(b + 1 + F, b + F, (uint32_t)(b + 1 + F) % R, (uint32_t)(b + F) % R);
  }
  if constexpr (BENCH) {
    if (lane == 0) bench_clk[blockIdx.x * 4 + wave] = clock64() - bench_t0;
  }

  lsum = pair_sum(lsum);
  DEERS_TRACE_POINT(30);
  if (qrow < T) {
    const float inv = 1.f / lsum;
    half_t* orow = O + (int64_t)qrow * p.so.t;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_block_f16(orow + 32 * db, oacc[db], inv, g);
    if (g == 0) p.lse[(int64_t)bh * T + qrow] = (m + fast_log2(lsum)) * kLn2;
  }
}

template <int D>
__global__ __launch_bounds__(256, (D == 128 ? 2 : BP_OCC)) void attn_fwd_f16_bp_kernel(FwdParams p, int BH, int n_qtiles,
                                                                                int heads_per_xcd,
                                                                                TileOrder order) {
  attn_fwd_f16_bp_body<D, false>(p, BH, n_qtiles, heads_per_xcd, order, 0, nullptr);
}

}  // namespace deers
