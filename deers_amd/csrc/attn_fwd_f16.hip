// Fused causal attention forward, f16 storage / f32 accumulate, gfx950.
//
// Replaces the op chain of src/models/gpt.rs:139-144 (matmul, scalar_mul,
// causal_mask + add, log_sum_exp, sub, exp, matmul) with one kernel that never
// materialises the [T,T] score tensor.
//
// Two kernels share this decomposition: the tile-pipelined one described below (two
// workgroups per CU; small launches) and, for launches with more than two tiles per CU, the
// block-pipelined one of attn_fwd_f16_bp.h (three workgroups per CU at head widths 32 and
// 64, two at 128), whose workgroups are all resident from the start when they fit.
//
// Work decomposition
//   grid  = one workgroup per (head, 128-row query tile), dealt to the XCDs so a
//           head stays on one XCD; 256 threads = 4 waves; wave w owns query rows
//           [q0 + 32w, q0 + 32w + 32) of the tile.
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
//
// Software pipeline (per wave, iteration j): the matrix pipe runs S(j+1) and
// PV(j-1) while the vector pipe runs the softmax of S(j); the three are
// independent, so MFMA latency hides behind exp/convert work inside one wave.
// K/V tiles travel global -> LDS without touching registers
// (global_load_lds_dwordx4) into rings of P+1 slots, requested P iterations ahead
// of their use so HBM/L2 latency is off the critical path; tiles are unpadded and
// XOR-swizzled by 16-byte chunk.  One barrier per iteration.
#include <algorithm>
#include <map>
#include <tuple>
#include <type_traits>
#include <vector>

#include "attn_fwd_f16_bp.h"
#include "common.h"

namespace deers {

// The running row maximum is only advanced when some row's new maximum exceeds
// the one in use by more than this many powers of two; until then probabilities
// are formed against the stale maximum (values up to 2^8, exact in f16/f32).
constexpr float kLazyRescale = 8.0f;

#define ZEROH8 half8{0, 0, 0, 0, 0, 0, 0, 0}


template <int D>
__global__ __launch_bounds__(256, 2) void attn_fwd_f16_kernel(FwdParams p, int BH, int n_qtiles,
                                                              int heads_per_xcd) {
  using Cfg = FwdCfg<D>;
  constexpr int P = Cfg::P, NS = Cfg::NS, RB = Cfg::RB, TILE_B = Cfg::TILE_B;
  constexpr int KS = D / 16;            // contraction steps over D
  constexpr int DB = D / 32;            // 32-wide blocks of D in the output
  constexpr int CH = D / 8;             // 16-byte chunks per row
  constexpr int RPW = 1024 / RB;        // tile rows covered by one wave-wide 1 KiB load
  constexpr int NWLW = TILE_B / 4096;   // 1 KiB loads per wave per tile
  constexpr int LPI = 2 * NWLW;         // loads per wave per iteration (K and V)

  extern __shared__ __attribute__((aligned(1024))) char smem[];  // K ring, then V ring

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  const int T = p.T;

  int bh, rank;
  if (!map_block(blockIdx.x, n_qtiles, heads_per_xcd, BH, &bh, &rank)) return;
  const int qtile = n_qtiles - 1 - rank;  // longest rows first
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  half_t* O = (half_t*)p.o + b * p.so.b + h * p.so.h;

  [[maybe_unused]] const int trace_row = blockIdx.x;
  const int q0 = qtile * kFwdBM;
  const int qw0 = q0 + 32 * wave;        // first query row of this wave
  const int qrow = qw0 + (lane & 31);    // this lane's query row

  int last_q = q0 + kFwdBM - 1;
  if (last_q > T - 1) last_q = T - 1;
  const int n_tiles = last_q / kFwdBN + 1;

  // ---- asynchronous tile loads: lane -> (row, chunk) of this wave's 1 KiB slabs ----
  // The global address is a wave-uniform tile base plus a constant per-lane byte
  // offset; only the tile that contains row T-1 needs its rows clamped.
  const uint32_t lds0 = lds_address(smem);
  const int tail_tile = (T - 1) / kFwdBN;
  const int skt = (int)p.sk.t, svt = (int)p.sv.t;  // T * row stride < 2^31 (checked on the host)
  uint32_t ld_k[NWLW], ld_v[NWLW], ld_k_tail[NWLW], ld_v_tail[NWLW];
#pragma unroll
  for (int i = 0; i < NWLW; ++i) {
    const int row = (wave * NWLW + i) * RPW + lane / CH;
    const int col = 16 * ((lane % CH) ^ lds_swizzle<CH>(row));
    const int row_tail = min(row, T - 1 - tail_tile * kFwdBN);
    ld_k[i] = (uint32_t)(row * skt * 2 + col);
    ld_v[i] = (uint32_t)(row * svt * 2 + col);
    ld_k_tail[i] = (uint32_t)(row_tail * skt * 2 + col);
    ld_v_tail[i] = (uint32_t)(row_tail * svt * 2 + col);
  }
  // Requests K(kt) and V(vt) into their ring slots.  Tile indices outside
  // [0, n_tiles) are clamped: such tiles are never consumed (or only multiplied by
  // masked, zero probabilities).
  auto request = [&](int kt, int vt) {
    const int kc = min(max(kt, 0), n_tiles - 1), vc = min(max(vt, 0), n_tiles - 1);
    const uint32_t kdst = lds0 + ((kt + NS) % NS) * TILE_B + wave * (NWLW * 1024);
    const uint32_t vdst = lds0 + (NS + (vt + NS) % NS) * TILE_B + wave * (NWLW * 1024);
    const half_t* kbase = K + (uint32_t)(kc * kFwdBN * skt);
    const half_t* vbase = V + (uint32_t)(vc * kFwdBN * svt);
#pragma unroll
    for (int i = 0; i < NWLW; ++i) {
      async_load16_to_lds(kbase, kc == tail_tile ? ld_k_tail[i] : ld_k[i], kdst + i * 1024);
      async_load16_to_lds(vbase, vc == tail_tile ? ld_v_tail[i] : ld_v[i], vdst + i * 1024);
    }
  };

  // ---- prologue requests: K(0) alone (paired with a throw-away V), then P groups ----
  request(0, -P - 1);
#pragma unroll
  for (int i = -P; i < 0; ++i) request(i + 1 + P, i - 1 + P);

  // Q fragments: B operand of S^T = K Q^T, lane holds Q[qrow][16ks + 8g .. +7].
  half8 qf[KS];
  // Rows past T-1 read row T-1 instead (they are not stored, and a query owns its
  // accumulator column), so the loads issue as one batch without a branch.
  {
    const half_t* qp = Q + (int64_t)min(qrow, T - 1) * p.sq.t + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const half8*)(qp + 16 * ks);
  }

  // ---- per-lane swizzled read offsets (bytes within a tile) ----
  int koff[KS];  // A operand of S^T: row lane%32 (+32 for the second block), chunk 2ks+g
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    koff[ks] = (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  // transposed V fragments: this lane supplies row 4g + (lane%16)/4 (+8 for the upper
  // half) and 8 bytes at halfs column 32db + 16*((lane/16)%2) + 4*(lane%4)
  int voff_lo[DB], voff_hi[DB];
  {
    const int lrow = 4 * g + ((lane & 15) >> 2);
    const int c4 = lane & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      voff_lo[db] = lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      voff_hi[db] = (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }

  floatx16 oacc[DB];
#pragma unroll
  for (int i = 0; i < DB; ++i) oacc[i] = ZERO16;
  // m: running maximum of the RAW scores (scale > 0 is applied inside the exponent);
  // lsum: this lane's half of the row sum (the other half lives in lane+32).
  float m = -INFINITY, lsum = 0.f;
  // kept in a vector register: v_fma_f32 with a scalar-register operand issues at 4.4 clocks
  // per SIMD against 2.6 with three vector registers, and every score passes through one
  float c = p.scale_log2;
  asm volatile("" : "+v"(c));

  // Operand fetch and MFMA issue are separate steps: all LDS reads of an iteration
  // are issued right after its barrier, so their latency is covered by the row-maximum
  // pass, and the MFMAs later find their fragments in registers.  Reads use explicit
  // 32-bit LDS addresses (slot base + per-lane offset, one add each per iteration) so
  // the row-block offsets become instruction immediates.
  auto load_k = [&](int kt, half8* kfr) {  // kfr[2ks + blk]
    const uint32_t kb = lds0 + (kt % NS) * TILE_B;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint32_t addr = opaque(kb + koff[ks]);
      kfr[2 * ks] = *(DEERS_LDS const half8*)(uintptr_t)addr;
      kfr[2 * ks + 1] = *(DEERS_LDS const half8*)(uintptr_t)(addr + 32 * RB);
    }
  };
  // S^T(tile) into (a0, a1): two 32-row blocks, independent accumulators interleaved.
  auto mfma_s = [&](const half8* kfr, floatx16& a0, floatx16& a1) {
    a0 = ZERO16;
    a1 = ZERO16;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      a0 = mfma_f16(kfr[2 * ks], qf[ks], a0);
      a1 = mfma_f16(kfr[2 * ks + 1], qf[ks], a1);
    }
  };
  auto load_v = [&](int vt, half8* vfr) {  // vfr[(2mb + st) * DB + db]
    const uint32_t vb = lds0 + (NS + vt % NS) * TILE_B;
    uint32_t alo[DB], ahi[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      alo[db] = opaque(vb + voff_lo[db]);
      ahi[db] = opaque(vb + voff_hi[db]);
    }
#pragma unroll
    for (int ms = 0; ms < 4; ++ms)
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const uint32_t ro = 16 * ms * RB;
        const half4 lo = lds_read_tr16_at(alo[db] + ro);
        const half4 hi = lds_read_tr16_at(ahi[db] + ro);
        vfr[ms * DB + db] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
  };
  half8 pf[4];  // P of the previous tile, packed as B operands: index 2*mb + st
  auto mfma_pv = [&](const half8* vfr) {
#pragma unroll
    for (int ms = 0; ms < 4; ++ms)
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] = mfma_f16(vfr[ms * DB + db], pf[ms], oacc[db]);
  };

  // One pipelined iteration: softmax of (c0,c1) = S(j); if HAS_S, S(j+1) into
  // (n0,n1); if HAS_PV, O += V(j-1) P(j-1).  Leaves P(j) in pf.
  // Block A: row maxima (vector pipe) beside the first half of PV(j-1) (matrix
  // pipe).  Block B: exponentials, row sums and f16 packing beside the second
  // half of PV(j-1) and all of S(j+1).  The rare maximum update sits between.
  auto iterate = [&](auto has_s, auto has_pv, int j, floatx16& c0, floatx16& c1, floatx16& n0,
                     floatx16& n1) {
    constexpr bool HAS_S = decltype(has_s)::value;
    constexpr bool HAS_PV = decltype(has_pv)::value;
    const int kv0 = j * kFwdBN;
    // K(j+1) and V(j-1) were requested P iterations ago: all but the last P-1
    // request groups of this wave have landed; the barrier extends that to the
    // other waves' slabs and retires every read of the slots reused below.
    wait_vmcnt<(P - 1) * LPI>();
    __syncthreads();
    request(j + 1 + P, j - 1 + P);
    // D = 32: every fragment of the iteration is fetched here, ahead of the vector work.
    // D >= 64: a window of kJit fragments runs ahead of the MFMAs that consume them (see
    // the chunk loop).  At D = 128 the whole set would be 128 registers of operands; at
    // D = 64 the window spreads the LDS reads over the iteration instead of issuing all
    // 24 behind the barrier, where four waves' bursts queue up (31.5 -> 30.7 us at
    // 8x12x1024x64, 252 -> 208 registers).
    constexpr bool JIT = D >= 64;
    constexpr int kJit = 4;
    constexpr int NMS_ = HAS_S ? 2 * KS : 0;
    constexpr int NM_ = NMS_ + (HAS_PV ? 4 * DB : 0);
    half8 kfr[(HAS_S && !JIT) ? 2 * KS : 1], vfr[(HAS_PV && !JIT) ? 4 * DB : 1];
    half8 fr[JIT ? kJit : 1];
    // fragment of MFMA number mi of this iteration (S(j+1) first, then PV(j-1)); the
    // address is formed at the fetch (an add or two) rather than kept for the iteration
    const uint32_t kb_jit = lds0 + ((j + 1) % NS) * TILE_B;
    const uint32_t vb_jit = lds0 + (NS + (j + NS - 1) % NS) * TILE_B;
    auto fetch = [&](int mi) -> half8 {
      if (mi < NMS_) {
        const int ks = mi >> 1;
        const uint32_t addr = opaque(kb_jit + koff[ks]);
        return *(DEERS_LDS const half8*)(uintptr_t)(addr + (mi & 1) * 32 * RB);
      }
      const int ms = (mi - NMS_) / DB, db = (mi - NMS_) % DB;
      const uint32_t ro = 16 * ms * RB;
      const half4 lo = lds_read_tr16_at(opaque(vb_jit + voff_lo[db]) + ro);
      const half4 hi = lds_read_tr16_at(opaque(vb_jit + voff_hi[db]) + ro);
      return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    if constexpr (JIT) {
#pragma unroll
      for (int mi = 0; mi < kJit && mi < NM_; ++mi) fr[mi] = fetch(mi);
    } else {
      if constexpr (HAS_PV) load_v(j - 1, vfr);
      if constexpr (HAS_S) load_k(j + 1, kfr);
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the fetches ahead of the vector work below

    if (kv0 + kFwdBN - 1 > qw0) {  // tile reaches past this wave's first row: element mask
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kv = kv0 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (kv > qrow) c0[r] = -INFINITY;
        if (kv + 32 > qrow) c1[r] = -INFINITY;
      }
    }
    // four independent max3 chains: a dependent vector op issues only every other
    // slot, and with two waves per SIMD nothing else fills the gaps
    float mx4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) mx4[i] = fmaxf(c0[i], c1[i]);
#pragma unroll
    for (int r = 4; r < 16; ++r) mx4[r & 3] = fmaxf(fmaxf(mx4[r & 3], c0[r]), c1[r]);
    float mx = fmaxf(fmaxf(mx4[0], mx4[1]), fmaxf(mx4[2], mx4[3]));
    mx = pair_max(mx);
    if (__any((mx - m) * c > kLazyRescale)) {
      // Rare after the first tiles: move O, l and the not yet multiplied P(j-1)
      // to the new maximum (alpha <= 1, so the f16 P values cannot overflow).
      const float m_new = fmaxf(m, mx);
      const float alpha = fast_exp2((m - m_new) * c);
      m = m_new;
      lsum *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] *= alpha;
      if constexpr (HAS_PV) {
        const half_t ah = (half_t)alpha;
#pragma unroll
        for (int i = 0; i < 4; ++i) pf[i] *= ah;
      }
    }
    const float mc = m * c;
    // ---- one straight-line block of 16 fenced chunks ----
    // Chunk i issues its share of the MFMAs (S(j+1) first: the next iteration's row
    // maxima wait on it; then PV(j-1)), the exponentials of two scores, and the f16
    // packing of the previous chunk's pair, so that no instruction waits on the one
    // just before it.  The fences keep the compiler from regrouping the chunks: left
    // alone it issues the MFMAs back to back and the vector work after them.
    // Row sums use v_dot2_f32_f16 against (1,1): one vector issue slot per pair.  It
    // executes on the matrix pipe, which has slack here (the vector issue port is the
    // busier one), so it is cheaper than two f32 adds.
    constexpr int NMS = HAS_S ? 2 * KS : 0;
    constexpr int NM = NMS + (HAS_PV ? 4 * DB : 0);
    if constexpr (HAS_S) {
      n0 = ZERO16;
      n1 = ZERO16;
    }
    uint32_t pw[16];  // P(j) as packed f16 pairs; words 4k..4k+3 form B operand k
    auto row_sum = [&](int i) {  // from the f16-rounded pair, i.e. exactly what PV multiplies
      lsum = add_half2(__builtin_bit_cast(half2v, pw[i]), lsum);
      asm volatile("" : "+v"(lsum));
    };
    auto pack_pair = [&](int i) {  // scores 2(i%8), 2(i%8)+1 of block i/8
      const floatx16& cc = (i < 8) ? c0 : c1;
      const int r = 2 * (i & 7);
      pw[i] = __builtin_bit_cast(uint32_t, half2v{(half_t)cc[r], (half_t)cc[r + 1]});
      asm volatile("" : "+v"(pw[i]));  // keep the conversion in its chunk
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#pragma unroll
      for (int mi = i * NM / 16; mi < (i + 1) * NM / 16; ++mi) {
        if (mi < NMS) {
          const int ks = mi >> 1;
          const half8 a = JIT ? fr[mi % kJit] : kfr[JIT ? 0 : mi];
          if (mi & 1)
            n1 = mfma_f16(a, qf[ks], n1);
          else
            n0 = mfma_f16(a, qf[ks], n0);
        } else {
          const int ms = (mi - NMS) / DB, db = (mi - NMS) % DB;
          const half8 a = JIT ? fr[mi % kJit] : vfr[JIT ? 0 : ms * DB + db];
          oacc[db] = mfma_f16(a, pf[ms], oacc[db]);
        }
        if constexpr (JIT) {
          if (mi + kJit < NM) fr[mi % kJit] = fetch(mi + kJit);
        }
      }
      floatx16& cc = (i < 8) ? c0 : c1;
      const int r = 2 * (i & 7);
      cc[r] = fast_exp2(__builtin_fmaf(cc[r], c, -mc));
      cc[r + 1] = fast_exp2(__builtin_fmaf(cc[r + 1], c, -mc));
      if (i > 0) pack_pair(i - 1);
      if (i > 1) row_sum(i - 2);
      __builtin_amdgcn_sched_barrier(0);
    }
    pack_pair(15);
    row_sum(14);
    row_sum(15);
    half8 pn[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      pn[k] = __builtin_bit_cast(half8, u32x4{pw[4 * k], pw[4 * k + 1], pw[4 * k + 2], pw[4 * k + 3]});
    }
    // Pin P(j) and the row sum here: without a use in this block the compiler sinks
    // the exponentials past the barrier into the next iteration, away from the MFMAs
    // they are meant to overlap.
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      asm volatile("" : "+v"(pn[i]));
      pf[i] = pn[i];
    }
    asm volatile("" : "+v"(lsum));
  };

  // ---- S(0): K(0) is the oldest request ----
  wait_vmcnt<P * LPI>();
  __syncthreads();
  floatx16 sa0, sa1, sb0, sb1;
  {
    half8 kfr[2 * KS];
    load_k(0, kfr);
    mfma_s(kfr, sa0, sa1);
  }

  constexpr std::true_type yes{};
  constexpr std::false_type no{};
  if (n_tiles == 1) {
    iterate(no, no, 0, sa0, sa1, sb0, sb1);
  } else {
    iterate(yes, no, 0, sa0, sa1, sb0, sb1);
    int j = 1;
    for (; j + 2 < n_tiles; j += 2) {
      iterate(yes, yes, j, sb0, sb1, sa0, sa1);
      iterate(yes, yes, j + 1, sa0, sa1, sb0, sb1);
    }
    if (j + 1 < n_tiles) {
      iterate(yes, yes, j, sb0, sb1, sa0, sa1);
      iterate(no, yes, j + 1, sa0, sa1, sb0, sb1);
    } else {
      iterate(no, yes, j, sb0, sb1, sa0, sa1);
    }
  }
  // ---- drain: O += V(n-1) P(n-1) ----
  wait_vmcnt<(P - 1) * LPI>();  // V(n-1) precedes the last P-1 (never consumed) groups
  __syncthreads();
  {
    half8 vfr[4 * DB];
    load_v(n_tiles - 1, vfr);
    mfma_pv(vfr);
  }

  // ---- epilogue: O = acc / l, LSE = ln(l) + m*scale ----
  lsum = pair_sum(lsum);
  if (qrow < T) {
    const float inv = 1.f / lsum;
    half_t* orow = O + (int64_t)qrow * p.so.t;
#pragma unroll
    for (int db = 0; db < DB; ++db) store_block_f16(orow + 32 * db, oacc[db], inv, g);
    if (g == 0) p.lse[(int64_t)bh * T + qrow] = (m * c + fast_log2(lsum)) * kLn2;
  }
}


// Builds the TileOrder of a launch whose workgroups are all resident at once (their
// number does not exceed what the chip holds).  Workgroup position p of an XCD (id / 8)
// lands on CU p % cus_per_xcd when the dispatcher fills an empty chip, so positions p,
// p + cus, p + 2 cus share a CU and its issue ports: tiles are dealt longest first to the
// CU with the smallest total that still has a free slot.  Returns nullptr when the tiles
// do not all fit (then the dispatcher's own longest-first hand-out is the better order).
// *use_resident_kernel tells whether the launch is large enough for the plain kernel at
// all.  Built at the first launch of a geometry and kept on the host for the life of the
// process; no device memory.
template <int D>
static const TileOrder* resident_order(int heads_per_xcd, int T, bool* use_resident_kernel) {
  struct Key {
    int dev, heads, T;
    bool operator<(const Key& o) const { return std::tie(dev, heads, T) < std::tie(o.dev, o.heads, o.T); }
  };
  struct Entry {
    bool usable = false;    // the table is filled in
    bool resident = false;  // the launch is large enough for the plain kernel
    TileOrder order{};
  };
  static std::map<Key, Entry> cache;  // launches are serialised by the caller
  int dev = 0;
  (void)hipGetDevice(&dev);
  const Key key{dev, heads_per_xcd, T};
  auto it = cache.find(key);
  if (it != cache.end()) {
    *use_resident_kernel = it->second.resident;
    return it->second.usable ? &it->second.order : nullptr;
  }
  Entry& entry = cache[key];
  *use_resident_kernel = false;
  int cus = 0, per_cu = 0;
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  (void)hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_fwd_f16_bp_kernel<D>, 256,
                                                     BpCfg<D>::kLds);
  const int n_cu = std::max(cus / 8, 1);
  const int n_qtiles = (T + kFwdBM - 1) / kFwdBM;
  const int n_items = heads_per_xcd * n_qtiles;
  // launches that fit the pipelined kernel's two workgroups per CU are faster there
  // (head width 128: both kernels hold two workgroups per CU and the block-pipelined one is the
  // faster from the same size on: 1x16x8192x128 267 against 296 us)
  entry.resident = (D == 128 ? per_cu >= 2 : per_cu > 2) && n_items > 2 * n_cu;
  *use_resident_kernel = entry.resident;
  if (!entry.resident || n_items > n_cu * per_cu || n_items > kMaxResidentTiles) return nullptr;
  std::vector<long> load(n_cu, 0);
  std::vector<int> used(n_cu, 0);
  std::vector<char> filled((size_t)n_items, 0);
  for (int qt = n_qtiles - 1; qt >= 0; --qt) {  // descending cost
    const int cost = std::min(T - 1, qt * kFwdBM + kFwdBM - 1) / kFwdBN + 1;
    for (int h = 0; h < heads_per_xcd; ++h) {
      int best = -1;
      for (int c = 0; c < n_cu; ++c)
        if (used[c] < per_cu && used[c] * n_cu + c < n_items && (best < 0 || load[c] < load[best])) best = c;
      if (best < 0) return nullptr;
      const int pos = used[best] * n_cu + best;
      entry.order.code[pos] = (h << 16) | qt;
      filled[pos] = 1;
      load[best] += cost;
      ++used[best];
    }
  }
  for (int i = 0; i < n_items; ++i)
    if (!filled[i]) return nullptr;
  entry.usable = true;
  return &entry.order;
}

template <int D>
static void launch_fwd_f16_d(const FwdParams& p, int B, hipStream_t stream) {
  const int BH = B * p.H;
  const int n_qtiles = (p.T + kFwdBM - 1) / kFwdBM;
  const int heads_per_xcd = (BH + 7) / 8;
  const size_t lds = FwdCfg<D>::kLds;
  static bool attr_set = false;  // launches are serialised by the caller
  if (!attr_set) {
    if (lds > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_fwd_f16_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds);
    if (BpCfg<D>::kLds > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)attn_fwd_f16_bp_kernel<D>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)BpCfg<D>::kLds);
    attr_set = true;
  }
  LaunchScope scope("attn_fwd_f16", stream);
  {
    // More tiles than the tile-pipelined kernel holds at once (two workgroups per CU): the
    // block-pipelined kernel, at three workgroups per CU for head widths 32 and 64.  While they all fit, every workgroup
    // is resident from the start, placed for even CU totals, and nothing is left to a tail of
    // late, short workgroups; beyond that the dispatcher hands out each XCD's list longest
    // first.  Smaller launches are faster on the tile-pipelined kernel (2x12x2048x64: 33.6
    // against 34.6 us).
    bool use_resident = false;
    const TileOrder* table = resident_order<D>(heads_per_xcd, p.T, &use_resident);
    static const TileOrder kNoTable = [] {
      TileOrder t{};
      t.code[0] = -1;
      return t;
    }();
    if (const TileOrder* order = use_resident ? (table ? table : &kNoTable) : nullptr) {
      hipLaunchKernelGGL(attn_fwd_f16_bp_kernel<D>, dim3(8 * n_qtiles * heads_per_xcd), dim3(256), BpCfg<D>::kLds,
                         stream, p, BH, n_qtiles, heads_per_xcd, *order);
      return;
    }
  }
  hipLaunchKernelGGL(attn_fwd_f16_kernel<D>, dim3(8 * n_qtiles * heads_per_xcd), dim3(256), lds,
                     stream, p, BH, n_qtiles, heads_per_xcd);
}

void launch_attn_fwd_f16(const FwdParams& p, int B, int D, hipStream_t stream) {
  switch (D) {
    case 32: launch_fwd_f16_d<32>(p, B, stream); break;
    case 64: launch_fwd_f16_d<64>(p, B, stream); break;
    case 128: launch_fwd_f16_d<128>(p, B, stream); break;
  }
}

}  // namespace deers
