// Fused causal attention forward, f16 storage / f32 accumulate, gfx950.
//
// Replaces the op chain of src/models/gpt.rs:139-144 (matmul, scalar_mul,
// causal_mask + add, log_sum_exp, sub, exp, matmul) with one kernel that never
// materialises the [T,T] score tensor.
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
#include <type_traits>

#include "common.h"

namespace deers {

constexpr int kFwdBM = 128;  // query rows per workgroup
constexpr int kFwdBN = 64;   // key/value rows per iteration
// The running row maximum is only advanced when some row's new maximum exceeds
// the one in use by more than this many powers of two; until then probabilities
// are formed against the stale maximum (values up to 2^8, exact in f16/f32).
constexpr float kLazyRescale = 8.0f;

#define ZERO16 floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#define ZEROH8 half8{0, 0, 0, 0, 0, 0, 0, 0}
// Hook for a timestamp-tracing build of this kernel; expands to nothing in the library.
#ifndef DEERS_TRACE_POINT
#define DEERS_TRACE_POINT(slot)
#endif

template <int D>
struct FwdCfg {
  static constexpr int P = 2;                   // prefetch distance in iterations
  static constexpr int NS = P + 1;              // ring slots per tensor
  static constexpr int RB = D * 2;              // row bytes
  static constexpr int TILE_B = kFwdBN * RB;    // tile bytes
  static constexpr size_t kLds = 2 * NS * TILE_B;
};

template <int D>
__global__ __launch_bounds__(256, (D == 128 ? 1 : 2)) void attn_fwd_f16_kernel(FwdParams p, int BH, int n_qtiles,
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

  // Workgroups are dealt round-robin to the 8 XCDs.  Keep every tile of one head
  // on one XCD (its K/V stay in that XCD's L2) and give each XCD the same mix of
  // long and short rows, longest first.
  // Within an XCD the dispatcher deals workgroups to its 32 CUs in order, so a CU
  // receives items i, i+32, i+64, ... of the XCD's list: the list is sorted longest
  // first and every second group of 32 is reversed, which evens out the per-CU sums.
  const int xcd = blockIdx.x & 7;
  int idx = blockIdx.x >> 3;
  const int per_xcd = n_qtiles * heads_per_xcd;
  {
    const int grp = idx >> 5, pos = idx & 31;
    const int grp_len = min(32, per_xcd - 32 * grp);
    if (grp & 1) idx = 32 * grp + (grp_len - 1 - pos);
  }
  const int bh = (idx % heads_per_xcd) * 8 + xcd;
  if (bh >= BH) return;
  const int qtile = n_qtiles - 1 - idx / heads_per_xcd;
  const int b = bh / p.H, h = bh % p.H;

  const half_t* Q = (const half_t*)p.q + b * p.sq.b + h * p.sq.h;
  const half_t* K = (const half_t*)p.k + b * p.sk.b + h * p.sk.h;
  const half_t* V = (const half_t*)p.v + b * p.sv.b + h * p.sv.h;
  half_t* O = (half_t*)p.o + b * p.so.b + h * p.so.h;

  DEERS_TRACE_POINT(0);
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
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (qrow < T)
      qf[ks] = *(const half8*)(Q + (int64_t)qrow * p.sq.t + 16 * ks + 8 * g);
    else
      qf[ks] = ZEROH8;
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
  const float c = p.scale_log2;

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
    half8 kfr[HAS_S ? 2 * KS : 1], vfr[HAS_PV ? 4 * DB : 1];
    if constexpr (HAS_PV) load_v(j - 1, vfr);
    if constexpr (HAS_S) load_k(j + 1, kfr);
    __builtin_amdgcn_sched_barrier(0);  // keep the fetches ahead of the vector work below

    if (kv0 + kFwdBN - 1 > qw0) {  // tile reaches past this wave's first row: element mask
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int kv = kv0 + 8 * (r >> 2) + 4 * g + (r & 3);
        if (kv > qrow) c0[r] = -INFINITY;
        if (kv + 32 > qrow) c1[r] = -INFINITY;
      }
    }
    float mx = fmaxf(c0[0], c1[0]);
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, c0[r]), c1[r]);
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
    // ---- one straight-line block: 16 MFMAs beside the exponentials ----
    if constexpr (HAS_PV) mfma_pv(vfr);
    if constexpr (HAS_S) mfma_s(kfr, n0, n1);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      c0[r] = fast_exp2(__builtin_fmaf(c0[r], c, -mc));
      c1[r] = fast_exp2(__builtin_fmaf(c1[r], c, -mc));
    }
    half8 pn[4];
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      pn[st] = pack_half8(c0[8 * st + 0], c0[8 * st + 1], c0[8 * st + 2], c0[8 * st + 3],
                          c0[8 * st + 4], c0[8 * st + 5], c0[8 * st + 6], c0[8 * st + 7]);
      pn[2 + st] = pack_half8(c1[8 * st + 0], c1[8 * st + 1], c1[8 * st + 2], c1[8 * st + 3],
                              c1[8 * st + 4], c1[8 * st + 5], c1[8 * st + 6], c1[8 * st + 7]);
    }
    // row sums from the f16-rounded probabilities, i.e. exactly what PV multiplies
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 8; e += 2)
        lsum = add_half2(half2v{pn[i][e], pn[i][e + 1]}, lsum);
    // Ask the scheduler for the interleaving: per MFMA, two exponentials and a few
    // plain vector ops.
    if constexpr (HAS_PV || HAS_S) {
      constexpr int NM = (HAS_PV ? 8 : 0) + (HAS_S ? 8 : 0);
#pragma unroll
      for (int i = 0; i < NM; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x400, (NM == 16) ? 2 : 4, 0);  // exp
        __builtin_amdgcn_sched_group_barrier(0x002, (NM == 16) ? 5 : 10, 0);  // VALU
      }
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
    DEERS_TRACE_POINT(2 + j);
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
  DEERS_TRACE_POINT(1);

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
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        half4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = (half_t)(oacc[db][4 * rq + e] * inv);
        *(half4*)(orow + 32 * db + 8 * rq + 4 * g) = out;
      }
    if (g == 0) p.lse[(int64_t)bh * T + qrow] = (m * c + fast_log2(lsum)) * kLn2;
  }
  DEERS_TRACE_POINT(30);
}

template <int D>
static void launch_fwd_f16_d(const FwdParams& p, int B, hipStream_t stream) {
  const int BH = B * p.H;
  const int n_qtiles = (p.T + kFwdBM - 1) / kFwdBM;
  const int heads_per_xcd = (BH + 7) / 8;
  const size_t lds = FwdCfg<D>::kLds;
  static bool attr_set = false;  // launches are serialised by the caller
  if (!attr_set && lds > 64 * 1024) {
    (void)hipFuncSetAttribute((const void*)attn_fwd_f16_kernel<D>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    attr_set = true;
  }
  LaunchScope scope("attn_fwd_f16", stream);
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
