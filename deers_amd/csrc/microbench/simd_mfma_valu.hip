// Micro-benchmarks behind the attention kernels' roofline argument: what one gfx950 SIMD does
// with the instruction mix of the f16 attention loops, with no memory system in the way.
//
//   0  a bare MFMA stream on every SIMD: sustained matrix rate and shader clock
//   A  vector issue rate of 1..4 waves per SIMD (independent v_fma_f32 chains, a dependent
//      chain, v_exp_f32, v_max3_f32, v_fma_f32 with a scalar-register operand,
//      v_cvt_pk_f16_f32, v_dot2c_f32_f16, v_exp_f16)
//   B  one wave streaming v_mfma_f32_32x32x16_f16 beside one wave streaming vector ops on
//      the same SIMD: each alone, then together
//   C  one instruction stream with NV vector ops between consecutive MFMAs, 1 and 2 waves
//   D  the forward's wave-iteration (S = K Q^T on 64 keys, online softmax on the results,
//      O += V^T P) with its memory features switched on one at a time: LDS fragment reads,
//      the per-iteration barrier, asynchronous global->LDS tile loads; 1, 2, 3 waves per SIMD
//   E  phase alternation: every wave alternates a matrix phase (16 MFMAs) and a vector phase
//      (the softmax ops of 32 scores); free running, two wave groups held in opposite phases by
//      barriers ("ping-pong"), and both groups in the same phase
//   F  the block-pipelined forward's own loop, compiled in its bench mode
//   G  one stream of chunks, each one MFMA followed by a given handful of other instructions
//      (what fits in the 32 clocks of an MFMA, and what each further instruction costs)
//   H  one or two MFMAs per 1 KiB operand fragment read from LDS, with and without the
//      softmax's vector ops, and the rate of MFMAs chained through one accumulator
//   P  a bare MFMA stream again, on operands of zeros, a constant, and random values: the
//      device is power limited and the clock it sustains depends on the data
//   Q  v_mfma_f32_32x32x2_f32 (the f32 attention kernels' instruction) with every A operand
//      read from LDS, 1..8 reads in flight, through one or four accumulation chains, at one and
//      two waves per SIMD: whether a chain of dependent products or an LDS read per product
//      slows the pipe
//
// Every launch covers all CUs (256 workgroups x waves); times are clock64() deltas from the
// common start of a CU's waves to the end of its slowest wave, averaged over the CUs, so
// figures are shader clocks.  A first section times a bare MFMA stream on all CUs with events:
// the matrix rate and the shader clock the device actually sustains.  Build: make -C deers_amd/csrc
// microbench; run: deers_amd/csrc/microbench/simd_mfma_valu.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../attn_fwd_f16_bp.h"
#include "../common.h"

using namespace deers;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define CK(x)                                                              \
  do {                                                                     \
    hipError_t e_ = (x);                                                   \
    if (e_ != hipSuccess) {                                                \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); \
      exit(1);                                                             \
    }                                                                      \
  } while (0)
#define ZERO16 floatx16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}
#define MF(acc) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b))
#define FM(v) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v) : "v"(c1), "v"(c2))
#define EX(v) asm volatile("v_exp_f32 %0, %0" : "+v"(v))
#define MX(v, w) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(v) : "v"(w), "v"(c2))
#define FMS(v) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v) : "s"(sc), "v"(c2))
#define CVT(d, x, y) asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(d) : "v"(x), "v"(y))
#define DOT(acc, x) asm volatile("v_dot2c_f32_f16 %0, %1, %2" : "+v"(acc) : "v"(x), "v"(ones))
#define EXH(v) asm volatile("v_exp_f16 %0, %0" : "+v"(v))
#define REP8(X) X X X X X X X X

static long long* g_clk = nullptr;  // per-wave elapsed clocks of the last launch
static float* g_out = nullptr;
// Clocks from the common start of a workgroup's waves to the end of the slowest of waves
// [first_wave, first_wave + n_waves) of each workgroup, averaged over the workgroups.  (The
// SIMD serves its waves oldest first, so their end times differ; the last one bounds the
// SIMD's time.)
static double slowest_wave_clocks(int n_blocks, int first_wave, int n_waves) {
  static long long h[256 * 16];
  CK(hipMemcpy(h, g_clk, sizeof(h), hipMemcpyDeviceToHost));
  double s = 0;
  for (int blk = 0; blk < n_blocks; ++blk) {
    long long mx = 0;
    for (int w = first_wave; w < first_wave + n_waves; ++w) mx = h[blk * 16 + w] > mx ? h[blk * 16 + w] : mx;
    s += (double)mx;
  }
  return s / n_blocks;
}

// ---- 0: bare MFMA stream on all CUs, by events and by the 100 MHz wall clock ---------------
__global__ __launch_bounds__(1024) void mfma_stream_kernel(float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  half8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (half_t)(0.001f * (lane + i));
    b[i] = (half_t)(0.002f * (lane - i));
  }
  floatx16 acc0 = ZERO16, acc1 = ZERO16, acc2 = ZERO16, acc3 = ZERO16;
  __syncthreads();
  const long long w0 = wall_clock64(), t0 = clock64();
  for (int it = 0; it < iters; ++it) { REP8(MF(acc0); MF(acc1);) REP8(MF(acc2); MF(acc3);) }
  const long long t1 = clock64(), w1 = wall_clock64();
  float s = 0;
  for (int i = 0; i < 16; ++i) s += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (lane == 0) clk[blockIdx.x * 16 + wave] = wave == 0 ? ((t1 - t0) << 32 | (w1 - w0)) : 0;
}
static void run_mfma_stream() {
  const int iters = 10000;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  for (int rep = 0; rep < 3; ++rep)
    for (int waves = 4; waves <= 16; waves += 4) {
      mfma_stream_kernel<<<256, 64 * waves>>>(g_out, g_clk, 100);
      CK(hipEventRecord(e0));
      mfma_stream_kernel<<<256, 64 * waves>>>(g_out, g_clk, iters);
      CK(hipEventRecord(e1));
      CK(hipEventSynchronize(e1));
      float ms;
      CK(hipEventElapsedTime(&ms, e0, e1));
      static long long h[256 * 16];
      CK(hipMemcpy(h, g_clk, sizeof(h), hipMemcpyDeviceToHost));
      double ghz = 0;
      for (int blk = 0; blk < 256; ++blk) ghz += (double)(h[blk * 16] >> 32) / ((double)(h[blk * 16] & 0xffffffff) * 10.0);
      ghz /= 256;
      const double mfmas_per_simd = (double)iters * 32.0 * (waves / 4);
      const double ns = ms * 1e6 / mfmas_per_simd;
      if (rep == 2)
        printf("0 bare MFMA stream, %d wave(s)/SIMD: %5.2f ns per MFMA per SIMD = %4.0f TFLOP/s on 1024 SIMDs, shader clock %4.2f "
               "GHz (%4.1f clocks per MFMA)\n",
               waves / 4, ns, 32768.0 * 1024 / ns / 1e3, ghz, ns * ghz);
    }
}

// ---- A: vector issue rate --------------------------------------------------------------
template <int KIND>
__global__ __launch_bounds__(1024) void valu_rate_kernel(float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float v0 = lane, v1 = lane + 1, v2 = lane + 2, v3 = lane + 3, v4 = lane + 4, v5 = lane + 5, v6 = lane + 6,
        v7 = lane + 7;
  float c1 = 0.999f, c2 = 0.001f;
  const float sc = 0.18f;                   // stays in a scalar register
  unsigned h0 = 0xb800b400u + lane, h1 = 0xb900b500u + lane, h2 = 0xba00b600u + lane, h3 = 0xbb00b700u + lane;
  const unsigned ones = 0x3c003c00u;        // (1, 1) as packed halfs
  __syncthreads();
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {  // 32 ops per pass
    if (KIND == 0) { REP8(FM(v0); FM(v1); FM(v2); FM(v3);) }
    if (KIND == 1) { REP8(FM(v0); FM(v0); FM(v0); FM(v0);) }
    if (KIND == 2) { REP8(EX(v0); EX(v1); EX(v2); EX(v3);) }
    if (KIND == 3) { REP8(MX(v0, v4); MX(v1, v5); MX(v2, v6); MX(v3, v7);) }
    if (KIND == 4) { REP8(FMS(v0); FMS(v1); FMS(v2); FMS(v3);) }
    if (KIND == 5) { REP8(CVT(h0, v0, v1); CVT(h1, v1, v2); CVT(h2, v2, v3); CVT(h3, v3, v0);) }
    if (KIND == 6) { REP8(DOT(v0, h0); DOT(v1, h1); DOT(v2, h2); DOT(v3, h3);) }
    if (KIND == 7) { REP8(EXH(h0); EXH(h1); EXH(h2); EXH(h3);) }
  }
  const long long t1 = clock64();
  out[blockIdx.x * blockDim.x + threadIdx.x] = v0 + v1 + v2 + v3 + v4 + v5 + v6 + v7 + (float)(h0 + h1 + h2 + h3);
  if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
}
template <int KIND>
static void run_valu_rate(const char* name) {
  const int iters = 4000;
  for (int waves = 4; waves <= 16; waves += 4) {
    valu_rate_kernel<KIND><<<256, 64 * waves>>>(g_out, g_clk, 50);
    valu_rate_kernel<KIND><<<256, 64 * waves>>>(g_out, g_clk, iters);
    CK(hipDeviceSynchronize());
    const double per_op = slowest_wave_clocks(256, 0, waves) / (iters * 32.0);
    printf("A %-22s %d wave(s)/SIMD: %5.2f clocks per op per wave = one op per %4.2f clocks per SIMD\n", name,
           waves / 4, per_op, per_op / (waves / 4));
  }
}

// ---- B: an MFMA wave beside a vector wave ------------------------------------------------
__global__ __launch_bounds__(512) void side_by_side_kernel(float* out, long long* clk, int iters, int mfma_on,
                                                           int valu_kind) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  half8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (half_t)(0.001f * (lane + i));
    b[i] = (half_t)(0.002f * (lane - i));
  }
  floatx16 acc0 = ZERO16, acc1 = ZERO16;
  float v0 = lane, v1 = lane + 1, v2 = lane + 2, v3 = lane + 3;
  float c1 = 0.999f, c2 = 0.001f;
  __syncthreads();
  const long long t0 = clock64();
  if (wave < 4) {  // two dependent chains, as the S and dP accumulators of a block
    if (mfma_on)
      for (int it = 0; it < iters; ++it) { REP8(MF(acc0); MF(acc1);) }
  } else {
    if (valu_kind == 1)
      for (int it = 0; it < 4 * iters; ++it) { REP8(FM(v0); FM(v1); FM(v2); FM(v3);) }
    if (valu_kind == 2)
      for (int it = 0; it < 4 * iters; ++it) { REP8(EX(v0); EX(v1); EX(v2); EX(v3);) }
  }
  const long long t1 = clock64();
  float s = v0 + v1 + v2 + v3;
  for (int i = 0; i < 16; ++i) s += acc0[i] + acc1[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
}
static void run_side_by_side() {
  const int iters = 2000;
  const int cfg[][2] = {{1, 0}, {0, 1}, {0, 2}, {1, 1}, {1, 2}};
  for (const auto& c : cfg) {
    side_by_side_kernel<<<256, 512>>>(g_out, g_clk, 50, c[0], c[1]);
    side_by_side_kernel<<<256, 512>>>(g_out, g_clk, iters, c[0], c[1]);
    CK(hipDeviceSynchronize());
    const double m = slowest_wave_clocks(256, 0, 4) / (iters * 16.0);
    const double v = slowest_wave_clocks(256, 4, 4) / (iters * 128.0);
    printf("B MFMA wave %s, vector wave %-4s: %5.1f clocks per MFMA, %5.2f clocks per vector op\n",
           c[0] ? "on " : "off", c[1] == 0 ? "off" : c[1] == 1 ? "fma" : "exp", c[0] ? m : 0.0, c[1] ? v : 0.0);
  }
}

// ---- C: NV vector ops between consecutive MFMAs of one wave -------------------------------
template <int NV>
__global__ __launch_bounds__(512) void interleaved_kernel(float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  half8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (half_t)(0.001f * (lane + i));
    b[i] = (half_t)(0.002f * (lane - i));
  }
  floatx16 acc0 = ZERO16, acc1 = ZERO16, acc2 = ZERO16, acc3 = ZERO16;
  float v0 = lane, v1 = lane + 1, v2 = lane + 2, v3 = lane + 3, v4 = lane + 4, v5 = lane + 5, v6 = lane + 6,
        v7 = lane + 7;
  float c1 = 0.999f, c2 = 0.001f;
#define VGRP()                                                                                      \
  do {                                                                                              \
    if (NV >= 1) FM(v0); if (NV >= 2) FM(v1); if (NV >= 3) FM(v2); if (NV >= 4) FM(v3);             \
    if (NV >= 5) FM(v4); if (NV >= 6) FM(v5); if (NV >= 7) FM(v6); if (NV >= 8) FM(v7);             \
    if (NV >= 9) FM(v0); if (NV >= 10) FM(v1); if (NV >= 11) FM(v2); if (NV >= 12) FM(v3);          \
    if (NV >= 13) FM(v4); if (NV >= 14) FM(v5); if (NV >= 15) FM(v6); if (NV >= 16) FM(v7);         \
  } while (0)
  __syncthreads();
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      MF(acc0); VGRP(); MF(acc1); VGRP(); MF(acc2); VGRP(); MF(acc3); VGRP();
    }
  }
  const long long t1 = clock64();
  float s = v0 + v1 + v2 + v3 + v4 + v5 + v6 + v7;
  for (int i = 0; i < 16; ++i) s += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
}
template <int NV>
static void run_interleaved() {
  const int iters = 3000;
  for (int waves = 4; waves <= 8; waves += 4) {
    interleaved_kernel<NV><<<256, 64 * waves>>>(g_out, g_clk, 50);
    interleaved_kernel<NV><<<256, 64 * waves>>>(g_out, g_clk, iters);
    CK(hipDeviceSynchronize());
    const double per_mfma = slowest_wave_clocks(256, 0, waves) / (iters * 16.0) / (waves / 4);
    printf("C %2d vector ops per MFMA, %d wave(s)/SIMD: %5.1f clocks of SIMD time per MFMA (32 = matrix pipe full)\n",
           NV, waves / 4, per_mfma);
  }
}

// ---- D: the forward's wave-iteration --------------------------------------------------------
constexpr int D = 64, KS = 4, DB = 2, CH = 8, RB = 128, TILE_B = 64 * RB, P = 2, NS = 3, NWLW = 2, LPI = 4,
              RPW = 8;
template <bool F_LDS, bool F_BAR, bool F_REQ>
__global__ __launch_bounds__(256, 3) void fwd_iteration_kernel(const half_t* Kg, const half_t* Vg, float* out,
                                                               long long* clk, int iters, float c) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t lds0 = lds_address(smem);
  const half_t* K = Kg + (size_t)(blockIdx.x % 96) * 1024 * D;
  const half_t* V = Vg + (size_t)(blockIdx.x % 96) * 1024 * D;
  uint32_t ld_k[NWLW];
  for (int i = 0; i < NWLW; ++i) {
    const int row = (wave * NWLW + i) * RPW + lane / CH;
    ld_k[i] = (uint32_t)(row * D * 2 + 16 * ((lane % CH) ^ lds_swizzle<CH>(row)));
  }
  auto request = [&](int t) {  // K and V tile t % 16 of this head into ring slot t % NS
    const int tc = t & 15;
    const uint32_t kdst = lds0 + (t % NS) * TILE_B + wave * (NWLW * 1024);
    const uint32_t vdst = kdst + NS * TILE_B;
#pragma unroll
    for (int i = 0; i < NWLW; ++i) {
      async_load16_to_lds(K + (uint32_t)(tc * 64 * D), ld_k[i], kdst + i * 1024);
      async_load16_to_lds(V + (uint32_t)(tc * 64 * D), ld_k[i], vdst + i * 1024);
    }
  };
  for (int t = 0; t < NS; ++t) request(t);
  half8 qf[KS], kreg[8], vreg[8];
  for (int ks = 0; ks < KS; ++ks)
    for (int i = 0; i < 8; ++i) qf[ks][i] = (half_t)(0.02f * ((lane - i - ks) % 11));
  for (int j = 0; j < 8; ++j)
    for (int i = 0; i < 8; ++i) {
      kreg[j][i] = (half_t)(0.01f * ((lane + i + j) % 13) - 0.05f);
      vreg[j][i] = (half_t)(0.01f * ((lane ^ (i + j)) % 7));
    }
  int koff[KS], voff_lo[DB], voff_hi[DB];
  for (int ks = 0; ks < KS; ++ks) koff[ks] = (lane & 31) * RB + (((2 * ks + g) ^ lds_swizzle<CH>(lane & 31)) << 4);
  {
    const int lrow = 4 * g + ((lane & 15) >> 2), c4 = lane & 3;
    for (int db = 0; db < DB; ++db) {
      const int chunk = 4 * db + 2 * ((lane >> 4) & 1) + (c4 >> 1);
      voff_lo[db] = lrow * RB + ((chunk ^ lds_swizzle<CH>(lrow)) << 4) + (c4 & 1) * 8;
      voff_hi[db] = (lrow + 8) * RB + ((chunk ^ lds_swizzle<CH>(lrow + 8)) << 4) + (c4 & 1) * 8;
    }
  }
  floatx16 oacc[DB] = {ZERO16, ZERO16};
  float m = -1e30f, lsum = 0.f;
  wait_all_vmem();
  __syncthreads();
  const long long t0 = clock64();
  for (int j = 0; j < iters; ++j) {
    if (F_REQ) wait_vmcnt<(P - 1) * LPI>();
    if (F_BAR) __syncthreads();
    if (F_REQ) request(j + P);
    const uint32_t kb = lds0 + (j % NS) * TILE_B, vb = kb + NS * TILE_B;
    floatx16 cb[2] = {ZERO16, ZERO16};
    if (!F_LDS)
      for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(kreg[i]), "+v"(vreg[i]));
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const uint32_t addr = opaque(kb + koff[ks]);
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
        cb[nb] = mfma_f16(F_LDS ? *(DEERS_LDS const half8*)(uintptr_t)(addr + nb * 32 * RB) : kreg[2 * ks + nb],
                          qf[ks], cb[nb]);
    }
    half8 vfr[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      if (F_LDS) {
        const half4 lo = lds_read_tr16_at(opaque(vb + voff_lo[db]));
        const half4 hi = lds_read_tr16_at(opaque(vb + voff_hi[db]));
        vfr[db] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      } else {
        vfr[db] = vreg[db];
      }
    }
    float mx4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) mx4[i] = fmaxf(cb[0][i], cb[1][i]);
#pragma unroll
    for (int r = 4; r < 16; ++r) mx4[r & 3] = fmaxf(fmaxf(mx4[r & 3], cb[0][r]), cb[1][r]);
    const float mx = pair_max(fmaxf(fmaxf(mx4[0], mx4[1]), fmaxf(mx4[2], mx4[3])));
    if (__any((mx - m) * c > 8.f)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = fast_exp2((m - m_new) * c);
      m = m_new;
      lsum *= alpha;
      oacc[0] *= alpha;
      oacc[1] *= alpha;
    }
    const float mc = m * c;
    uint32_t pw[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const floatx16& cc = cb[i >> 3];
      const int r = 2 * (i & 7);
      const float e0 = fast_exp2(__builtin_fmaf(cc[r], c, -mc));
      const float e1 = fast_exp2(__builtin_fmaf(cc[r + 1], c, -mc));
      pw[i] = __builtin_bit_cast(uint32_t, half2v{(half_t)e0, (half_t)e1});
      lsum = add_half2(__builtin_bit_cast(half2v, pw[i]), lsum);
    }
#pragma unroll
    for (int ms = 0; ms < 4; ++ms) {
      const half8 pb = __builtin_bit_cast(half8, u32x4{pw[4 * ms], pw[4 * ms + 1], pw[4 * ms + 2], pw[4 * ms + 3]});
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        half8 av;
        if (ms == 0) {
          av = vfr[db];
        } else if (F_LDS) {
          const uint32_t ro = 16 * ms * RB;
          const half4 lo = lds_read_tr16_at(opaque(vb + voff_lo[db]) + ro);
          const half4 hi = lds_read_tr16_at(opaque(vb + voff_hi[db]) + ro);
          av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        } else {
          av = vreg[2 * ms + db];
        }
        oacc[db] = mfma_f16(av, pb, oacc[db]);
      }
    }
  }
  const long long t1 = clock64();
  wait_all_vmem();
  float sum = lsum + m;
  for (int i = 0; i < 16; ++i) sum += oacc[0][i] + oacc[1][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
  if (lane == 0) clk[(blockIdx.x % 256) * 16 + (blockIdx.x / 256) * 4 + wave] = t1 - t0;
}
template <bool F_LDS, bool F_BAR, bool F_REQ>
static void run_fwd_iteration(const half_t* Kg, const half_t* Vg) {
  const int iters = 3000;
  const size_t lds = 2 * NS * TILE_B;
  for (int wgs = 1; wgs <= 3; ++wgs) {
    fwd_iteration_kernel<F_LDS, F_BAR, F_REQ><<<256 * wgs, 256, lds>>>(Kg, Vg, g_out, g_clk, 50, 0.18f);
    fwd_iteration_kernel<F_LDS, F_BAR, F_REQ><<<256 * wgs, 256, lds>>>(Kg, Vg, g_out, g_clk, iters, 0.18f);
    CK(hipDeviceSynchronize());
    const double per_iter = slowest_wave_clocks(256, 0, 4 * wgs) / iters;
    printf("D lds reads %d, barrier %d, tile loads %d, %d wave(s)/SIMD: %5.0f clocks per wave-iteration = %4.0f of "
           "SIMD time (its 16 MFMAs alone: 512)\n",
           (int)F_LDS, (int)F_BAR, (int)F_REQ, wgs, per_iter, per_iter / wgs);
  }
}


// ---- F: the block-pipelined forward's own loop (attn_fwd_f16_bp.h compiled in its bench mode) ----
template <int OCC, int DH>
__global__ __launch_bounds__(256, OCC) void fwd_bp_bench_kernel(FwdParams p, int BH, int n_qtiles, int heads_per_xcd,
                                                                TileOrder order, int stages, long long* clk) {
  attn_fwd_f16_bp_body<DH, true>(p, BH, n_qtiles, heads_per_xcd, order, stages, clk);
}
template <int OCC, int DH = 64>
static void run_fwd_bp(int wgs) {
  const int stages = 4000, T = 1024, n_qtiles = 8, heads_per_xcd = 4 * wgs, BH = 8 * heads_per_xcd;
  const size_t elems = (size_t)BH * T * DH;
  half_t *q, *k, *v, *o;
  float* lse;
  long long* clk;
  CK(hipMalloc(&q, elems * 2)); CK(hipMalloc(&k, elems * 2)); CK(hipMalloc(&v, elems * 2)); CK(hipMalloc(&o, elems * 2));
  CK(hipMalloc(&lse, (size_t)BH * T * 4));
  CK(hipMalloc(&clk, 256 * 4 * 4 * sizeof(long long)));
  {  // random operands (sigma 0.25, scores stay small): the clock the loop sustains depends on the data
    static std::vector<_Float16> h;
    h.resize(elems);
    unsigned s = 99;
    for (size_t i = 0; i < elems; ++i) {
      float u = 0;
      for (int j = 0; j < 4; ++j) { s = s * 1664525u + 1013904223u; u += (s >> 8) / 16777216.0f; }
      h[i] = (_Float16)((u - 2.0f) * 1.73f * 0.25f);
    }
    CK(hipMemcpy(q, h.data(), elems * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(k, h.data(), elems * 2, hipMemcpyHostToDevice));
    CK(hipMemcpy(v, h.data(), elems * 2, hipMemcpyHostToDevice));
  }
  FwdParams p{};
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.sq = p.sk = p.sv = p.so = Strides3{(int64_t)T * DH, (int64_t)T * DH, DH};  // B = BH "batches" of one head
  p.H = 1; p.T = T; p.scale_log2 = 0.18f;
  TileOrder order{};
  order.code[0] = -1;
  const size_t lds = BpCfg<DH>::kLds;
  if (lds > 64 * 1024)
    CK(hipFuncSetAttribute((const void*)fwd_bp_bench_kernel<OCC, DH>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  fwd_bp_bench_kernel<OCC, DH><<<256 * wgs, 256, lds>>>(p, BH, n_qtiles, heads_per_xcd, order, 100, clk);
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  CK(hipEventRecord(e0));
  fwd_bp_bench_kernel<OCC, DH><<<256 * wgs, 256, lds>>>(p, BH, n_qtiles, heads_per_xcd, order, stages, clk);
  CK(hipEventRecord(e1));
  CK(hipDeviceSynchronize());
  float ms = 0;
  CK(hipEventElapsedTime(&ms, e0, e1));
  CK(hipEventDestroy(e0)); CK(hipEventDestroy(e1));
  static long long h[256 * 4 * 4];
  CK(hipMemcpy(h, clk, sizeof(long long) * 256 * wgs * 4, hipMemcpyDeviceToHost));
  double s = 0;
  for (int i = 0; i < 256 * wgs * 4; ++i) s += (double)h[i];
  const double per_stage = s / (256.0 * wgs * 4) / stages;
  printf("F block-pipelined forward, head width %d (launch bound %d), %d workgroup(s) = wave(s)/SIMD per CU: %5.0f clocks per wave-stage (32 keys) = %4.0f of SIMD time (its %d MFMAs alone: %d); %.2f GHz\n",
         DH, OCC, wgs, per_stage, per_stage / wgs, DH / 8, DH * 4, per_stage * stages / (ms * 1e6));
  CK(hipFree(q)); CK(hipFree(k)); CK(hipFree(v)); CK(hipFree(o)); CK(hipFree(lse)); CK(hipFree(clk));
}

// ---- E: phase alternation ---------------------------------------------------------------------
// MODE 0: free running; 1: a barrier between the phases, the two wave groups of a workgroup in
// opposite phases; 2: barriers, all waves in the same phase.  VSET 0: the tile-pipelined
// loops' vector mix per 32 scores (32 fma, 32 exp, 16 cvt_pk, 16 dot2c, 16 max3, 8 fma); 1:
// without the fma before each exponential and the maxima.
template <int MODE, int VSET>
__global__ __launch_bounds__(1024) void phase_kernel(float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  half8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (half_t)(0.001f * (lane + i)); b[i] = (half_t)(0.002f * (lane - i)); }
  floatx16 acc0 = ZERO16, acc1 = ZERO16, acc2 = ZERO16, acc3 = ZERO16;
  float v0 = lane, v1 = lane + 1, v2 = lane + 2, v3 = lane + 3, v4 = lane + 4, v5 = lane + 5, v6 = lane + 6, v7 = lane + 7;
  float c1 = 0.999f, c2 = 0.001f, s0 = 0, s1 = 0, mx0 = 0, mx1 = 0;
  unsigned h0, h1; const unsigned ones = 0x3c003c00u;
  const int group = (wave >> 2) & 1;
  __syncthreads();
  const long long t0 = clock64();
  auto phase_m = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) { MF(acc0); MF(acc1); MF(acc2); MF(acc3); }
  };
  auto phase_v = [&]() {
#pragma unroll
    for (int i = 0; i < 8; ++i) {  // 4 scores per round
      if (VSET == 0) { FM(v0); FM(v1); FM(v2); FM(v3); }
      EX(v0); EX(v1); EX(v2); EX(v3);
      CVT(h0, v0, v1); CVT(h1, v2, v3);
      DOT(s0, h0); DOT(s1, h1);
      if (VSET == 0) { MX(mx0, v4); MX(mx1, v6); }
      FM(v4);
    }
  };
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) { phase_m(); phase_v(); }
    if (MODE == 1) {
      if (group == 0) { phase_m(); __builtin_amdgcn_s_barrier(); phase_v(); __builtin_amdgcn_s_barrier(); }
      else { phase_v(); __builtin_amdgcn_s_barrier(); phase_m(); __builtin_amdgcn_s_barrier(); }
    }
    if (MODE == 2) { phase_m(); __builtin_amdgcn_s_barrier(); phase_v(); __builtin_amdgcn_s_barrier(); }
  }
  const long long t1 = clock64();
  float s = v0 + v1 + v2 + v3 + v4 + v5 + v6 + v7 + s0 + s1 + mx0 + mx1;
  for (int i = 0; i < 16; ++i) s += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
}
template <int MODE, int VSET>
static void run_phase(const char* mode_name) {
  const int iters = 3000;
  for (int waves = 4; waves <= 16; waves += 4) {
    if (MODE != 0 && (waves == 4 || waves == 12)) continue;  // two equal groups
    phase_kernel<MODE, VSET><<<256, 64 * waves>>>(g_out, g_clk, 50);
    phase_kernel<MODE, VSET><<<256, 64 * waves>>>(g_out, g_clk, iters);
    CK(hipDeviceSynchronize());
    const double per_wave_iter = slowest_wave_clocks(256, 0, waves) / iters;
    printf("E %-15s vector mix %d, %d wave(s)/SIMD: %5.0f clocks of SIMD time per wave-iteration (its 16 MFMAs alone: 512)\n",
           mode_name, VSET, waves / 4, per_wave_iter / (waves / 4));
  }
}

// ---- G: chunks of one MFMA and a handful of other instructions ------------------------------------
#define ADDF(v, w) asm volatile("v_add_f32 %0, %0, %1" : "+v"(v) : "v"(w))
#define MULF(v, w) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(v) : "v"(w))
template <int ID>
__global__ __launch_bounds__(1024) void chunk_kernel(float* out, long long* clk, int iters) {
  __shared__ __attribute__((aligned(16))) char lds[16384];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  half8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (half_t)(0.001f * (lane + i)); b[i] = (half_t)(0.002f * (lane - i)); }
  floatx16 acc0 = ZERO16, acc1 = ZERO16, acc2 = ZERO16, acc3 = ZERO16;
  float v0 = lane, v1 = lane + 1, v2 = lane + 2, v3 = lane + 3, v4 = lane + 4, v5 = lane + 5, v6 = lane + 6, v7 = lane + 7;
  float c1 = 0.999f, c2 = 0.001f, s0 = 0, s1 = 0;
  unsigned h0 = 0, h1 = 0; const unsigned ones = 0x3c003c00u;
  for (int i = threadIdx.x; i < 4096; i += blockDim.x) ((float*)lds)[i] = 0.f;
  const uint32_t la = lds_address(lds) + lane * 16;
  half8 fr0 = a, fr1 = a;
  __syncthreads();
  const long long t0 = clock64();
#define OPS(x, y, hh, ss, fr)                                                                   \
  do {                                                                                          \
    if (ID == 0) { EX(x); EX(y); CVT(hh, x, y); }                                               \
    if (ID == 1) { EX(x); EX(y); CVT(hh, x, y); ADDF(ss, x); }                                  \
    if (ID == 2) { EX(x); EX(y); CVT(hh, x, y); ADDF(ss, x); ADDF(ss, y); }                     \
    if (ID == 3) { EX(x); EX(y); CVT(hh, x, y); DOT(ss, hh); }                                  \
    if (ID == 4) { EX(x); EX(y); CVT(hh, x, y); FM(v4); FM(v5); FM(v6); FM(v7); }               \
    if (ID == 5) { EX(x); MULF(v4, x); CVT(hh, x, v4); }                                        \
    if (ID == 6) { EX(x); EX(y); CVT(hh, x, y); ADDF(ss, x); ADDF(ss, y); fr = lds_read_half8_at(la); } \
    if (ID == 7) { EX(x); EX(y); CVT(hh, x, y); ADDF(ss, x); ADDF(ss, y);                       \
                   const half4 lo = lds_read_tr16_at(la), hi = lds_read_tr16_at(la + 2048);     \
                   fr = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); }              \
    if (ID == 8) { EX(x); MULF(v4, x); CVT(hh, x, v4); fr = lds_read_half8_at(la); }            \
  } while (0)
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc0) : "v"(fr0), "v"(b)); OPS(v0, v1, h0, s0, fr0);
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc1) : "v"(fr1), "v"(b)); OPS(v2, v3, h1, s1, fr1);
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc2) : "v"(fr0), "v"(b)); OPS(v0, v1, h0, s0, fr0);
      asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc3) : "v"(fr1), "v"(b)); OPS(v2, v3, h1, s1, fr1);
    }
  }
#undef OPS
  const long long t1 = clock64();
  float s = v0 + v1 + v2 + v3 + v4 + v5 + v6 + v7 + s0 + s1 + (float)h0 + (float)h1;
  for (int i = 0; i < 16; ++i) s += acc0[i] + acc1[i] + acc2[i] + acc3[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
  if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
}
template <int ID>
static void run_chunk(const char* name) {
  const int iters = 3000;
  printf("G MFMA + %-44s", name);
  for (int waves = 4; waves <= 12; waves += 4) {
    chunk_kernel<ID><<<256, 64 * waves>>>(g_out, g_clk, 50);
    chunk_kernel<ID><<<256, 64 * waves>>>(g_out, g_clk, iters);
    CK(hipDeviceSynchronize());
    printf("  %d wave(s)/SIMD: %5.1f", waves / 4, slowest_wave_clocks(256, 0, waves) / (iters * 16.0) / (waves / 4));
  }
  printf("  clocks of SIMD time per chunk\n");
}

// ---- H: MFMAs per LDS fragment, and MFMAs chained through one accumulator -----------------------
// MPR: MFMAs per 1 KiB fragment read (1 or 2); VALU: the softmax ops of two scores per MFMA
template <int MPR, bool VALU>
__global__ __launch_bounds__(1024) void reuse_kernel(float* out, long long* clk, int iters) {
  __shared__ __attribute__((aligned(16))) char lds[65536];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) ((float*)lds)[i] = 1e-4f * (i & 1023);
  const uint32_t la = lds_address(lds) + (wave & 3) * 8192 + lane * 16;
  half8 fr[4], b0, b1;
  for (int i = 0; i < 8; ++i) { b0[i] = (half_t)(0.002f * (lane - i)); b1[i] = (half_t)(0.001f * (lane + i)); }
  for (int i = 0; i < 4; ++i) fr[i] = b0;
  floatx16 acc0 = ZERO16, acc1 = ZERO16;
  float v0 = lane, v1 = lane + 1, s0 = 0;
  unsigned h0 = 0;
  __syncthreads();
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      acc0 = mfma_f16(fr[c & 3], b0, acc0);
      if (VALU) { EX(v0); EX(v1); CVT(h0, v0, v1); ADDF(s0, v0); ADDF(s0, v1); }
      if (MPR == 2) {
        acc1 = mfma_f16(fr[c & 3], b1, acc1);
        if (VALU) { EX(v0); EX(v1); CVT(h0, v0, v1); ADDF(s0, v0); ADDF(s0, v1); }
      }
      fr[c & 3] = lds_read_half8_at(opaque(la) + (c & 3) * 1024 + (c >> 2) * 4096);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const long long t1 = clock64();
  float r = v0 + v1 + s0 + (float)h0;
  for (int i = 0; i < 8; ++i) r += (float)fr[0][i] + (float)fr[1][i] + (float)fr[2][i] + (float)fr[3][i];
  for (int i = 0; i < 16; ++i) r += acc0[i] + acc1[i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (lane == 0) clk[blockIdx.x * 16 + wave] = t1 - t0;
}
template <int MPR, bool VALU>
static void run_reuse() {
  const int iters = 2000;
  for (int waves = 4; waves <= 12; waves += 4) {
    reuse_kernel<MPR, VALU><<<256, 64 * waves>>>(g_out, g_clk, 50);
    reuse_kernel<MPR, VALU><<<256, 64 * waves>>>(g_out, g_clk, iters);
    CK(hipDeviceSynchronize());
    printf("H %d MFMA(s) per LDS fragment, softmax ops %s, %d wave(s)/SIMD: %5.1f clocks of SIMD time per MFMA\n", MPR,
           VALU ? "on " : "off", waves / 4, slowest_wave_clocks(256, 0, waves) / ((double)iters * 8 * MPR * (waves / 4)));
  }
}
template <int DIST>
__global__ __launch_bounds__(256) void chain_kernel(float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63;
  half8 a, b;
  for (int i = 0; i < 8; ++i) { a[i] = (half_t)(0.002f * (lane - i)); b[i] = (half_t)(0.001f * (lane + i)); }
  floatx16 acc[4] = {ZERO16, ZERO16, ZERO16, ZERO16};
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[c % DIST] = mfma_f16(a, b, acc[c % DIST]);
  }
  const long long t1 = clock64();
  float r = 0;
  for (int j = 0; j < 4; ++j) for (int i = 0; i < 16; ++i) r += acc[j][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (lane == 0) clk[blockIdx.x * 16 + (threadIdx.x >> 6)] = t1 - t0;
}
template <int DIST>
static void run_chain() {
  chain_kernel<DIST><<<256, 256>>>(g_out, g_clk, 2000);
  CK(hipDeviceSynchronize());
  printf("H MFMAs through %d accumulator(s) in turn: %5.1f clocks per MFMA\n", DIST, slowest_wave_clocks(256, 0, 4) / (2000.0 * 16));
}

// ---- P: what the operand DATA does to a bare MFMA stream (the device is power limited) --------
// Eight A and four B fragments read once from memory, then only MFMAs, ~5 ms per run on every
// CU.  Rate by events; shader clock = wave clocks / event time.
__global__ __launch_bounds__(256) void mfma_data_kernel(const half8* src, float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63;
  half8 a[8], b[4];
  for (int i = 0; i < 8; ++i) a[i] = src[i * 64 + lane];
  for (int i = 0; i < 4; ++i) b[i] = src[(8 + i) * 64 + lane];
  floatx16 acc[4] = {ZERO16, ZERO16, ZERO16, ZERO16};
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[c & 3] = mfma_f16(a[c & 7], b[(c >> 1) & 3], acc[c & 3]);
    if ((it & 63) == 63)  // keeps the accumulators finite without touching the operands
      for (int j = 0; j < 4; ++j)
        for (int e = 0; e < 16; ++e) acc[j][e] *= 0.0009765625f;
  }
  const long long t1 = clock64();
  float r = 0;
  for (int j = 0; j < 4; ++j)
    for (int e = 0; e < 16; ++e) r += acc[j][e];
  out[blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (threadIdx.x == 0) clk[blockIdx.x] = t1 - t0;
}
// The f32 matrix instruction (v_mfma_f32_32x32x2_f32, 64 clocks) the same way.
__global__ __launch_bounds__(256) void mfma_f32_data_kernel(const float* src, float* out, long long* clk, int iters) {
  const int lane = threadIdx.x & 63;
  float a[8], b[4];
  for (int i = 0; i < 8; ++i) a[i] = src[i * 64 + lane];
  for (int i = 0; i < 4; ++i) b[i] = src[(8 + i) * 64 + lane];
  floatx16 acc[4] = {ZERO16, ZERO16, ZERO16, ZERO16};
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < 16; ++c)
      acc[c & 3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[c & 7], b[(c >> 1) & 3], acc[c & 3], 0, 0, 0);
    if ((it & 63) == 63)
      for (int j = 0; j < 4; ++j)
        for (int e = 0; e < 16; ++e) acc[j][e] *= 0.0009765625f;
  }
  const long long t1 = clock64();
  float r = 0;
  for (int j = 0; j < 4; ++j)
    for (int e = 0; e < 16; ++e) r += acc[j][e];
  out[blockIdx.x * blockDim.x + threadIdx.x] = r;
  if (threadIdx.x == 0) clk[blockIdx.x] = t1 - t0;
}
static void run_mfma_f32_data() {
  float* src;
  CK(hipMalloc(&src, 12 * 64 * sizeof(float)));
  static float h[12 * 64];
  const char* names[] = {"zeros", "random values, sigma 1"};
  for (int mode = 0; mode < 2; ++mode) {
    unsigned s = 777;
    for (int i = 0; i < 12 * 64; ++i) {
      float u = 0;
      for (int j = 0; j < 4; ++j) { s = s * 1664525u + 1013904223u; u += (s >> 8) / 16777216.0f; }
      h[i] = mode == 0 ? 0.f : (u - 2.0f) * 1.73f;
    }
    CK(hipMemcpy(src, h, sizeof(h), hipMemcpyHostToDevice));
    const int iters = 10000;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    mfma_f32_data_kernel<<<256, 256>>>(src, g_out, g_clk, 200);
    CK(hipEventRecord(e0));
    mfma_f32_data_kernel<<<256, 256>>>(src, g_out, g_clk, iters);
    CK(hipEventRecord(e1));
    CK(hipDeviceSynchronize());
    float ms = 0;
    CK(hipEventElapsedTime(&ms, e0, e1));
    long long c0 = 0;
    CK(hipMemcpy(&c0, g_clk, 8, hipMemcpyDeviceToHost));
    printf("P bare f32 MFMA stream (32x32x2), operands = %-30s: %5.1f TFLOP/s, shader clock %.2f GHz\n", names[mode],
           256.0 * 4 * iters * 16.0 * 4096.0 / (ms * 1e-3) / 1e12, (double)c0 / (ms * 1e6));
    CK(hipEventDestroy(e0)); CK(hipEventDestroy(e1));
  }
  CK(hipFree(src));
}
static void run_mfma_data() {
  half8* src;
  CK(hipMalloc(&src, 12 * 64 * sizeof(half8)));
  static _Float16 h[12 * 64 * 8];
  const char* names[] = {"zeros", "the constant 0.5", "random values, sigma 1", "random values, sigma 1, every other lane zero"};
  for (int mode = 0; mode < 4; ++mode) {
    unsigned s = 12345;
    for (int i = 0; i < 12 * 64 * 8; ++i) {
      float u = 0;
      for (int j = 0; j < 4; ++j) { s = s * 1664525u + 1013904223u; u += (s >> 8) / 16777216.0f; }
      const float g = (u - 2.0f) * 1.73f;  // sum of four uniforms, unit variance
      h[i] = (_Float16)(mode == 0 ? 0.f : mode == 1 ? 0.5f : (mode == 3 && ((i / 8) & 1)) ? 0.f : g);
    }
    CK(hipMemcpy(src, h, sizeof(h), hipMemcpyHostToDevice));
    const int iters = 20000;
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    mfma_data_kernel<<<256, 256>>>(src, g_out, g_clk, 200);
    CK(hipEventRecord(e0));
    mfma_data_kernel<<<256, 256>>>(src, g_out, g_clk, iters);
    CK(hipEventRecord(e1));
    CK(hipDeviceSynchronize());
    float ms = 0;
    CK(hipEventElapsedTime(&ms, e0, e1));
    long long c0 = 0;
    CK(hipMemcpy(&c0, g_clk, 8, hipMemcpyDeviceToHost));
    printf("P bare MFMA stream, operands = %-46s: %5.0f TFLOP/s, shader clock %.2f GHz\n", names[mode],
           256.0 * 4 * iters * 16.0 * 32768.0 / (ms * 1e-3) / 1e12, (double)c0 / (ms * 1e6));
    CK(hipEventDestroy(e0)); CK(hipEventDestroy(e1));
  }
  CK(hipFree(src));
}

// ---- Q: f32 MFMA, A operand from LDS, AHEAD reads in flight, NCHAIN accumulators ----
template <int AHEAD, int NCHAIN>
__global__ void mfma_f32_lds_kernel(float* out, const float* in, int iters) {
  __shared__ float lds[64 * 68];
  for (int i = threadIdx.x; i < 64 * 68; i += blockDim.x) lds[i] = in[i & 1023];
  __syncthreads();
  floatx16 acc[NCHAIN];
  for (int c = 0; c < NCHAIN; ++c)
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  const float b = in[threadIdx.x & 63];
  const float* base = lds + (threadIdx.x & 31) + 4 * 68 * ((threadIdx.x >> 5) & 1);
  for (int it = 0; it < iters; ++it) {
    float a[AHEAD];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) a[u] = base[(u % 8) * 68 * 8 + (u / 8)];
#pragma unroll
    for (int u = 0; u < 64; ++u) {
      const float cur = a[u % AHEAD];
      if (u + AHEAD < 64) a[u % AHEAD] = base[((u + AHEAD) % 8) * 68 * 8 + ((u + AHEAD) / 8)];
      acc[u % NCHAIN] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur, b, acc[u % NCHAIN], 0, 0, 0);
    }
  }
  float s = 0.f;
  for (int c = 0; c < NCHAIN; ++c)
    for (int i = 0; i < 16; ++i) s += acc[c][i];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <int AHEAD, int NCHAIN>
static void run_mfma_f32_lds_one(int threads, const float* in) {
  const int iters = 400;
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  mfma_f32_lds_kernel<AHEAD, NCHAIN><<<256, threads>>>(g_out, in, iters);
  CK(hipEventRecord(e0));
  mfma_f32_lds_kernel<AHEAD, NCHAIN><<<256, threads>>>(g_out, in, iters);
  CK(hipEventRecord(e1));
  CK(hipEventSynchronize(e1));
  float ms;
  CK(hipEventElapsedTime(&ms, e0, e1));
  const double per_simd = (double)iters * 64 * (threads / 256);
  std::printf("Q  f32 MFMA, A from LDS: %d reads in flight, %d chain(s), %d wave(s)/SIMD: %5.1f ns per MFMA per SIMD "
              "(64 clocks at 2.4 GHz = 26.7), %6.1f TFLOP/s\n",
              AHEAD, NCHAIN, threads / 256, ms * 1e6 / per_simd, 1024.0 * per_simd * 4096 / (ms * 1e-3) * 1e-12);
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
}

static void run_mfma_f32_lds() {
  float* in;
  CK(hipMalloc(&in, 4096));
  float h[1024];
  for (int i = 0; i < 1024; ++i) h[i] = 0.001f * ((i * 37) % 101 - 50);
  CK(hipMemcpy(in, h, 4096, hipMemcpyHostToDevice));
  for (int rep = 0; rep < 2; ++rep) {  // the first round also brings the clocks up
    run_mfma_f32_lds_one<1, 4>(256, in);
    run_mfma_f32_lds_one<2, 4>(256, in);
    run_mfma_f32_lds_one<8, 4>(256, in);
    run_mfma_f32_lds_one<2, 1>(256, in);
    run_mfma_f32_lds_one<1, 4>(512, in);
    run_mfma_f32_lds_one<2, 4>(512, in);
    run_mfma_f32_lds_one<8, 4>(512, in);
    run_mfma_f32_lds_one<2, 1>(512, in);
  }
  CK(hipFree(in));
}

int main() {
  CK(hipMalloc(&g_out, 1024 * 1024 * sizeof(float)));
  CK(hipMalloc(&g_clk, 256 * 16 * sizeof(long long)));
  if (getenv("MICROBENCH_ONLY_P")) {
    run_mfma_data();
    run_mfma_f32_data();
    return 0;
  }
  if (getenv("MICROBENCH_ONLY_Q")) {
    run_mfma_f32_lds();
    return 0;
  }
  if (getenv("MICROBENCH_ONLY_F")) {
    run_fwd_bp<3>(1); run_fwd_bp<3>(2); run_fwd_bp<3>(3); run_fwd_bp<2, 128>(1); run_fwd_bp<2, 128>(2);
    return 0;
  }
  run_mfma_stream();
  run_mfma_data();
  run_mfma_f32_data();
  run_valu_rate<0>("v_fma_f32 independent");
  run_valu_rate<1>("v_fma_f32 dependent");
  run_valu_rate<2>("v_exp_f32");
  run_valu_rate<3>("v_max3_f32");
  run_valu_rate<4>("v_fma_f32 v, s, v");
  run_valu_rate<5>("v_cvt_pk_f16_f32");
  run_valu_rate<6>("v_dot2c_f32_f16");
  run_valu_rate<7>("v_exp_f16");
  run_side_by_side();
  run_interleaved<0>();
  run_interleaved<4>();
  run_interleaved<8>();
  run_interleaved<12>();
  run_interleaved<16>();
  half_t *Kg, *Vg;
  CK(hipMalloc(&Kg, 96 * 1024 * D * 2));
  CK(hipMalloc(&Vg, 96 * 1024 * D * 2));
  CK(hipMemset(Kg, 0, 96 * 1024 * D * 2));
  CK(hipMemset(Vg, 0, 96 * 1024 * D * 2));
  run_fwd_iteration<false, false, false>(Kg, Vg);
  run_fwd_iteration<true, false, false>(Kg, Vg);
  run_fwd_iteration<true, true, false>(Kg, Vg);
  run_fwd_iteration<true, true, true>(Kg, Vg);
  run_phase<0, 0>("free running");
  run_phase<1, 0>("opposite phases");
  run_phase<2, 0>("same phase");
  run_phase<0, 1>("free running");
  run_phase<1, 1>("opposite phases");
  run_fwd_bp<3>(1); run_fwd_bp<3>(2); run_fwd_bp<3>(3);
  run_fwd_bp<2, 128>(1); run_fwd_bp<2, 128>(2);
  run_chunk<0>("2 exp, cvt_pk");
  run_chunk<1>("2 exp, cvt_pk, add");
  run_chunk<2>("2 exp, cvt_pk, 2 add");
  run_chunk<3>("2 exp, cvt_pk, dot2c");
  run_chunk<4>("2 exp, cvt_pk, 4 fma");
  run_chunk<5>("exp, mul, cvt_pk");
  run_chunk<6>("2 exp, cvt_pk, 2 add, ds_read_b128");
  run_chunk<7>("2 exp, cvt_pk, 2 add, 2 ds_read_b64_tr_b16");
  run_chunk<8>("exp, mul, cvt_pk, ds_read_b128");
  run_reuse<1, false>(); run_reuse<2, false>(); run_reuse<1, true>(); run_reuse<2, true>();
  run_chain<1>(); run_chain<2>(); run_chain<4>();
  run_mfma_f32_lds();
  return 0;
}
