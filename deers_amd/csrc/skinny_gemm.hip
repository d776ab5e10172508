// y[M, N] (+)= x[M, K] @ W[K, N] for M <= 32 rows, f16 storage, f32 accumulation: the
// projections of a generation step, where the batch is the only row dimension and the
// product is a single pass over the weights (src/nn.rs:183-190 with x of 32 rows;
// 1-5 MB of weights against 50-200 KB of activations).  A library GEMM spends 7-12 us on
// such a product; this kernel is one streaming read of W.
//
// Decomposition
//   grid   one workgroup per 32 columns of W; its 4 waves split K into quarters and
//          reduce their partial sums through LDS at the end (fixed order).
//   MFMA   C^T[n, m] += W^T[n, k] x^T[k, m] on v_mfma_f32_32x32x16_f16: the lane owns
//          one row m of y; W^T fragments come from the row-major W tile in LDS through
//          ds_read_b64_tr_b16 (the same transposed read the attention kernels use for V).
//   loads  global -> LDS without registers (global_load_lds_dwordx4), 4 k-steps of 16 per
//          chunk, a ring of 3 chunks per wave (2 in flight while one is consumed).  Each
//          wave reads only the LDS it filled itself: no barrier inside the loop.
//   split  when the column blocks alone are too few to occupy the chip (N = 768 gives 24),
//          K is also split over S workgroups per column block.  All S of a block run on
//          one XCD (block id % 8), write their partial tiles to a workspace in that XCD's
//          L2, and the one that arrives last (a counter per column block, reset by that
//          workgroup) adds the S partials in index order: one launch, same bits whoever
//          is last.
//   x      optionally transformed on the way in, so that a generation step needs no launch
//          of its own for them: kSkinnyReluSq squares the positive part of every x element
//          as it leaves LDS (the MLP's activation, src/models/gpt.rs:196-203; the same
//          f32 arithmetic and single rounding as the stand-alone kernel); kSkinnyRmsNorm
//          multiplies row m of the result by (mean(x[m,:]^2) + eps)^-1/2, which is
//          rms_norm(x) @ W (src/nn.rs:244-251) without the rounding of the normalised row
//          to f16 in between; the sums of squares are taken from the x tiles the MFMAs
//          read anyway.  The latter needs a workgroup to see all of K (no split).
//   W      row-major [K][N], or packed as [N/32 column blocks][K][32]: a workgroup's share of
//          a row-major W is 64 bytes out of every row, and fetched from HBM (a generation
//          step cycles through more weights and cache than the last-level cache holds) such
//          scattered pieces cost 2-3 us per launch more than the same bytes in one run.
// Shapes: K a multiple of 256 (every wave then owns whole chunks), N a multiple of 8,
// rows 16-byte aligned; the caller falls back to the library otherwise.
#include "common.h"

namespace deers {

namespace {

constexpr int kSkinnyPlain = 0, kSkinnyRmsNorm = 1, kSkinnyReluSq = 2;  // the entry point's codes
constexpr int kSkWaves = 4;
constexpr int kSkStepsPerChunk = 4;           // k-steps of 16
constexpr int kSkRing = 3;                    // chunks per wave in LDS
constexpr int kSkStepBytes = 2048;            // W tile [16 k x 32 n] + x tile [32 m x 16 k], f16
constexpr int kSkChunkBytes = kSkStepsPerChunk * kSkStepBytes;
constexpr int kSkWaveBytes = kSkRing * kSkChunkBytes;
constexpr int kSkLds = kSkWaves * kSkWaveBytes;  // 96 KB
constexpr int kSkPieceBytes = 256 * 64;          // prefetch unit: 256 rows of a packed tile

template <bool ACCUMULATE, int PROLOGUE>
__global__ __launch_bounds__(256) void skinny_gemm_f16_kernel(const half_t* __restrict__ x, int64_t ldx,
                                                              const half_t* __restrict__ W, int64_t ldw,
                                                              half_t* __restrict__ y, int64_t ldy, int M,
                                                              int N, int K, int S, float* __restrict__ partial,
                                                              int* __restrict__ counters, float eps,
                                                              int64_t w_block_stride, int main_blocks,
                                                              const char* __restrict__ next_w,
                                                              int next_tiles, int next_tile_bytes) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  if ((int)blockIdx.x >= main_blocks) {
    // Prefetch role (workgroups past the product's own, on CUs the product leaves idle):
    // touch the packed weight of the product that follows, each tile from the XCD whose L2
    // its consumer will read it through (block id % 8, the same mapping as below), so that
    // product finds its weights in L2 instead of HBM.  Results are discarded.
    // A tile of K rows (64 bytes each) is cut into pieces of 256 rows, one workgroup each,
    // so that a long K does not make the prefetch outlast the product it rides on.
    const int pid = (int)blockIdx.x - main_blocks;  // main_blocks is a multiple of 8
    const int pieces = next_tile_bytes / kSkPieceBytes;
    const int q = pid >> 3;
    const int tile = (q / pieces) * 8 + (pid & 7), piece = q % pieces;
    if (tile < next_tiles) {
      // the same register-free loads as the product's own, all in flight at once; they land
      // in this wave's LDS ring, where nobody reads them
      const int pw = __builtin_amdgcn_readfirstlane(tid >> 6);
      const int per_wave = kSkPieceBytes / kSkWaves;  // 4 KB
      const char* src = next_w + (int64_t)tile * next_tile_bytes + (int64_t)piece * kSkPieceBytes +
                        (int64_t)pw * per_wave;
      const uint32_t dst = lds_address(smem) + pw * kSkWaveBytes;
      for (int i = 0; i < per_wave / 1024; ++i)
        async_load16_to_lds((const half_t*)(src + i * 1024), (uint32_t)(lane * 16),
                            dst + (uint32_t)((i % (kSkWaveBytes / 1024)) * 1024));
      wait_vmcnt<0>();  // the LDS allocation must outlive the writes into it
    }
    return;
  }
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 5;
  // block id -> (column block, K split): the S splits of a column block share id % 8
  const int n_col_blocks = (N + 31) / 32;
  const int xcd = blockIdx.x & 7, t_id = blockIdx.x >> 3;
  const int split = t_id % S;
  const int col_block = (t_id / S) * 8 + xcd;
  if (col_block >= n_col_blocks) return;
  const int n0 = col_block * 32;
  const int k_per_wave = K / (S * kSkWaves);               // a multiple of 64
  const int n_chunks = k_per_wave / (16 * kSkStepsPerChunk);
  const int k_begin = (split * kSkWaves + wave) * k_per_wave;
  const uint32_t lds_wave = lds_address(smem) + wave * kSkWaveBytes;

  // W tile of a step: lane -> row lane/4 of 16, 16-byte piece lane%4 of the 64-byte row;
  // pieces past column N repeat the last valid one (their results are never stored)
  const int w_row = lane >> 2;
  const int w_piece = min(lane & 3, (N - n0) / 8 - 1);
  const uint32_t w_lane_off = (uint32_t)((w_row * ldw + 8 * w_piece) * 2);
  // x tile of a step: lane -> row lane/2 of 32 (clamped to M-1), 16-byte piece lane%2
  const int x_row = min(lane >> 1, M - 1);
  const uint32_t x_lane_off = (uint32_t)((x_row * ldx + 8 * (lane & 1)) * 2);
  // row-major W: the block's 32 columns start 32 elements after the previous block's, rows
  // ldw apart; packed W ([column block][K][32]): blocks K*32 apart, rows 32 apart
  const half_t* w_base = W + col_block * w_block_stride;

  auto issue = [&](int chunk) {
    const uint32_t dst = lds_wave + (chunk % kSkRing) * kSkChunkBytes;
#pragma unroll
    for (int i = 0; i < kSkStepsPerChunk; ++i) {
      const int k0 = k_begin + (chunk * kSkStepsPerChunk + i) * 16;
      async_load16_to_lds(w_base + (int64_t)k0 * ldw, w_lane_off, dst + i * kSkStepBytes);
      async_load16_to_lds(x + k0, x_lane_off, dst + i * kSkStepBytes + 1024);
    }
  };
  issue(0);
  if (n_chunks > 1) issue(1);

  floatx16 acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  float sum_sq = 0.f;  // kSkinnyRmsNorm: this lane's share of sum(x[m,:]^2), m = lane % 32
  for (int c = 0; c < n_chunks; ++c) {
    if (c + 2 < n_chunks) {
      issue(c + 2);
      wait_vmcnt<4 * kSkStepsPerChunk>();  // two younger chunks may still be in flight
    } else if (c + 1 < n_chunks) {
      wait_vmcnt<2 * kSkStepsPerChunk>();
    } else {
      wait_vmcnt<0>();
    }
    const char* chunk = smem + wave * kSkWaveBytes + (c % kSkRing) * kSkChunkBytes;
#pragma unroll
    for (int i = 0; i < kSkStepsPerChunk; ++i) {
      const half_t* wt = (const half_t*)(chunk + i * kSkStepBytes);          // [16][32]
      const half_t* xt = (const half_t*)(chunk + i * kSkStepBytes + 1024);   // [32][16]
      const half8 a = lds_frag_transposed(wt, 32, 0, 0, lane);  // column lane%32; k = 4g..4g+3, 8+4g..
      const half4 b_lo = *(const half4*)(xt + (lane & 31) * 16 + 4 * g);
      const half4 b_hi = *(const half4*)(xt + (lane & 31) * 16 + 8 + 4 * g);
      half8 b = __builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7);
      if constexpr (PROLOGUE == kSkinnyReluSq) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float r = fmaxf((float)b[e], 0.f);
          b[e] = (half_t)(r * r);
        }
      }
      if constexpr (PROLOGUE == kSkinnyRmsNorm) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sum_sq = fmaf((float)b[e], (float)b[e], sum_sq);
      }
      acc = mfma_f16(a, b, acc);
    }
    // the ring slot this chunk sat in is refilled two iterations from now by this same
    // wave, after these reads have returned (the MFMAs above consumed them)
  }

  // ---- reduce the four waves' partial sums (fixed order) and write 16 bytes per lane ----
  __syncthreads();  // every wave is done with its ring: reuse the start of LDS
  float* red = (float*)smem;  // [wave][reg][lane]
#pragma unroll
  for (int r = 0; r < 16; ++r) red[(wave * 16 + r) * 64 + lane] = acc[r];
  float* red_sq = red + kSkWaves * 16 * 64;  // [wave][lane]
  if constexpr (PROLOGUE == kSkinnyRmsNorm) red_sq[wave * 64 + lane] = sum_sq;
  __syncthreads();
  float s[8];
  const int rp = wave & 1;  // waves 0 and 1 sum and store output columns n0 + 16 rp .. + 15
  if (wave < 2) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float t = red[(0 * 16 + 8 * rp + e) * 64 + lane];
#pragma unroll
      for (int w = 1; w < kSkWaves; ++w) t += red[(w * 16 + 8 * rp + e) * 64 + lane];
      s[e] = t;
    }
    if constexpr (PROLOGUE == kSkinnyRmsNorm) {
      // row m's sum of squares: both lane halves of all four waves, in a fixed order
      float t = 0.f;
#pragma unroll
      for (int w = 0; w < kSkWaves; ++w) t += red_sq[w * 64 + (lane & 31)] + red_sq[w * 64 + 32 + (lane & 31)];
      const float inv = 1.0f / sqrtf(t / (float)K + eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] *= inv;
    }
  }
  if (S > 1) {
    // this workgroup's partial tile: [column block][split][rp][lane][8] floats
    float* mine = partial + ((((int64_t)col_block * S + split) * 2 + rp) * 64 + lane) * 8;
    if (wave < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) mine[e] = s[e];
    }
    // The S workgroups of a column block share one XCD and so one L2: a completed store
    // (vmcnt 0) is in that L2, and relaxed device-scope atomics, which bypass the CU's
    // own cache, are all the ordering needed; no cache write-back or invalidation.
    wait_all_vmem();
    __syncthreads();
    __shared__ int last_flag;
    if (tid == 0) {
      const int arrived =
          __hip_atomic_fetch_add(counters + col_block, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = arrived == S - 1;
      if (last_flag)  // ready for the next launch
        __hip_atomic_store(counters + col_block, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last_flag) return;
    if (wave < 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = 0.f;
      for (int sp = 0; sp < S; ++sp) {  // index order, whoever arrived last
        const float* theirs = partial + ((((int64_t)col_block * S + sp) * 2 + rp) * 64 + lane) * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          s[e] += __hip_atomic_load(theirs + e, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  if (wave < 2) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int m = lane & 31;
    const int col = n0 + 16 * rp + 8 * g;  // this lane's 8 output columns after the exchange
    // Before the exchange the lane holds columns 16rp + 4g + {0..3} (s[0..3]) and
    // 16rp + 8 + 4g + {0..3} (s[4..7]) of row m; its partner (lane ^ 32) the other halves.
    half4 lo, hi;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lo[e] = (half_t)s[e];
      hi[e] = (half_t)s[4 + e];
    }
    if constexpr (ACCUMULATE) {
      // the addend is added in f32 before the one rounding: fetch the lane's own columns
      if (m < M) {
        const int c_lo = n0 + 16 * rp + 4 * g, c_hi = c_lo + 8;
        if (c_lo < N) {
          const half4 old = *(const half4*)(y + (int64_t)m * ldy + c_lo);
#pragma unroll
          for (int e = 0; e < 4; ++e) lo[e] = (half_t)(s[e] + (float)old[e]);
        }
        if (c_hi < N) {
          const half4 old = *(const half4*)(y + (int64_t)m * ldy + c_hi);
#pragma unroll
          for (int e = 0; e < 4; ++e) hi[e] = (half_t)(s[4 + e] + (float)old[e]);
        }
      }
    }
    const u32x2 xu = __builtin_bit_cast(u32x2, lo), yu = __builtin_bit_cast(u32x2, hi);
    const auto r0 = __builtin_amdgcn_permlane32_swap(xu[0], yu[0], false, false);
    const auto r1 = __builtin_amdgcn_permlane32_swap(xu[1], yu[1], false, false);
    if (m < M && col < N) *(u32x4*)(y + (int64_t)m * ldy + col) = u32x4{r0[0], r1[0], r0[1], r1[1]};
  }
}

}  // namespace

// true if the kernel takes this product (see the shape rules above)
bool skinny_gemm_takes(int64_t m, int64_t n, int64_t k, int64_t ldx, int64_t ldw, int64_t ldy,
                       const void* x, const void* w, const void* y) {
  if (m < 1 || m > 32 || n < 8 || n % 8 || k < 256 || k % 256) return false;
  if (ldx % 8 || ldw % 8 || ldy % 8 || ldx < k || ldw < n || ldy < n) return false;
  if (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) return false;
  if (k * ldw * 2 >= ((int64_t)1 << 31) || 32 * ldx * 2 >= ((int64_t)1 << 31)) return false;
  return true;
}

// Number of K splits per column block for this shape.  A split costs a trip through the
// workspace and the arrival counter (~1.5 us), so it only pays when one workgroup's share
// of K is long: every split keeps at least 768 of K (32x768x3072: 12.0 us unsplit, 8.5 us
// in four splits; 32x768x768: 4.0 us unsplit, 5.6 us in three).
int skinny_gemm_splits(int64_t n, int64_t k) {
  const int64_t col_blocks = (n + 31) / 32, units = k / 256;  // a split owns whole 256-deep units
  int best = 1;
  for (int sp = 2; sp <= units / 3 && sp <= 16; ++sp)
    if (units % sp == 0) {
      best = sp;
      if (col_blocks * sp >= 96) break;
    }
  return col_blocks >= 96 ? 1 : best;
}
size_t skinny_gemm_workspace_bytes(int64_t n, int splits) {
  return splits > 1 ? (size_t)((n + 31) / 32) * splits * 2 * 64 * 8 * sizeof(float) : 0;
}

template <bool ACCUMULATE, int PROLOGUE>
static void launch_one(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy, int m,
                       int n, int k, int splits, float* partial, int* counters, float eps, bool packed,
                       const SkinnyPrefetch& next, hipStream_t stream) {
  static bool attr_set = false;  // launches are serialised by the caller
  if (!attr_set) {
    (void)hipFuncSetAttribute((const void*)skinny_gemm_f16_kernel<ACCUMULATE, PROLOGUE>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, kSkLds);
    attr_set = true;
  }
  const int col_blocks = (n + 31) / 32;
  const int main_blocks = 8 * splits * ((col_blocks + 7) / 8);
  const int next_tiles = next.w ? (int)((next.n + 31) / 32) : 0;
  const int pieces = next.w ? (int)(next.k / 256) : 0;  // K % 256 == 0 for every weight the kernel takes
  const dim3 grid((unsigned)(main_blocks + 8 * ((next_tiles + 7) / 8) * pieces));
  hipLaunchKernelGGL((skinny_gemm_f16_kernel<ACCUMULATE, PROLOGUE>), grid, dim3(256), kSkLds, stream,
                     (const half_t*)x, ldx, (const half_t*)w, packed ? (int64_t)32 : ldw, (half_t*)y, ldy, m, n, k,
                     splits, partial, counters, eps, packed ? (int64_t)k * 32 : (int64_t)32, main_blocks,
                     (const char*)next.w, next_tiles, (int)(next.k * 64));
}

// prologue: kSkinnyPlain, kSkinnyRmsNorm (splits must be 1) or kSkinnyReluSq; packed: w is
// [ceil(n/32)][k][32] (each workgroup's columns contiguous) instead of row-major
void launch_skinny_gemm_f16(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy,
                            int m, int n, int k, bool accumulate, int prologue, float eps, bool packed,
                            int splits, float* partial, int* counters, const SkinnyPrefetch& next,
                            hipStream_t stream) {
#define DEERS_SKINNY_CASE(ACC, PRO)                                                                      \
  if (accumulate == ACC && prologue == PRO)                                                              \
    return launch_one<ACC, PRO>(x, ldx, w, ldw, y, ldy, m, n, k, splits, partial, counters, eps, packed, next, stream);
  DEERS_SKINNY_CASE(false, kSkinnyPlain)
  DEERS_SKINNY_CASE(true, kSkinnyPlain)
  DEERS_SKINNY_CASE(false, kSkinnyRmsNorm)
  DEERS_SKINNY_CASE(true, kSkinnyRmsNorm)
  DEERS_SKINNY_CASE(false, kSkinnyReluSq)
  DEERS_SKINNY_CASE(true, kSkinnyReluSq)
#undef DEERS_SKINNY_CASE
}

}  // namespace deers
