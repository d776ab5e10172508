// Shared device-side types and helpers for the gfx950 attention kernels.
//
// MFMA operand conventions used throughout (wave64, lane l, g = l / 32):
//   v_mfma_f32_32x32x16_f16   A: lane holds A[i = l%32][k = 8g .. 8g+7]
//                             B: lane holds B[k = 8g .. 8g+7][j = l%32]
//   v_mfma_f32_32x32x2_f32    A: lane holds A[i = l%32][k = g],  B: B[k = g][j = l%32]
//   accumulator (16 floats)   reg r holds C[i = 8*(r/4) + 4g + r%4][j = l%32]
// The k index of a contraction is only a label: any assignment of contraction
// elements to (g, slot) works as long as A and B use the same one.  The kernels
// use this to feed an accumulator tile straight back in as a B operand: regs
// 8s..8s+7 of a 32x32 accumulator are rows {4g..4g+3, 8+4g..8+4g+3} + 16s.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace deers {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __attribute__((__vector_size__(4 * sizeof(__fp16)))) __fp16 fp16x4_raw;

#define DEERS_LDS __attribute__((address_space(3)))

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ floatx16 mfma_f16(half8 a, half8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mfma_f32(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// Reductions over the lane pair (l, l^32) with v_permlane32_swap: called with
// (x, x) it returns {low half broadcast to both halves, high half broadcast}.
__device__ __forceinline__ float pair_max(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float pair_sum(float x) {
  const unsigned u = __float_as_uint(x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// Writes one 32-column block of an output row from a 32x32 accumulator (the lane owns
// the row; element 4*rq + e is column 8*rq + 4*g + e, g = lane / 32).  A lane holds 4
// consecutive columns of each 8-column group and its partner (lane ^ 32) the other 4:
// the pair trades halves of two groups, so each lane writes 16 contiguous bytes (two
// 16-byte stores per block instead of four 8-byte ones).  `dst` points at the block's
// first column in this lane's row and must be 16-byte aligned.
__device__ __forceinline__ void store_block_f16(half_t* dst, const floatx16& acc, float mul, int g) {
  typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int rp = 0; rp < 2; ++rp) {
    half4 x, y;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x[e] = (half_t)(acc[8 * rp + e] * mul);
      y[e] = (half_t)(acc[8 * rp + 4 + e] * mul);
    }
    const u32x2 xu = __builtin_bit_cast(u32x2, x), yu = __builtin_bit_cast(u32x2, y);
    const auto r0 = __builtin_amdgcn_permlane32_swap(xu[0], yu[0], false, false);
    const auto r1 = __builtin_amdgcn_permlane32_swap(xu[1], yu[1], false, false);
    *(u32x4*)(dst + 16 * rp + 8 * g) = u32x4{r0[0], r1[0], r0[1], r1[1]};
  }
}
// Kept for the f32 kernels: exchange with the lane 32 away.
__device__ __forceinline__ float swap32(float x) { return __shfl_xor(x, 32, 64); }

// ds_read_b64_tr_b16: within each group of 16 lanes, lane 4r+c supplies the
// address of 4 consecutive halfs (row r, columns 4c..4c+3 of a 4x16 block) and
// lane i receives column i of rows 0..3.
__device__ __forceinline__ half4 lds_read_tr16(const half_t* p) {
  fp16x4_raw r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((DEERS_LDS fp16x4_raw*)(p));
  return __builtin_bit_cast(half4, r);
}

// Hides a value's provenance from the optimiser.  Used on per-iteration LDS base
// addresses: without it the compiler re-associates (slot base + lane offset + row
// constant) into one add per read instead of one add per iteration plus an
// instruction immediate.
__device__ __forceinline__ uint32_t opaque(uint32_t x) {
  asm volatile("" : "+v"(x));
  return x;
}

// 16-byte reads from a 32-bit LDS byte address (constant parts of the address written as
// "+ constant" at the call site end up in the instruction's offset field).
__device__ __forceinline__ half8 lds_read_half8_at(uint32_t lds_addr) {
  return *(DEERS_LDS const half8*)(uintptr_t)lds_addr;
}
__device__ __forceinline__ floatx4 lds_read_float4_at(uint32_t lds_addr) {
  return *(DEERS_LDS const floatx4*)(uintptr_t)lds_addr;
}

// Same read from a 32-bit LDS byte address.
__device__ __forceinline__ half4 lds_read_tr16_at(uint32_t lds_addr) {
  fp16x4_raw r =
      __builtin_amdgcn_ds_read_tr16_b64_v4f16((DEERS_LDS fp16x4_raw*)(uintptr_t)lds_addr);
  return __builtin_bit_cast(half4, r);
}

// A-operand fragment (8 halfs) for the lane's fixed column `col_base + l%32` of a
// row-major LDS tile, contraction rows {4g..4g+3} + row_base and {8+4g..} + row_base:
// the transposed operand that pairs with accumulator regs 8s..8s+7 used as B.
// `tile` points at element [0][0]; `ld` is the row stride in halfs.
__device__ __forceinline__ half8 lds_frag_transposed(const half_t* tile, int ld, int row_base,
                                                     int col_base, int lane) {
  const int g = lane >> 5;
  const int r = (lane & 15) >> 2;
  const int c = lane & 3;
  const int col = col_base + ((lane >> 4) & 1) * 16 + 4 * c;
  const half_t* p0 = tile + (row_base + 4 * g + r) * ld + col;
  half4 lo = lds_read_tr16(p0);
  half4 hi = lds_read_tr16(p0 + 8 * ld);
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Asynchronous global -> LDS copy of 16 bytes per lane (global_load_lds_dwordx4):
// lane i's 16 bytes land at lds_addr + 16*i, where lds_addr is a wave-uniform LDS
// byte address.  Completion is tracked by vmcnt; pair with wait_vmcnt<N>() and a
// barrier before other waves read the data.
__device__ __forceinline__ void async_load16_to_lds(const void* gptr, uint32_t lds_addr) {
  const uint32_t uniform = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(uniform)
               : "memory");
}
// Same copy with the address split into a wave-uniform 64-bit base (SGPR pair) and a
// per-lane unsigned 32-bit byte offset, so advancing to the next tile is scalar work.
__device__ __forceinline__ void async_load16_to_lds(const void* uniform_base, uint32_t lane_off,
                                                    uint32_t lds_addr) {
  const uint32_t uniform = __builtin_amdgcn_readfirstlane(lds_addr);
  const uint64_t b = (uint64_t)uniform_base;
  // readfirstlane returns a signed int: widen through uint32_t, never sign-extend
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sbase = ((uint64_t)hi << 32) | (uint64_t)lo;
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(sbase),
               "s"(uniform)
               : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Waits for every outstanding vector-memory operation with an instruction the
// compiler can see.  The compiler's own wait insertion knows nothing of the
// asynchronous copies above; if a register filled by an ordinary global load might
// still be pending when a loop is entered, it puts "s_waitcnt vmcnt(0)" at the
// first use inside the loop, which also waits for the copies prefetched for later
// iterations.  Call this once after the prologue's ordinary loads.
__device__ __forceinline__ void wait_all_vmem() {
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), expcnt and lgkmcnt untouched
}
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(size_t)(DEERS_LDS const void*)p;
}

// XOR swizzle of 16-byte chunks for unpadded row-major f16 tiles in LDS (rows of
// CH chunks).  Chunk c of row r is stored at chunk position c ^ lds_swizzle(r), so
// that 8 consecutive rows read at the same logical chunk hit 8 different 16-byte
// bank groups.  Invariant under r -> r + 32 (and r + 16 for CH <= 16).
template <int CH>
__device__ __forceinline__ int lds_swizzle(int row) {
  // Two access patterns must be conflict-free.  (a) 16-byte reads by 16 lanes on 16
  // consecutive rows at one logical chunk: rows that share a 256-byte bank line
  // position need distinct swizzles.  (b) transposed 8-byte reads by 32 lanes on 4
  // consecutive rows x 4 consecutive chunks: rows on the same bank line position
  // must move the aligned group of 4 chunks as a whole, i.e. differ in chunk bit 2+.
  if constexpr (CH == 4) return (row >> 2) & 3;  // 4 rows per bank line
  if constexpr (CH == 8) {                       // 2 rows per bank line
    const int t = (row >> 1) & 7;
    return ((t & 1) << 2) | (t >> 1);
  }
  return ((row & 3) << 2) | ((row >> 2) & 3);    // CH == 16: every row on the same banks
}

// 4 bytes per lane variant (global_load_lds_dword): lane i's dword lands at
// lds_addr + 4*i.
__device__ __forceinline__ void async_load4_to_lds(const void* uniform_base, uint32_t lane_off,
                                                   uint32_t lds_addr) {
  const uint32_t uniform = __builtin_amdgcn_readfirstlane(lds_addr);
  const uint64_t b = (uint64_t)uniform_base;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sbase = ((uint64_t)hi << 32) | (uint64_t)lo;
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dword %0, %1" ::"v"(lane_off), "s"(sbase),
               "s"(uniform)
               : "memory");
}

__device__ __forceinline__ half8 pack_half8(float a0, float a1, float a2, float a3, float a4,
                                            float a5, float a6, float a7) {
  half8 r;
  r[0] = (half_t)a0; r[1] = (half_t)a1; r[2] = (half_t)a2; r[3] = (half_t)a3;
  r[4] = (half_t)a4; r[5] = (half_t)a5; r[6] = (half_t)a6; r[7] = (half_t)a7;
  return r;
}

// sum += a.x + a.y in f32 (v_dot2_f32_f16 against (1,1)).
__device__ __forceinline__ float add_half2(half2v a, float sum) {
  return __builtin_amdgcn_fdot2(a, half2v{(half_t)1.f, (half_t)1.f}, sum, false);
}

// Element strides of one [B,H,T,D] tensor (D stride is 1).
struct Strides3 {
  int64_t b, h, t;
};

struct FwdParams {
  const void* q; const void* k; const void* v; void* o; float* lse;
  Strides3 sq, sk, sv, so;
  int H, T;
  float scale_log2;  // scale * log2(e)
};

// Whether the single-launch f16 backward runs its dQ groups shortest first: when a group
// (one block length over all heads) is at least an eighth of the workgroups the device
// holds at once (attn_bwd_f16.hip).
inline bool bwd_dq_short_first(int group_wgs, int capacity) { return 8 * group_wgs >= capacity; }

struct BwdParams {
  const void* q; const void* k; const void* v; const void* o; const void* d_o;
  const float* lse; float* delta;  // delta: [B,H,T] workspace, rowsum(dO o O)
  // f16 path workspace, rows padded to a multiple of 64 per head (t_pad), written by the dQ
  // role and read by the dK/dV role: lse2 = -LSE*log2(e) (-inf in the padding), negdelta =
  // -rowsum(dO o O) (0 in the padding), and qs = f16(Q * scale * log2(e)), [B*H][t_pad][D]
  // compact: the scaled queries the forward and the dQ role form their scores from, so that
  // all three kernels exponentiate the same scores
  float* lse2; float* negdelta; void* qs; int t_pad;
  // ready[bh * n_blocks + q_block] == epoch once the lse2 / negdelta rows of that 128-row
  // query block are published (f16 path, hand-over inside one launch); epoch 0: the flags
  // are not used (two launches in stream order).  *error is set to 1 by a workgroup whose
  // bounded wait for a flag ran out (spin_limit polls) and read by the host after the next sync.
  int* ready; int* error; int epoch; int spin_limit;
  void* dq; void* dk; void* dv;
  Strides3 sq, sk, sv, so, sdo, sdq, sdk, sdv;
  int H, T;
  float scale, scale_log2;
};

struct DecodeParams {
  const void* q; const void* k; const void* v; void* o;
  float* part_o; float* part_ml;  // split partials: [B*H, splits, D], [B*H, splits, 2]
  int64_t skb, skh, skl;          // cache strides (elements)
  int H, L, splits, chunk;
  float scale_log2;
  // append form: the new token's projections [B,H,D] by element strides in_b, in_h, the
  // D/2 cos / sin entries of its position; its rotated key and its value become cache
  // row L (the cache holds L rows when the kernel starts) and take part in the softmax
  const void* q_in; const void* k_in; const void* v_in;
  const void* cos_row; const void* sin_row;
  int64_t in_b, in_h;
};

// The packed weight ([ceil(n/32)][k][32] f16) of the few-rows product that will follow the
// one being launched; w == nullptr: none.
struct SkinnyPrefetch {
  const void* w = nullptr;
  int64_t n = 0, k = 0;
};

// Maps a block id (blockIdx.x, or blockIdx.x minus a multiple of 8) to (head, block
// rank).  Workgroups are dealt round-robin to the 8 XCDs, so id % 8 is the XCD: every block of one head is given to one XCD
// (its operands stay in that XCD's L2) and each XCD's list is ordered longest
// first (rank 0 = the block with the most iterations), which is what the
// dispatcher's in-order hand-out to free slots needs for an even finish.
// Returns false for padding ids.
// (The head and rank stay in vector registers on purpose: forcing them into scalar
// registers with readfirstlane was measured and raises the kernels' vector register
// count through the address arithmetic the compiler then hoists out of the loops.)
__device__ __forceinline__ bool map_block(int block_id, int n_blocks, int heads_per_xcd, int BH,
                                          int* bh, int* rank) {
  const int xcd = block_id & 7;
  const int idx = block_id >> 3;
  *bh = (idx % heads_per_xcd) * 8 + xcd;
  *rank = idx / heads_per_xcd;
  return *bh < BH;
}

// Brackets one kernel launch with a hipEvent pair when per-kernel profiling is
// switched on (deers_rocm_profile_enable); a no-op otherwise.  Defined in
// runtime.hip.
struct LaunchScope {
  LaunchScope(const char* name, hipStream_t stream);
  ~LaunchScope();
  LaunchScope(const LaunchScope&) = delete;
  LaunchScope& operator=(const LaunchScope&) = delete;

 private:
  void* rec_;
  hipStream_t stream_;
};

}  // namespace deers
