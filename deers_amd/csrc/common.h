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

// Exchange with the lane 32 away (the other half of the wave).
__device__ __forceinline__ float swap32(float x) { return __shfl_xor(x, 32, 64); }

// ds_read_b64_tr_b16: within each group of 16 lanes, lane 4r+c supplies the
// address of 4 consecutive halfs (row r, columns 4c..4c+3 of a 4x16 block) and
// lane i receives column i of rows 0..3.
__device__ __forceinline__ half4 lds_read_tr16(const half_t* p) {
  fp16x4_raw r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((DEERS_LDS fp16x4_raw*)(p));
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

__device__ __forceinline__ half8 pack_half8(float a0, float a1, float a2, float a3, float a4,
                                            float a5, float a6, float a7) {
  half8 r;
  r[0] = (half_t)a0; r[1] = (half_t)a1; r[2] = (half_t)a2; r[3] = (half_t)a3;
  r[4] = (half_t)a4; r[5] = (half_t)a5; r[6] = (half_t)a6; r[7] = (half_t)a7;
  return r;
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

struct BwdParams {
  const void* q; const void* k; const void* v; const void* o; const void* d_o;
  const float* lse; float* delta;  // delta: [B,H,T] workspace, rowsum(dO o O)
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
};

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
