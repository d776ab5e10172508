// Row-wise log-softmax forward and backward over the innermost axis.
//
// Replaces BackendStorage::log_softmax_fwd / log_softmax_bwd
// (src/storage.rs:284-302; CPU form src/storage/cpu.rs:793-888) behind the
// FusedLogSoftmax op (src/ops.rs:1186-1251), which the GPT loss applies to
// [B*T, vocab] logits (config 5: 8192 x 50257 f32 = 1.65 GB).
//   fwd: out = x - (ln(sum exp(x - max)) + max)       per row
//   bwd: out = g - exp(lsm) * sum(g)                   per row
// HBM-bound, and the point of the design is to touch each element of x (or grad) in
// HBM once: a row of up to ~64 K chunks-worth of elements (65 K f32, 131 K f16) is held
// in the registers of the thread group that owns it (50257 f32 = 201 KB is more than
// LDS holds, but only 52 VGPRs per thread of a 1024-thread workgroup), reduced in a
// fixed order, and written from those registers.  Narrow rows get a narrower group (a
// wavefront, or 256 threads) so that every lane has work.  Wider rows, and operands
// whose rows sit at different offsets within 16 bytes, fall back to two sweeps over
// global memory with an online (max, sum) pair.  f16 rows compute in f32 and round once.
#include "common.h"

namespace deers {

namespace {

constexpr int kLsmThreads = 512;
constexpr int kLsmUnroll = 8;  // independent loads in flight per thread

__device__ __forceinline__ void merge_ms(float& m, float& s, float m2, float s2) {
  const float mn = fmaxf(m, m2);
  // (-inf, 0) is the neutral element; guard its exp(-inf - -inf)
  const float a = (m == -INFINITY) ? 0.f : __expf(m - mn);
  const float b = (m2 == -INFINITY) ? 0.f : __expf(m2 - mn);
  s = s * a + s2 * b;
  m = mn;
}

template <typename T>
__global__ __launch_bounds__(kLsmThreads) void log_softmax_fwd_kernel(const T* x, T* out,
                                                                      int64_t inner) {
  __shared__ float red_m[kLsmThreads / 64], red_s[kLsmThreads / 64];
  const T* row = x + (int64_t)blockIdx.x * inner;
  T* orow = out + (int64_t)blockIdx.x * inner;
  const int tid = threadIdx.x;
  float m = -INFINITY, s = 0.f;
  for (int64_t i0 = tid; i0 < inner; i0 += (int64_t)kLsmThreads * kLsmUnroll) {
    float v[kLsmUnroll];
#pragma unroll
    for (int u = 0; u < kLsmUnroll; ++u) {
      const int64_t i = i0 + (int64_t)u * kLsmThreads;
      v[u] = i < inner ? (float)row[i] : -INFINITY;
    }
    float mx = v[0];
#pragma unroll
    for (int u = 1; u < kLsmUnroll; ++u) mx = fmaxf(mx, v[u]);
    if (mx > m) {  // rescale the running sum only when the maximum moves
      s *= (m == -INFINITY) ? 0.f : __expf(m - mx);
      m = mx;
    }
    if (m != -INFINITY) {
#pragma unroll
      for (int u = 0; u < kLsmUnroll; ++u) s += __expf(v[u] - m);
    }
  }
  // wave reduction (fixed butterfly order), then across waves through LDS
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(s, off, 64);
    merge_ms(m, s, m2, s2);
  }
  if ((tid & 63) == 0) {
    red_m[tid >> 6] = m;
    red_s[tid >> 6] = s;
  }
  __syncthreads();
  m = red_m[0];
  s = red_s[0];
#pragma unroll
  for (int w = 1; w < kLsmThreads / 64; ++w) merge_ms(m, s, red_m[w], red_s[w]);
  const float lse = __logf(s) + m;
  for (int64_t i0 = tid; i0 < inner; i0 += (int64_t)kLsmThreads * kLsmUnroll) {
#pragma unroll
    for (int u = 0; u < kLsmUnroll; ++u) {
      const int64_t i = i0 + (int64_t)u * kLsmThreads;
      if (i < inner) orow[i] = (T)((float)row[i] - lse);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kLsmThreads) void log_softmax_bwd_kernel(const T* grad, const T* lsm,
                                                                      T* out, int64_t inner) {
  __shared__ float red[kLsmThreads / 64];
  const T* g = grad + (int64_t)blockIdx.x * inner;
  const T* l = lsm + (int64_t)blockIdx.x * inner;
  T* orow = out + (int64_t)blockIdx.x * inner;
  const int tid = threadIdx.x;
  float s = 0.f;
  for (int64_t i0 = tid; i0 < inner; i0 += (int64_t)kLsmThreads * kLsmUnroll) {
#pragma unroll
    for (int u = 0; u < kLsmUnroll; ++u) {
      const int64_t i = i0 + (int64_t)u * kLsmThreads;
      s += i < inner ? (float)g[i] : 0.f;
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
  if ((tid & 63) == 0) red[tid >> 6] = s;
  __syncthreads();
  s = red[0];
#pragma unroll
  for (int w = 1; w < kLsmThreads / 64; ++w) s += red[w];
  for (int64_t i0 = tid; i0 < inner; i0 += (int64_t)kLsmThreads * kLsmUnroll) {
#pragma unroll
    for (int u = 0; u < kLsmUnroll; ++u) {
      const int64_t i = i0 + (int64_t)u * kLsmThreads;
      if (i < inner) orow[i] = (T)((float)g[i] - __expf((float)l[i]) * s);
    }
  }
}

// ---- rows held in registers ----
// GROUP threads own one row; a workgroup of kRegBlock threads holds kRegBlock / GROUP
// rows.  The row is cut into 16-byte chunks counted from the 128-byte line its first
// element lies in (rows start at any element: 50257 is odd), so that every access is a
// full-width dwordx4 and every wavefront access covers whole cache lines.  Chunks
// before the row are skipped; the chunks that straddle the row's ends hold neighbours'
// elements, which are replaced by the reduction's neutral element after the load and
// never stored.
// Thread t of the group holds chunks t, t + GROUP, ... (NREG of them, packed as loaded,
// so an f16 row takes half the registers of an f32 row).

constexpr int kRegBlockOf(int group) { return group < 256 ? 256 : group; }
// Waves per SIMD to compile the forward for.  A 1024-thread group is 4 waves per SIMD;
// with up to 8 chunks per thread two such groups fit a CU (64 VGPRs each), and the
// loads of one overlap the stores of the other.  (The backward streams lsm between
// its stores and does not need it; capped at 64 VGPRs it would spill.)
constexpr int kRegWavesOf(int group, int nreg) { return group == 1024 && nreg <= 8 ? 8 : 1; }

template <int GROUP>
__device__ __forceinline__ void group_reduce_ms(float& m, float& s, float* red_m, float* red_s,
                                                int t) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const float m2 = __shfl_xor(m, off, 64), s2 = __shfl_xor(s, off, 64);
    merge_ms(m, s, m2, s2);
  }
  if constexpr (GROUP > 64) {
    if ((t & 63) == 0) {
      red_m[t >> 6] = m;
      red_s[t >> 6] = s;
    }
    __syncthreads();
    m = red_m[0];
    s = red_s[0];
#pragma unroll
    for (int w = 1; w < GROUP / 64; ++w) merge_ms(m, s, red_m[w], red_s[w]);
  }
}

template <int GROUP>
__device__ __forceinline__ float group_reduce_sum(float s, float* red, int t) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
  if constexpr (GROUP > 64) {
    if ((t & 63) == 0) red[t >> 6] = s;
    __syncthreads();
    s = red[0];
#pragma unroll
    for (int w = 1; w < GROUP / 64; ++w) s += red[w];
  }
  return s;
}

// A 16-byte chunk as loaded, and its elements as floats.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <typename T> struct Elems { T e[16 / sizeof(T)]; };

template <typename T>
__device__ __forceinline__ void unpack(u32x4 c, float (&f)[16 / sizeof(T)]) {
  const Elems<T> x = __builtin_bit_cast(Elems<T>, c);
#pragma unroll
  for (int e = 0; e < (int)(16 / sizeof(T)); ++e) f[e] = (float)x.e[e];
}
template <typename T>
__device__ __forceinline__ u32x4 pack(const float (&f)[16 / sizeof(T)]) {
  Elems<T> x;
#pragma unroll
  for (int e = 0; e < (int)(16 / sizeof(T)); ++e) x.e[e] = (T)f[e];
  return __builtin_bit_cast(u32x4, x);
}

// Makes the compiler forget what it knows about a packed chunk, so that f16 -> f32
// conversions are redone where the values are used instead of being kept live (which
// would triple the registers an f16 row takes).
template <typename T>
__device__ __forceinline__ void keep_packed(u32x4& c) {
  if constexpr (sizeof(T) == 2) asm volatile("" : "+v"(c));
}

// Slices of a row are addressed through buffer descriptors (base and extent in SGPRs,
// advanced with scalar arithmetic) and ONE 32-bit byte offset per lane, which keeps
// address arithmetic out of the vector registers that hold the row.  The extent ends
// at the last chunk that overlaps the row: chunks past it load zeros and touch no
// memory.  aux = 2 marks the access non-temporal: every byte is used once.
using rsrc_t = __amdgpu_buffer_rsrc_t;
constexpr int kAuxNt = 2;

__device__ __forceinline__ rsrc_t slice_rsrc(const char* base, int n_chunks, int first_chunk) {
  const int left = n_chunks > first_chunk ? n_chunks - first_chunk : 0;
  return __builtin_amdgcn_make_buffer_rsrc((void*)(base + (int64_t)first_chunk * 16), 0, left * 16,
                                           0x00020000);
}
__device__ __forceinline__ u32x4 chunk_load(rsrc_t r, int byte_off) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, kAuxNt));
}
__device__ __forceinline__ void chunk_store(u32x4 c, rsrc_t r, int byte_off) {
  __builtin_amdgcn_raw_buffer_store_b128(
      __builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned int)))) unsigned int, c),
      r, byte_off, 0, kAuxNt);
}

// Where a row lies relative to its chunks.  Chunk 0 starts at the 128-byte line that
// holds the row's first element, so that every wavefront access covers whole cache
// lines; `head` elements (up to a line's worth) precede the row in chunks that are
// never loaded or stored.  Operands that move with the row (the output, lsm) use the
// same head, measured back from their own row start.
template <typename T>
struct RowGeom {
  int head;      // elements between the line start and the row
  int n_chunks;  // chunks from the line start to the row's end
  __device__ __forceinline__ RowGeom(const T* row, int inner) {
    constexpr int kEpc = 16 / sizeof(T);
    head = (int)((uintptr_t)row & 127) / (int)sizeof(T);
    n_chunks = (head + inner + kEpc - 1) / kEpc;
  }
  __device__ __forceinline__ const char* base_of(const T* row) const {
    return (const char*)(row - head);
  }
};

// Replaces the elements of chunk `c` (row positions lo .. lo + EPC - 1) that lie outside
// [0, inner) by `neutral`.
template <typename T>
__device__ __forceinline__ u32x4 patch_outside(u32x4 c, int lo, int inner, float neutral) {
  constexpr int kEpc = 16 / sizeof(T);
  Elems<T> x = __builtin_bit_cast(Elems<T>, c);
#pragma unroll
  for (int e = 0; e < kEpc; ++e)
    if (lo + e < 0 || lo + e >= inner) x.e[e] = (T)neutral;
  return __builtin_bit_cast(u32x4, x);
}

// Stores the elements of an edge chunk that belong to the row, one by one.
template <typename T>
__device__ __forceinline__ void store_inside(const float (&f)[16 / sizeof(T)], T* orow, int lo,
                                             int inner) {
#pragma unroll
  for (int e = 0; e < (int)(16 / sizeof(T)); ++e)
    if (lo + e >= 0 && lo + e < inner) orow[lo + e] = (T)f[e];
}

template <typename T, int GROUP, int NREG>
__global__ __launch_bounds__(kRegBlockOf(GROUP), kRegWavesOf(GROUP, NREG)) void log_softmax_fwd_reg_kernel(
    const T* x, T* out, int64_t outer, int inner) {
  __shared__ float red_m[16], red_s[16];
  constexpr int kRows = kRegBlockOf(GROUP) / GROUP;
  constexpr int kEpc = 16 / sizeof(T);
  const int t = threadIdx.x % GROUP;
  const int64_t r = (int64_t)blockIdx.x * kRows + threadIdx.x / GROUP;
  const bool live = r < outer;  // whole groups only: GROUP == 64 when kRows > 1
  const T* row = x + (live ? r : 0) * inner;
  const RowGeom<T> geo(row, inner);
  const int n_chunks = live ? geo.n_chunks : 0;  // a dead group's descriptors cover nothing
  const int lo0 = t * kEpc - geo.head;  // row position of this thread's chunk 0, element 0
  u32x4 c[NREG];
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    c[u] = u32x4{0u, 0u, 0u, 0u};
    // chunks wholly before the row (slice 0 only) are not read
    if (u > 0 || lo0 + kEpc > 0)
      c[u] = chunk_load(slice_rsrc(geo.base_of(row), n_chunks, u * GROUP), t * 16);
  }
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    const int lo = lo0 + u * GROUP * kEpc;
    if (lo < 0 || lo + kEpc > inner) c[u] = patch_outside<T>(c[u], lo, inner, -INFINITY);
  }
  float m = -INFINITY;
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    float f[kEpc];
    unpack<T>(c[u], f);
#pragma unroll
    for (int e = 0; e < kEpc; ++e) m = fmaxf(m, f[e]);
  }
  float s = 0.f;
  if (m != -INFINITY) {
#pragma unroll
    for (int u = 0; u < NREG; ++u) {
      float f[kEpc];
      keep_packed<T>(c[u]);
      unpack<T>(c[u], f);
#pragma unroll
      for (int e = 0; e < kEpc; ++e) s += __expf(f[e] - m);
    }
  }
  group_reduce_ms<GROUP>(m, s, red_m, red_s, t);
  if (!live) return;
  const float lse = __logf(s) + m;
  T* orow = out + r * inner;
  const char* obase = geo.base_of(orow);  // 16-byte aligned: checked by the launcher
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    const int lo = lo0 + u * GROUP * kEpc;
    float f[kEpc];
    keep_packed<T>(c[u]);
    unpack<T>(c[u], f);
#pragma unroll
    for (int e = 0; e < kEpc; ++e) f[e] -= lse;
    if (lo >= 0 && lo + kEpc <= inner)
      chunk_store(pack<T>(f), slice_rsrc(obase, n_chunks, u * GROUP), t * 16);
    else
      store_inside<T>(f, orow, lo, inner);
  }
}

template <typename T, int GROUP, int NREG>
__global__ __launch_bounds__(kRegBlockOf(GROUP)) void log_softmax_bwd_reg_kernel(
    const T* grad, const T* lsm, T* out, int64_t outer, int inner) {
  __shared__ float red[16];
  constexpr int kRows = kRegBlockOf(GROUP) / GROUP;
  constexpr int kEpc = 16 / sizeof(T);
  const int t = threadIdx.x % GROUP;
  const int64_t r = (int64_t)blockIdx.x * kRows + threadIdx.x / GROUP;
  const bool live = r < outer;
  const T* grow = grad + (live ? r : 0) * inner;
  const RowGeom<T> geo(grow, inner);
  const int n_chunks = live ? geo.n_chunks : 0;
  const int lo0 = t * kEpc - geo.head;
  u32x4 c[NREG];
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    c[u] = u32x4{0u, 0u, 0u, 0u};
    if (u > 0 || lo0 + kEpc > 0)
      c[u] = chunk_load(slice_rsrc(geo.base_of(grow), n_chunks, u * GROUP), t * 16);
  }
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    const int lo = lo0 + u * GROUP * kEpc;
    if (lo < 0 || lo + kEpc > inner) c[u] = patch_outside<T>(c[u], lo, inner, 0.f);
  }
  float s = 0.f;
#pragma unroll
  for (int u = 0; u < NREG; ++u) {
    float f[kEpc];
    unpack<T>(c[u], f);
#pragma unroll
    for (int e = 0; e < kEpc; ++e) s += f[e];
  }
  s = group_reduce_sum<GROUP>(s, red, t);
  if (!live) return;
  T* orow = out + r * inner;
  // 16-byte aligned like the gradient's chunks: checked by the launcher
  const char* lbase = geo.base_of(lsm + r * inner);
  const char* obase = geo.base_of(orow);
  constexpr int kBatch = NREG < 4 ? NREG : 4;  // lsm chunks in flight per thread
#pragma unroll
  for (int u0 = 0; u0 < NREG; u0 += kBatch) {
    u32x4 lc[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u)
      if (u0 + u < NREG) {
        lc[u] = u32x4{0u, 0u, 0u, 0u};
        if (u0 + u > 0 || lo0 + kEpc > 0)
          lc[u] = chunk_load(slice_rsrc(lbase, n_chunks, (u0 + u) * GROUP), t * 16);
      }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      if (u0 + u >= NREG) continue;
      const int lo = lo0 + (u0 + u) * GROUP * kEpc;
      float f[kEpc], l[kEpc];
      keep_packed<T>(c[u0 + u]);
      unpack<T>(c[u0 + u], f);
      unpack<T>(lc[u], l);
      // elements outside the row hold arbitrary lsm values; they are computed, not stored
#pragma unroll
      for (int e = 0; e < kEpc; ++e) f[e] -= __expf(l[e]) * s;
      if (lo >= 0 && lo + kEpc <= inner)
        chunk_store(pack<T>(f), slice_rsrc(obase, n_chunks, (u0 + u) * GROUP), t * 16);
      else
        store_inside<T>(f, orow, lo, inner);
    }
  }
}

template <typename T, int GROUP, int NREG>
void launch_fwd_reg(const T* x, T* out, int64_t outer, int inner, hipStream_t stream) {
  constexpr int kBlock = kRegBlockOf(GROUP);
  const int64_t blocks = (outer + kBlock / GROUP - 1) / (kBlock / GROUP);
  hipLaunchKernelGGL((log_softmax_fwd_reg_kernel<T, GROUP, NREG>), dim3((unsigned)blocks),
                     dim3(kBlock), 0, stream, x, out, outer, inner);
}

template <typename T, int GROUP, int NREG>
void launch_bwd_reg(const T* g, const T* l, T* out, int64_t outer, int inner, hipStream_t stream) {
  constexpr int kBlock = kRegBlockOf(GROUP);
  const int64_t blocks = (outer + kBlock / GROUP - 1) / (kBlock / GROUP);
  hipLaunchKernelGGL((log_softmax_bwd_reg_kernel<T, GROUP, NREG>), dim3((unsigned)blocks),
                     dim3(kBlock), 0, stream, g, l, out, outer, inner);
}

// Chunks from a row's line start to its end, at worst over all rows.  Row r starts
// (first + r * pitch) mod 128 bytes into its line; those offsets step by gcd(pitch, 128).
template <typename T>
int64_t worst_chunks(const T* first_row, int64_t inner) {
  constexpr int kEpc = 16 / sizeof(T);
  const int64_t pitch = inner * (int64_t)sizeof(T);
  int64_t g = 128;
  while (pitch % g) g /= 2;
  const int64_t max_head_bytes = (int64_t)((uintptr_t)first_row % (uintptr_t)g) + 128 - g;
  return (max_head_bytes / (int64_t)sizeof(T) + inner + kEpc - 1) / kEpc;
}
inline bool same_phase(const void* a, const void* b) {
  return (((uintptr_t)a ^ (uintptr_t)b) & 15) == 0;
}

// 16 chunks of f32 (64 values) fill the 128 VGPRs a 1024-thread workgroup leaves each
// thread; an f16 chunk unpacks to 8 floats while it is worked on, so 8 is its limit.
template <typename T> constexpr int kMaxChunksPerThread = sizeof(T) == 4 ? 16 : 8;

template <typename T>
void dispatch_fwd(const T* x, T* out, int64_t outer, int64_t inner, hipStream_t stream) {
  const int64_t n = worst_chunks<T>(x, inner);
  // the chunked kernels need x and out rows at the same offset within 16 bytes
  if (!same_phase(x, out) || n > 1024 * kMaxChunksPerThread<T>)
    hipLaunchKernelGGL(log_softmax_fwd_kernel<T>, dim3((unsigned)outer), dim3(kLsmThreads), 0,
                       stream, x, out, inner);
  else if (n <= 64 * 1) launch_fwd_reg<T, 64, 1>(x, out, outer, (int)inner, stream);
  else if (n <= 64 * 4) launch_fwd_reg<T, 64, 4>(x, out, outer, (int)inner, stream);
  else if (n <= 256 * 4) launch_fwd_reg<T, 256, 4>(x, out, outer, (int)inner, stream);
  else if (n <= 256 * 8) launch_fwd_reg<T, 256, 8>(x, out, outer, (int)inner, stream);
  else if (n <= 256 * 13) launch_fwd_reg<T, 256, 13>(x, out, outer, (int)inner, stream);
  else if (n <= 1024 * 4) launch_fwd_reg<T, 1024, 4>(x, out, outer, (int)inner, stream);
  else if (n <= 1024 * 8) launch_fwd_reg<T, 1024, 8>(x, out, outer, (int)inner, stream);
  else if constexpr (sizeof(T) == 4) {
    if (n <= 1024 * 13) launch_fwd_reg<T, 1024, 13>(x, out, outer, (int)inner, stream);
    else launch_fwd_reg<T, 1024, 16>(x, out, outer, (int)inner, stream);
  }
}

template <typename T>
void dispatch_bwd(const T* g, const T* l, T* out, int64_t outer, int64_t inner,
                  hipStream_t stream) {
  const int64_t n = worst_chunks<T>(g, inner);
  if (!same_phase(g, l) || !same_phase(g, out) || n > 1024 * kMaxChunksPerThread<T>)
    hipLaunchKernelGGL(log_softmax_bwd_kernel<T>, dim3((unsigned)outer), dim3(kLsmThreads), 0,
                       stream, g, l, out, inner);
  else if (n <= 64 * 1) launch_bwd_reg<T, 64, 1>(g, l, out, outer, (int)inner, stream);
  else if (n <= 64 * 4) launch_bwd_reg<T, 64, 4>(g, l, out, outer, (int)inner, stream);
  else if (n <= 256 * 4) launch_bwd_reg<T, 256, 4>(g, l, out, outer, (int)inner, stream);
  else if (n <= 256 * 8) launch_bwd_reg<T, 256, 8>(g, l, out, outer, (int)inner, stream);
  else if (n <= 256 * 13) launch_bwd_reg<T, 256, 13>(g, l, out, outer, (int)inner, stream);
  else if (n <= 1024 * 4) launch_bwd_reg<T, 1024, 4>(g, l, out, outer, (int)inner, stream);
  else if (n <= 1024 * 8) launch_bwd_reg<T, 1024, 8>(g, l, out, outer, (int)inner, stream);
  else if constexpr (sizeof(T) == 4) {
    if (n <= 1024 * 13) launch_bwd_reg<T, 1024, 13>(g, l, out, outer, (int)inner, stream);
    else launch_bwd_reg<T, 1024, 16>(g, l, out, outer, (int)inner, stream);
  }
}

}  // namespace

void launch_log_softmax_fwd(int dtype_f16, const void* x, void* out, int64_t outer, int64_t inner,
                            hipStream_t stream) {
  LaunchScope scope("log_softmax_fwd", stream);
  if (dtype_f16) dispatch_fwd((const half_t*)x, (half_t*)out, outer, inner, stream);
  else dispatch_fwd((const float*)x, (float*)out, outer, inner, stream);
}

void launch_log_softmax_bwd(int dtype_f16, const void* grad, const void* lsm, void* out,
                            int64_t outer, int64_t inner, hipStream_t stream) {
  LaunchScope scope("log_softmax_bwd", stream);
  if (dtype_f16)
    dispatch_bwd((const half_t*)grad, (const half_t*)lsm, (half_t*)out, outer, inner, stream);
  else
    dispatch_bwd((const float*)grad, (const float*)lsm, (float*)out, outer, inner, stream);
}

}  // namespace deers
