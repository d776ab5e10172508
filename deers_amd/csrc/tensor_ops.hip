// Element-wise helpers the fused attention op needs from its storage backend:
// gradient accumulation (`existing + grad`, src/backprop.rs:101-112 through
// BinaryOp Add, src/storage.rs:231-236), compaction of a strided view
// (copy_compact, src/storage.rs:305; CPU form src/storage/cpu.rs:1063-1102),
// the constant fill behind ones_like/zeros_like (src/backprop.rs:54) and unary
// negation (src/ops.rs:100-127).  All are bandwidth-bound one-pass kernels.
#include "common.h"

namespace deers {

namespace {

template <typename T>
__device__ __forceinline__ float to_f32(T v) { return (float)v; }

template <typename T>
__global__ __launch_bounds__(256) void fill_kernel(T* dst, size_t n, float value) {
  const T v = (T)value;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    dst[i] = v;
}

// f16 adds go through f32 and round once, like `half`'s software `+`.
template <typename T>
__global__ __launch_bounds__(256) void add_kernel(const T* a, const T* b, T* out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    out[i] = (T)(to_f32(a[i]) + to_f32(b[i]));
}

template <typename T>
__global__ __launch_bounds__(256) void neg_kernel(const T* a, T* out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    out[i] = (T)(-to_f32(a[i]));
}

struct View6 {
  int64_t shape[6];
  int64_t stride[6];
};

// dst (compact, row-major over `shape`) <- src viewed through `stride`.
template <typename T>
__global__ __launch_bounds__(256) void copy_strided_kernel(const T* src, T* dst, View6 v,
                                                           size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    size_t rem = i;
    int64_t off = 0;
#pragma unroll
    for (int d = 5; d >= 0; --d) {
      const size_t idx = rem % (size_t)v.shape[d];
      rem /= (size_t)v.shape[d];
      off += (int64_t)idx * v.stride[d];
    }
    dst[i] = src[off];
  }
}

// Fast path of copy_strided for views whose rows are contiguous runs of 16-byte
// chunks (unit innermost stride, everything 16-byte aligned): one thread moves one
// chunk, index arithmetic is 32-bit and runs once per 16 bytes instead of once per
// element.  `v` describes the view in chunks.
struct View6u {
  uint32_t shape[6];
  uint32_t stride[6];
};
__global__ __launch_bounds__(256) void copy_chunks_kernel(const uint4* src, uint4* dst, View6u v,
                                                          uint32_t n) {
  for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
    uint32_t rem = i, off = 0;
#pragma unroll
    for (int d = 5; d >= 0; --d) {
      const uint32_t q = rem / v.shape[d];
      off += (rem - q * v.shape[d]) * v.stride[d];
      rem = q;
    }
    dst[i] = src[off];
  }
}

inline unsigned grid_for(size_t n) {
  const size_t blocks = (n + 255) / 256;
  return (unsigned)(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
}

}  // namespace

void launch_fill(int dtype_f16, void* dst, size_t n, float value, hipStream_t stream) {
  if (dtype_f16)
    hipLaunchKernelGGL(fill_kernel<half_t>, dim3(grid_for(n)), dim3(256), 0, stream, (half_t*)dst, n, value);
  else
    hipLaunchKernelGGL(fill_kernel<float>, dim3(grid_for(n)), dim3(256), 0, stream, (float*)dst, n, value);
}

void launch_add(int dtype_f16, const void* a, const void* b, void* out, size_t n,
                hipStream_t stream) {
  if (dtype_f16)
    hipLaunchKernelGGL(add_kernel<half_t>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const half_t*)a, (const half_t*)b, (half_t*)out, n);
  else
    hipLaunchKernelGGL(add_kernel<float>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const float*)a, (const float*)b, (float*)out, n);
}

void launch_neg(int dtype_f16, const void* a, void* out, size_t n, hipStream_t stream) {
  if (dtype_f16)
    hipLaunchKernelGGL(neg_kernel<half_t>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const half_t*)a, (half_t*)out, n);
  else
    hipLaunchKernelGGL(neg_kernel<float>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const float*)a, (float*)out, n);
}

// dst viewed through dst_strides <- src viewed through src_strides, same shape
// (element-wise; used for small scatters such as a KV-cache append).
template <typename T>
__global__ __launch_bounds__(256) void copy_view_kernel(const T* src, T* dst, View6 v, View6 w,
                                                        size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    size_t rem = i;
    int64_t so = 0, dof = 0;
#pragma unroll
    for (int d = 5; d >= 0; --d) {
      const size_t idx = rem % (size_t)v.shape[d];
      rem /= (size_t)v.shape[d];
      so += (int64_t)idx * v.stride[d];
      dof += (int64_t)idx * w.stride[d];
    }
    dst[dof] = src[so];
  }
}

void launch_copy_view(int dtype_f16, const void* src, const int64_t* src_strides, void* dst,
                      const int64_t* dst_strides, const int64_t* shape, int ndim,
                      hipStream_t stream) {
  View6 v, w;
  size_t n = 1;
  for (int d = 0; d < 6; ++d) {
    const int s = d - (6 - ndim);
    v.shape[d] = w.shape[d] = s >= 0 ? shape[s] : 1;
    v.stride[d] = s >= 0 ? src_strides[s] : 0;
    w.stride[d] = s >= 0 ? dst_strides[s] : 0;
    n *= (size_t)v.shape[d];
  }
  if (n == 0) return;
  if (dtype_f16)
    hipLaunchKernelGGL(copy_view_kernel<half_t>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const half_t*)src, (half_t*)dst, v, w, n);
  else
    hipLaunchKernelGGL(copy_view_kernel<float>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const float*)src, (float*)dst, v, w, n);
}

void launch_copy_strided(int dtype_f16, const void* src, const int64_t* shape,
                         const int64_t* strides, int ndim, void* dst, hipStream_t stream) {
  View6 v;
  size_t n = 1;
  for (int d = 0; d < 6; ++d) {  // right-align the view in six dimensions
    const int s = d - (6 - ndim);
    v.shape[d] = s >= 0 ? shape[s] : 1;
    v.stride[d] = s >= 0 ? strides[s] : 0;
    n *= (size_t)v.shape[d];
  }
  if (n == 0) return;
  // rows of whole 16-byte chunks, everything aligned, offsets within 32 bits
  const int64_t per16 = dtype_f16 ? 8 : 4;
  bool chunked = v.stride[5] == 1 && v.shape[5] % per16 == 0 && n / per16 < (size_t(1) << 31) &&
                 ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
  int64_t span = 0;
  for (int d = 0; d < 5 && chunked; ++d) {
    chunked = v.stride[d] % per16 == 0;
    span += (v.shape[d] - 1) * v.stride[d];
  }
  if (chunked && (span + v.shape[5]) / per16 < (int64_t(1) << 32)) {
    View6u u;
    for (int d = 0; d < 5; ++d) {
      u.shape[d] = (uint32_t)v.shape[d];
      u.stride[d] = (uint32_t)(v.stride[d] / per16);
    }
    u.shape[5] = (uint32_t)(v.shape[5] / per16);
    u.stride[5] = 1;
    const uint32_t nc = (uint32_t)(n / per16);
    hipLaunchKernelGGL(copy_chunks_kernel, dim3(grid_for(nc)), dim3(256), 0, stream,
                       (const uint4*)src, (uint4*)dst, u, nc);
    return;
  }
  if (dtype_f16)
    hipLaunchKernelGGL(copy_strided_kernel<half_t>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const half_t*)src, (half_t*)dst, v, n);
  else
    hipLaunchKernelGGL(copy_strided_kernel<float>, dim3(grid_for(n)), dim3(256), 0, stream,
                       (const float*)src, (float*)dst, v, n);
}

}  // namespace deers
