// Launchers of the generic BackendStorage kernels (storage_ops.hip).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace deers {

// values of the `op` argument of deers_rocm_unary / deers_rocm_binary
enum {
  kUnaryNeg = 0, kUnaryExp, kUnaryLog, kUnarySin, kUnaryCos, kUnaryTanh, kUnaryRelu,
  kUnaryReluBackward, kUnaryScalarAdd, kUnaryScalarMul, kUnaryScalarDiv, kUnaryPowf, kUnaryCount
};
enum { kBinaryAdd = 0, kBinarySub, kBinaryMul, kBinaryDiv, kBinaryPow, kBinaryEq, kBinaryCount };

constexpr int kMaxViewDims = 8;
// A strided view of at most 2^32 - 1 elements: extents and element strides (0 for a
// broadcast dimension, negative allowed), outermost dimension first.
struct StridedView {
  int ndim;
  uint32_t shape[kMaxViewDims];
  int64_t stride[kMaxViewDims];
};

// view == nullptr: the operand is compact
void launch_unary(int dtype_f16, int op, const void* x, const StridedView* view, void* out, int64_t n,
                  double param, hipStream_t stream);
void launch_binary(int dtype_f16, int op, const void* a, const StridedView* va, const void* b,
                   const StridedView* vb, void* out, int64_t n, hipStream_t stream);
void launch_reduce(int dtype_f16, int op_max, const void* x, void* out, int64_t outer, int64_t rs,
                   hipStream_t stream);
void launch_log_sum_exp(int dtype_f16, const void* x, void* out, int64_t outer, int64_t rs,
                        hipStream_t stream);
void launch_gather(int elem_bytes, const void* src, const int64_t* idx, void* out, int64_t left,
                   int64_t src_dim, int64_t index_len, int64_t right, int* error_flag,
                   hipStream_t stream);
void launch_scatter_add(int dtype_f16, const void* src, const int64_t* idx, void* dst, int64_t left,
                        int64_t dst_dim, int64_t index_len, int64_t right, int* error_flag,
                        hipStream_t stream);

}  // namespace deers
