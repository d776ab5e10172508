/*
 * deers_rocm.h — C ABI of the MI355X (gfx950) causal self-attention path for deers.
 *
 * This is the boundary a `Device::Rocm` storage backend in deers
 * (a `src/storage/rocm.rs` next to src/storage/cuda.rs) binds with `extern "C"`.
 * Plain pointers and sizes only.  Every function returns 0 on success and a
 * non-zero DEERS_ROCM_ERR_* code on failure; the message for the calling
 * thread's last failure is available from deers_rocm_last_error(), which is
 * what the Rust side wraps into its backend error variant (the role
 * `Error::Cuda(String)` plays at src/error.rs:40-41).
 *
 * Conventions shared by all entry points
 *  - One process-global runtime, one device ordinal, one in-order stream; every
 *    launch and copy below is enqueued on that stream and returns without
 *    waiting, except deers_rocm_dtoh and deers_rocm_sync (the reference's CUDA
 *    backend behaves the same way: src/storage/cuda.rs:462-521, 1541-1555,
 *    1598-1602).
 *  - The caller owns every buffer it passes.  The library keeps no pointer past
 *    the call and never frees caller memory.  Internal workspace (softmax
 *    statistics and scaled queries of the backward pass, split partial results of decode) is owned
 *    and cached by the library.
 *  - Entry points may be called from any thread; they serialise on an internal
 *    mutex.
 *  - dtype: DEERS_ROCM_F16 (IEEE half storage, f32 accumulate) or
 *    DEERS_ROCM_F32.
 *  - Tensors are logical [B,H,T,D].  A `strides` argument gives the four
 *    element strides in that order (the reference's Layout strides,
 *    src/layout.rs:151-155); NULL means compact row-major.  The innermost (D)
 *    stride must be 1 and rows must be 16-byte aligned; other layouts are
 *    rejected with DEERS_ROCM_ERR_LAYOUT and the caller compacts first, as
 *    FusedLogSoftmax::forward does for its argument (src/ops.rs:1205).
 */
#ifndef DEERS_ROCM_H
#define DEERS_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DEERS_ROCM_F16 0
#define DEERS_ROCM_F32 1
#define DEERS_ROCM_I64 2 /* DType::I64 data: accepted by deers_rocm_gather only */

#define DEERS_ROCM_OK 0
#define DEERS_ROCM_ERR_HIP 1         /* a HIP runtime call failed */
#define DEERS_ROCM_ERR_ARG 2         /* null pointer, bad dtype, unsupported size */
#define DEERS_ROCM_ERR_LAYOUT 3      /* strides the kernels cannot consume */
#define DEERS_ROCM_ERR_NOT_INIT 4    /* deers_rocm_init has not succeeded */
#define DEERS_ROCM_ERR_INDEX 5       /* an index tensor held a value out of range; reported by
                                        the next deers_rocm_sync / _dtoh (Error::IndexOutOfBounds) */
#define DEERS_ROCM_ERR_HANDOVER 6    /* a workgroup of the backward gave up waiting for another
                                        workgroup's results; reported by the next deers_rocm_sync /
                                        _dtoh, the way a backend failure becomes Error::Cuda(String)
                                        (src/error.rs:40-41) */

/* ---- runtime ------------------------------------------------------------ */

/* Creates the process-global runtime on device `ordinal` (idempotent for the
 * same ordinal).  Replaces the lazily-built CUDA runtime: context, default
 * stream, module load (src/storage/cuda.rs:492-528). */
int deers_rocm_init(int ordinal);

/* 1 if a gfx950 device is present and the runtime can be (or was) created,
 * else 0.  Replaces `is_available()` (src/storage/cuda.rs:647-649,
 * src/device.rs:36-46). */
int deers_rocm_available(void);

/* Blocks until all work enqueued so far has finished.  Replaces
 * `synchronize()` (src/storage/cuda.rs:1598-1602, src/device.rs:65-75). */
int deers_rocm_sync(void);

/* Message of the calling thread's most recent failure ("" if none).  The
 * pointer stays valid until the same thread's next failing call. */
const char* deers_rocm_last_error(void);

/* The HIP stream all work is enqueued on (a hipStream_t), for callers that
 * want to order their own work after it. */
void* deers_rocm_stream(void);

/* ---- hand-overs between workgroups ----------------------------------------
 * Two kernels pass data between workgroups inside one launch: the f16 attention backward
 * (row statistics published by one half of the grid, read by the other) and the few-rows
 * GEMM (K splits summed by the last workgroup to arrive).  Both publish with a drained
 * store plus a relaxed flag / counter, which is sufficient only while producer and
 * consumer run on the same XCD (one L2); the kernels arrange that by workgroup id % 8.
 * deers_rocm_init checks what that mapping assumes, in the spirit of the capability
 * checks of the reference's runtime construction (src/storage/cuda.rs:492-528), and
 * otherwise selects forms without such a hand-over: the backward as two launches in
 * stream order, the few-rows GEMM unsplit.  Same results either way (the backward bit for
 * bit). */
#define DEERS_ROCM_HANDOVER_STREAM_ORDER 0
#define DEERS_ROCM_HANDOVER_SAME_XCD 1
/* The rule itself, callable without a device: SAME_XCD only for an unpartitioned MI355X
 * (256 compute units) with no CU mask in the environment. */
int deers_rocm_handover_policy(int cu_count, int cu_mask_set);
/* The mode in force (after deers_rocm_init; -1 before), and an override: mode -1 returns
 * to the policy's choice for this device.  Asking for SAME_XCD on a device whose policy is
 * STREAM_ORDER is refused with DEERS_ROCM_ERR_ARG (the hand-over through one L2 is not valid
 * there).  A backward call made while the library stream is being captured into a HIP graph
 * takes the two-launch form without flags by itself: the single launch's flag epoch is a
 * kernel argument, so a replayed launch would find its flags already set.  Such a call must
 * have been made once outside capture with the same geometry (workspace and flags grow
 * there). */
int deers_rocm_handover_mode(void);
int deers_rocm_set_handover_mode(int mode);

/* ---- device memory (the storage backend's alloc / to-device / to_vec) ---- */

/* Replaces stream.alloc / alloc_zeros (src/storage/cuda.rs, `zeros` at
 * src/device.rs:77-90).  `bytes` may be 0 (returns a NULL pointer). */
int deers_rocm_alloc(size_t bytes, void** out_ptr);
int deers_rocm_alloc_zeros(size_t bytes, void** out_ptr);
/* Blocks are cached by size: free returns at once, without waiting for the device, and
 * a later alloc of the same size reuses the block.  That is safe because all of the
 * library's work runs in order on one stream (a buffer the caller also uses on another
 * stream must be ordered by the caller).  A block leaves the cache when hipMalloc runs
 * out of memory or deers_rocm_empty_cache is called. */
int deers_rocm_free(void* ptr);
int deers_rocm_empty_cache(void);

/* Host->device copy, replaces CpuStorage::to(device) (src/storage/cpu.rs:26-32).
 * Returns after the host buffer may be reused. */
int deers_rocm_htod(void* dst_device, const void* src_host, size_t bytes);
/* Device->host copy; waits for prior work, replaces to_vec
 * (src/storage/cuda.rs:1541-1555). */
int deers_rocm_dtoh(void* dst_host, const void* src_device, size_t bytes);
/* Device->device copy on the stream (storage clone). */
int deers_rocm_dtod(void* dst_device, const void* src_device, size_t bytes);

/* ---- device timers (hipEvent pairs on the library stream) ---------------- */
/* Replaces the per-launch start/end events the CUDA backend feeds its profiler
 * with (src/storage/cuda.rs:530-561). */
int deers_rocm_timer_create(void** out_timer);
int deers_rocm_timer_start(void* timer);
int deers_rocm_timer_stop(void* timer);
/* Waits for the stop event and returns the elapsed milliseconds. */
int deers_rocm_timer_elapsed_ms(void* timer, float* out_ms);
int deers_rocm_timer_destroy(void* timer);

/* ---- per-kernel device times ---------------------------------------------- */
/* When enabled, every kernel the library launches is bracketed by a hipEvent
 * pair, the way the reference's CUDA backend reports per-launch device time to
 * its profiler (src/storage/cuda.rs:530-561, src/profiler.rs:361-367).
 * enable(1) clears earlier records; collect() waits for the stream, aggregates
 * by kernel name and returns the number of rows; row(i) reads one aggregate
 * (name pointer valid until the next collect/enable). */
int deers_rocm_profile_enable(int on);
int deers_rocm_profile_collect(int* out_rows);
int deers_rocm_profile_row(int index, const char** out_name, int64_t* out_calls,
                           float* out_total_ms);

/* ---- the attention path --------------------------------------------------- */

/* Fused forward of the attention core of CausalSelfAttention::forward
 * (src/models/gpt.rs:139-144):
 *     O = softmax(Q K^T * scale + causal_mask) V
 * which the reference evaluates as matmul -> scalar_mul -> causal_mask
 * (src/nn/functional.rs:12-55) -> add -> log_sum_exp -> sub -> exp -> matmul,
 * materialising [B,H,T,T] at each step.  Also writes LSE[B,H,T] (float32,
 * compact), the natural-log row sums of the masked scaled scores, which is what
 * the backward pass consumes instead of a saved probability tensor.
 * q,k,v,o: [B,H,T,D] of `dtype`; D in {32,64,128}; T >= 1. */
int deers_rocm_attn_fwd(int dtype,
                        const void* q, const int64_t* q_strides,
                        const void* k, const int64_t* k_strides,
                        const void* v, const int64_t* v_strides,
                        void* o, const int64_t* o_strides,
                        float* lse,
                        int64_t B, int64_t H, int64_t T, int64_t D, float scale);

/* Fused backward: given dO, returns dQ, dK, dV equal to what the reference's
 * autograd sweep (src/backprop.rs:52-66) produces through MatMul, Exp, Sub,
 * Broadcast, LogSumExp, Add, ScalarMul and MatMul backward
 * (src/ops.rs:1089-1101, 422-425, 210-214, 777-799, 1162-1175, 638-643):
 *     P = exp(S*scale + mask - LSE);  dV = P^T dO;  dP = dO V^T;
 *     dS = P o (dP - rowsum(dO o O));  dQ = scale dS K;  dK = scale dS^T Q.
 * o and lse are the forward outputs.  dq,dk,dv are overwritten (not
 * accumulated into); the caller's GradientStore::accumulate
 * (src/backprop.rs:101-112) adds them to existing gradients. */
int deers_rocm_attn_bwd(int dtype,
                        const void* q, const int64_t* q_strides,
                        const void* k, const int64_t* k_strides,
                        const void* v, const int64_t* v_strides,
                        const void* o, const int64_t* o_strides,
                        const float* lse,
                        const void* d_o, const int64_t* do_strides,
                        void* dq, const int64_t* dq_strides,
                        void* dk, const int64_t* dk_strides,
                        void* dv, const int64_t* dv_strides,
                        int64_t B, int64_t H, int64_t T, int64_t D, float scale);

/* Decode: one query token per (b,h) against a KV cache of length L.  Same math
 * as the forward with tgt_len = 1 and seqlen_offset = L-1, where the mask row
 * is all zero (src/nn/functional.rs:26,42; tests/nn.rs:221-232); the reference
 * has no KV cache and re-runs the whole window per token
 * (examples/tinystories_train.rs:250-276).
 * q,o: [B,H,D] compact.  k_cache,v_cache: [B,H,L_cap,D] with element strides
 * `kv_strides` = {b,h,l} (NULL: compact with L_cap = L); only rows [0,L) are
 * read.  D in {32,64,128}. */
int deers_rocm_attn_decode(int dtype,
                           const void* q,
                           const void* k_cache, const void* v_cache,
                           const int64_t* kv_strides,
                           void* o,
                           int64_t B, int64_t H, int64_t L, int64_t D, float scale);

/* deers_rocm_attn_decode for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, same kernels and bit-identical results;
 * the split partial results live in a fixed 512 KiB device array that is part of the
 * library image, so the call performs no hipMalloc / hipFree and never grows a
 * workspace.  A problem whose partials (B*H*splits*(D+2) floats, only when heads are
 * split over workgroups, i.e. B*H < 256) would not fit is rejected with
 * DEERS_ROCM_ERR_ARG.  All calls on a device share the one array: calls that overlap
 * on the device (other streams, other processes' copies aside) would race; the library
 * stream runs them in order. */
int deers_rocm_attn_decode_noalloc(int dtype,
                                   const void* q,
                                   const void* k_cache, const void* v_cache,
                                   const int64_t* kv_strides,
                                   void* o,
                                   int64_t B, int64_t H, int64_t L, int64_t D, float scale);

/* One generation step of the attention core in one launch: deers_rocm_decode_qkv followed by
 * deers_rocm_attn_decode.  q, k, v are the new token's projections [B,H,D] by element strides
 * in_strides = {b, h} (D stride 1); q and k are rotated at the token's position (cos_row /
 * sin_row: the D/2 table entries of that position, src/models/gpt.rs:49-73), the rotated k and
 * v become row `pos` of the caches ([B,H,capacity,D] by cache_strides = {b, h, t}; rows
 * [0,pos) hold the earlier tokens) and o [B,H,D] (compact) is the attention of the rotated q
 * over rows [0,pos].  Same values as the two separate calls up to the order of the f32
 * softmax sums (the new row is merged last).  D in {32,64,128}, f16.  The reference has no KV
 * cache (examples/tinystories_train.rs:250-276 re-runs the window). */
int deers_rocm_attn_decode_append(int dtype, const void* q, const void* k, const void* v,
                                  const int64_t* in_strides, const void* cos_row,
                                  const void* sin_row, void* k_cache, void* v_cache,
                                  const int64_t* cache_strides, void* o, int64_t pos,
                                  int64_t capacity, int64_t B, int64_t H, int64_t D, float scale);

/* ---- element-wise helpers of the storage backend ---------------------------
 * The fused op's contract needs four more things from its backend: the seed of
 * the reverse sweep, gradient accumulation, compaction of strided views, and (for
 * the autograd contract tests) a unary op.  All work on `n` elements of `dtype`,
 * are enqueued on the library stream and may alias (`out` == `a`). */

/* dst[i] = value.  Replaces the backend half of Tensor::ones_like / zeros_like
 * (src/backprop.rs:54, 96-98). */
int deers_rocm_fill(int dtype, void* dst, size_t n, float value);

/* out[i] = a[i] + b[i] on compact operands: what GradientStore::accumulate does
 * through `&*existing + &grad` (src/backprop.rs:101-112; BinaryOp dispatch
 * src/storage.rs:231-236).  f16 adds round once from the f32 sum. */
int deers_rocm_add(int dtype, const void* a, const void* b, void* out, size_t n);

/* out[i] = -a[i] (UnaryOp Neg, src/ops.rs:100-127). */
int deers_rocm_neg(int dtype, const void* a, void* out, size_t n);

/* dst (compact row-major over `shape`) <- src read through element `strides`;
 * ndim in 1..6, strides non-negative (0 = broadcast).  Replaces
 * BackendStorage::copy_compact (src/storage.rs:305; src/storage/cpu.rs:1063-1102),
 * which the fused op calls on inputs whose innermost stride is not 1. */
int deers_rocm_copy_compact(int dtype, const void* src, const int64_t* shape,
                            const int64_t* strides, int ndim, void* dst);

/* ---- row-wise log-softmax --------------------------------------------------------
 * The fused op of the loss (FusedLogSoftmax, src/ops.rs:1186-1251) over compact
 * [outer, inner] data, innermost axis reduced; replaces
 * BackendStorage::log_softmax_fwd / log_softmax_bwd (src/storage.rs:284-302; CPU
 * src/storage/cpu.rs:793-888).  f16 computes in f32 and rounds once.  out may alias
 * x (forward) or grad (backward). */
int deers_rocm_log_softmax_fwd(int dtype, const void* x, void* out, int64_t outer, int64_t inner);
/* out = grad - exp(lsm) * rowsum(grad), lsm = the forward's output. */
int deers_rocm_log_softmax_bwd(int dtype, const void* grad, const void* lsm, void* out,
                               int64_t outer, int64_t inner);

/* ---- the other ops of a GPT training step -------------------------------------------
 * Indices and targets are int64 in device memory, as DType::I64 tensors are in the
 * reference.  A value out of range cannot be seen by the host before the launch: the
 * kernels skip it (they never follow it) and raise a flag that the next
 * deers_rocm_sync / deers_rocm_dtoh returns as DEERS_ROCM_ERR_INDEX, the counterpart of
 * Error::IndexOutOfBounds (src/storage/cpu.rs:591-597). */

/* out[i, :] = table[indices[i], :]: BackendStorage::index_select along dim 0
 * (src/storage.rs:263-270; CPU src/storage/cpu.rs:555-610), the embedding lookup of
 * src/nn.rs:216-224.  table [n_rows, width], out [n_indices, width], compact. */
int deers_rocm_index_select(int dtype, const void* table, const int64_t* indices, void* out,
                            int64_t n_rows, int64_t n_indices, int64_t width);
/* dst[indices[i], :] += src[i, :] for i ascending: BackendStorage::index_add along dim 0
 * (src/storage.rs:272-280; CPU src/storage/cpu.rs:612-660, 954-975), the backward of
 * index_select (src/ops.rs:1429-1447).  dst [n_rows, width] is accumulated into (zero
 * it first for the reference's semantics); additions happen in the reference's order,
 * so the result is the same bits and reproducible (any number of indices: the library
 * walks long index vectors in slices, in order). */
int deers_rocm_index_add(int dtype, const void* src, const int64_t* indices, void* dst,
                         int64_t n_rows, int64_t n_indices, int64_t width);
/* index_select / index_add along a dimension other than the first
 * (src/storage/cpu.rs:936-975 with left_len > 1): the `left` slabs of a compact
 * [left, dim, right] tensor are contiguous, so the caller issues one call per slab with
 * width = right.  CpuStorage::cat (src/storage/cpu.rs:47-90) concatenates compact
 * buffers: one deers_rocm_dtod per part. */

/* ---- the generic kernels of BackendStorage (src/storage.rs:227-306) ------------------
 * What the reference's op graph calls where no fused op applies.  Outputs are compact
 * (src/storage.rs:224-226).  Arithmetic is f32 with one rounding to the storage type,
 * as the reference's f16 kernels do (convert, operate, convert back). */

/* `op` of deers_rocm_unary: the UnaryOp kernels of src/storage.rs:32-123 and
 * ewise_powf (src/storage.rs:228).  `param` is the scalar of the SCALAR_* ops (cast
 * f64 -> f32 -> storage type, src/storage.rs:105-123) or the exponent of POWF (cast
 * f64 -> f32 only, src/storage/cpu.rs:203-235); ignored otherwise. */
#define DEERS_ROCM_UNARY_NEG 0
#define DEERS_ROCM_UNARY_EXP 1
#define DEERS_ROCM_UNARY_LOG 2
#define DEERS_ROCM_UNARY_SIN 3
#define DEERS_ROCM_UNARY_COS 4
#define DEERS_ROCM_UNARY_TANH 5
#define DEERS_ROCM_UNARY_RELU 6          /* max(x, 0); NaN -> 0 as f32::max */
#define DEERS_ROCM_UNARY_RELU_BACKWARD 7 /* x > 0 ? 1 : 0 */
#define DEERS_ROCM_UNARY_SCALAR_ADD 8
#define DEERS_ROCM_UNARY_SCALAR_MUL 9
#define DEERS_ROCM_UNARY_SCALAR_DIV 10
#define DEERS_ROCM_UNARY_POWF 11
/* out (compact, row-major over `shape`) = op(x read through element `strides`).
 * BackendStorage::unary_op / ewise_powf; CPU src/storage/cpu.rs:203-265, 1021-1061.
 * ndim in 1..8; strides NULL = compact, otherwise any sign, 0 = broadcast.  A strided
 * or not 16-byte aligned operand is limited to 2^32 - 1 elements. */
int deers_rocm_unary(int dtype, int op, const void* x, int ndim, const int64_t* shape,
                     const int64_t* strides, double param, void* out);

/* `op` of deers_rocm_binary: the BinaryOp kernels of src/storage.rs:126-190. */
#define DEERS_ROCM_BINARY_ADD 0
#define DEERS_ROCM_BINARY_SUB 1
#define DEERS_ROCM_BINARY_MUL 2
#define DEERS_ROCM_BINARY_DIV 3
#define DEERS_ROCM_BINARY_POW 4 /* powf(a, b) */
#define DEERS_ROCM_BINARY_EQ 5  /* a == b ? 1 : 0 */
/* out (compact) = op(a, b), both operands of `shape` read through their own strides
 * (NULL = compact; the Broadcast op hands over stride-0 views, src/ops.rs:730-804).
 * BackendStorage::binary_op; CPU src/storage/cpu.rs:267-321, 982-1019. */
int deers_rocm_binary(int dtype, int op, const void* a, const int64_t* a_strides, const void* b,
                      const int64_t* b_strides, int ndim, const int64_t* shape, void* out);

#define DEERS_ROCM_REDUCE_SUM 0
#define DEERS_ROCM_REDUCE_MAX 1 /* NaNs ignored unless the whole run is NaN, as f32::max */
/* out[i] = sum / max of x[i*reduce_size .. (i+1)*reduce_size), x compact.
 * BackendStorage::reduce (src/storage.rs:238; CPU src/storage/cpu.rs:323-357).  Runs of
 * up to 32 elements are reduced left to right in the storage type (the reference's
 * order and rounding); longer runs are summed in f32 in a fixed tree order, so a sum
 * differs from the reference's by reassociation (f32) and is more accurate than its
 * f16 accumulator (f16). */
int deers_rocm_reduce(int dtype, int op, const void* x, void* out, int64_t outer,
                      int64_t reduce_size);
/* out[i] = ln sum_j exp(x[i, j]) over compact rows: the maximum, then
 * ln(sum exp(x - max)) + max, special values as in the reference.
 * BackendStorage::log_sum_exp (src/storage.rs:282-283; CPU src/storage/cpu.rs:755-791). */
int deers_rocm_log_sum_exp(int dtype, const void* x, void* out, int64_t outer,
                           int64_t reduce_size);

/* out[l, i, r] = src[l, indices[l, i, r], r]; src compact [left, src_dim, right],
 * indices and out compact [left, index_len, right].  BackendStorage::gather
 * (src/storage.rs:243-249; CPU src/storage/cpu.rs:398-462, 891-912); F16, F32 or I64
 * data.  Out-of-range indices are skipped and reported as DEERS_ROCM_ERR_INDEX by the
 * next deers_rocm_sync / deers_rocm_dtoh. */
int deers_rocm_gather(int dtype, const void* src, const int64_t* indices, void* out, int64_t left,
                      int64_t src_dim, int64_t index_len, int64_t right);
/* dst[l, indices[l, i, r], r] += src[l, i, r] for i ascending; src and indices compact
 * [left, index_len, right], dst compact [left, dst_dim, right], accumulated into (zero
 * it first for the reference's semantics).  BackendStorage::scatter_add
 * (src/storage.rs:252-260; CPU src/storage/cpu.rs:464-553, 914-934).  One thread owns an
 * output column (l, :, r) and applies its additions in the reference's order with its
 * rounding (the storage type after every addition): same bits, no atomics. */
int deers_rocm_scatter_add(int dtype, const void* src, const int64_t* indices, void* dst,
                           int64_t left, int64_t dst_dim, int64_t index_len, int64_t right);

/* y = x * (mean(x^2 over the last axis) + eps)^-0.5: RMSNorm::forward (src/nn.rs:244-251)
 * in one pass over compact [outer, inner]; and its backward
 * dx = inv * dy - x * inv^3 * sum(dy * x) / inner from x and dy. */
int deers_rocm_rms_norm_fwd(int dtype, const void* x, void* y, int64_t outer, int64_t inner,
                            double eps);
int deers_rocm_rms_norm_bwd(int dtype, const void* x, const void* dy, void* dx, int64_t outer,
                            int64_t inner, double eps);
/* dx = addend + rms_norm_bwd(x, dy): RMSNorm's backward followed by GradientStore::accumulate
 * onto a gradient its input already holds (src/backprop.rs:101-112; in a block, the
 * residual branch's, src/models/gpt.rs:237-239) in one pass.  The gradient is rounded to
 * the storage type before the addition: same bits as deers_rocm_rms_norm_bwd followed by
 * deers_rocm_add.  addend may be dx. */
int deers_rocm_rms_norm_bwd_add(int dtype, const void* x, const void* dy, const void* addend, void* dx,
                                int64_t outer, int64_t inner, double eps);
/* y = relu(x)^2, the MLP activation `y.relu(); &y * &y` (src/models/gpt.rs:196-197), and
 * its backward dx = dy * 2 * relu(x). */
int deers_rocm_relu_sq_fwd(int dtype, const void* x, void* y, int64_t n);
int deers_rocm_relu_sq_bwd(int dtype, const void* x, const void* dy, void* dx, int64_t n);
/* out[i] (int64, device) = index of the largest element of row i of compact
 * [outer, inner] data, the lowest index on ties: the greedy (temperature 0) case of
 * the reference's sampling, which it does on the host after to_vec
 * (examples/tinystories_train.rs:262-272).  Keeping the pick on the device lets the next
 * token's embedding lookup read it without a host round trip. */
int deers_rocm_argmax_rows(int dtype, const void* x, int64_t* out, int64_t outer, int64_t inner);
/* loss::cross_entropy (src/loss.rs:11-24): *loss (a float in device memory) =
 * -mean_i log_softmax(logits)[i, targets[i]] over compact [n_rows, n_classes] logits,
 * without writing the log-probabilities; row_lse [n_rows] (f32, device) receives each
 * row's ln sum exp for the backward. */
int deers_rocm_cross_entropy_fwd(int dtype, const void* logits, const int64_t* targets,
                                 float* row_lse, float* loss, int64_t n_rows, int64_t n_classes);
/* dlogits = (softmax(logits) - onehot(targets)) * upstream / n_rows, from the logits and
 * the forward's row_lse; `upstream` is the gradient of the scalar loss in device memory
 * (NULL = 1). */
int deers_rocm_cross_entropy_bwd(int dtype, const void* logits, const int64_t* targets,
                                 const float* row_lse, const float* upstream, void* dlogits,
                                 int64_t n_rows, int64_t n_classes);
/* deers_rocm_cross_entropy_fwd that also writes dlogits = (softmax(logits) - onehot(targets)) / n_rows,
 * what deers_rocm_cross_entropy_bwd gives for an upstream gradient of one (same bits), while the
 * row it has just reduced is still in the caches: one pass over the logits less than the two
 * calls.  For the loss of a training step, whose gradient is the seed of the reverse sweep
 * (src/backprop.rs:52-66, Tensor::backward seeds ones); another upstream gradient is applied
 * afterwards with deers_rocm_scale_by_scalar. */
int deers_rocm_cross_entropy_fwd_grad(int dtype, const void* logits, const int64_t* targets, float* row_lse,
                                      float* loss, void* dlogits, int64_t n_rows, int64_t n_classes);
/* x[i] *= *factor, with the factor in device memory (a scalar tensor such as the gradient of a
 * loss); a launch that finds the factor equal to one leaves x untouched and costs a few
 * microseconds.  ScalarMul by a tensor-valued scalar (src/ops.rs:638-643) without a host read. */
int deers_rocm_scale_by_scalar(int dtype, void* x, int64_t n, const float* factor);

/* ---- optimizer step ---------------------------------------------------------------
 * One AdamW update of one parameter tensor in place, the body of the loop in
 * AdamW::step_with_grads (src/optim.rs:214-251): w, m, v (n elements each, compact) are
 * read and rewritten, grad is read.  `step` is the 1-based step count AFTER the
 * increment at src/optim.rs:215; lr, betas, eps, weight_decay are the optimizer's f64
 * fields.  The arithmetic follows the reference's chain of tensor ops, rounding to the
 * tensor's type after each, so results are bit-identical to it for f32 and f16 alike
 * (for f16 that includes eps = 1e-8 rounding to zero).  grad_scale != 1 first scales
 * the gradient as clip_grad_norm would (src/optim.rs:288-293) without another pass
 * over memory; grad itself is not modified. */
int deers_rocm_adamw_step(int dtype, void* w, const void* grad, void* m, void* v, int64_t n,
                          double lr, double beta1, double beta2, double eps, double weight_decay,
                          int64_t step, double grad_scale);
/* The same update for n_tensors parameter tensors in as few launches as their number
 * allows (48 tensors per launch): w, grad, m, v are host arrays of device pointers, sizes
 * the element counts; every tensor gets exactly what deers_rocm_adamw_step would give it.
 * This is the whole parameter loop of AdamW::step_with_grads (src/optim.rs:221-247) for
 * the parameters that have a gradient. */
int deers_rocm_adamw_step_multi(int dtype, int n_tensors, void* const* w, const void* const* grad,
                                void* const* m, void* const* v, const int64_t* sizes, double lr,
                                double beta1, double beta2, double eps, double weight_decay,
                                int64_t step, double grad_scale);
/* *total = or += the sum of squares of all the tensors, the whole reduction loop of
 * clip_grad_norm (src/optim.rs:270-277) in one or two launches plus a fixed-order final
 * sum; tensors must be 16-byte aligned (DEERS_ROCM_ERR_LAYOUT otherwise).  Reproducible;
 * the order of additions differs from per-tensor deers_rocm_sum_squares calls. */
int deers_rocm_sum_squares_multi(int dtype, int n_tensors, const void* const* x, const int64_t* sizes,
                                 float* total, int accumulate);
/* *total (a float in device memory) = or += sum of x[i]^2 in f32, the reduction of
 * clip_grad_norm (src/optim.rs:270-277) for one gradient; the partition and the order
 * of additions are fixed, so repeated calls give the same bits. */
int deers_rocm_sum_squares(int dtype, const void* x, int64_t n, float* total, int accumulate);
/* x *= scale in place, scale cast as the reference's scalar ops cast it
 * (storage::ScalarMul, src/storage.rs:108-123): clip_grad_norm's rescaling. */
int deers_rocm_scale(int dtype, void* x, int64_t n, double scale);

/* dst viewed through dst_strides <- src viewed through src_strides, both of `shape`
 * (ndim in 1..6, non-negative strides).  The scatter counterpart of copy_compact;
 * used to append value rows to a KV cache.  The reference has no KV cache (it
 * re-runs the window per token, examples/tinystories_train.rs:250-276); the closest
 * reference routine is the strided copy of src/storage/cpu.rs:1063-1102. */
int deers_rocm_copy_view(int dtype, const void* src, const int64_t* src_strides,
                         void* dst, const int64_t* dst_strides,
                         const int64_t* shape, int ndim);

/* ---- batched matrix product ---------------------------------------------------
 * c[batch,m,n] (compact, row-major) = a[batch,m,k] @ b[batch,k,n].  Replaces
 * BackendStorage::matmul (src/storage.rs:270-279; CPU src/storage/cpu.rs:688-753,
 * CUDA src/storage/cuda.rs:1100-1125, which calls cuBLAS: this one calls rocBLAS, a
 * plain library GEMM, f16 with f32 accumulation or f32).  Operands are described by
 * element strides (row, column, batch) the way the CPU backend passes Layout strides
 * to gemm: transposed views cost nothing, a batch stride of 0 broadcasts (weights).
 * Each operand needs a unit row or column stride, otherwise DEERS_ROCM_ERR_LAYOUT
 * and the caller compacts (MatMul::new does that for the Metal backend,
 * src/ops.rs:1058-1062).  Used by the projections around the attention core
 * (src/models/gpt.rs:101-133, 146-147). */
int deers_rocm_matmul(int dtype,
                      const void* a, int64_t a_row_stride, int64_t a_col_stride, int64_t a_batch_stride,
                      const void* b, int64_t b_row_stride, int64_t b_col_stride, int64_t b_batch_stride,
                      void* c, int64_t batch, int64_t m, int64_t n, int64_t k);
/* c += a @ b, same operand rules; c holds the other addend on entry.  One launch for
 * the block's residual connections `x + attn(..)` and `x + mlp(..)`
 * (src/models/gpt.rs:237-239: a matmul followed by a binary add in the reference) and
 * for `GradientStore::accumulate` of a matmul's gradient (src/backprop.rs:101-112).  The
 * sum is formed in f32 inside the product's accumulator and rounded once, where the
 * reference rounds the product and then the sum (f16: at most one ulp apart). */
int deers_rocm_matmul_acc(int dtype,
                          const void* a, int64_t a_row_stride, int64_t a_col_stride, int64_t a_batch_stride,
                          const void* b, int64_t b_row_stride, int64_t b_col_stride, int64_t b_batch_stride,
                          void* c, int64_t batch, int64_t m, int64_t n, int64_t k);
/* c = a @ b + addend, addend compact like c (it may be c: then this is
 * deers_rocm_matmul_acc).  The out-of-place form serves an autograd graph, where the
 * addend (the residual stream, or a gradient another consumer also holds) must stay
 * as it is.  Same rounding as deers_rocm_matmul_acc. */
int deers_rocm_matmul_add(int dtype,
                          const void* a, int64_t a_row_stride, int64_t a_col_stride, int64_t a_batch_stride,
                          const void* b, int64_t b_row_stride, int64_t b_col_stride, int64_t b_batch_stride,
                          const void* addend, void* c, int64_t batch, int64_t m, int64_t n, int64_t k);
/* y[m,n] (+)= f(x)[m,k] @ w[k,n] for the few rows of a generation step (m <= 32), f16 only,
 * one streaming pass over w by a kernel of this library; x, w, y row-major with row strides
 * ldx, ldw and n.  `prologue` picks f:
 *   DEERS_ROCM_LINEAR_PLAIN     f(x) = x (what deers_rocm_matmul runs for such shapes anyway);
 *   DEERS_ROCM_LINEAR_RMS_NORM  f(x) = x * (mean(x^2 over the row) + eps)^-1/2, the weightless
 *                               RMSNorm in front of both branches of a block
 *                               (src/nn.rs:244-251, src/models/gpt.rs:240-247); the row factor
 *                               is applied to the f32 sums, so the normalised row is not
 *                               rounded to f16 in between as it is by deers_rocm_rms_norm_fwd
 *                               followed by deers_rocm_matmul;
 *   DEERS_ROCM_LINEAR_RELU_SQ   f(x) = relu(x)^2, the MLP's activation
 *                               (src/models/gpt.rs:196-203); same bits as
 *                               deers_rocm_relu_sq_fwd followed by deers_rocm_matmul.
 * w is row-major with row stride ldw, or, with ldw = DEERS_ROCM_LINEAR_W_PACKED, stored as
 * [ceil(n/32)][k][32]: element (kk, j) at ((j / 32) * k + kk) * 32 + j % 32, i.e. the 32
 * columns one workgroup reads are one contiguous run (deers_rocm_copy_view with shape
 * {n/32, k, 32}, source strides {32, n, 1} and destination strides {32k, 32, 1} packs a
 * row-major matrix).  Weights that are streamed from HBM every step are 2-3 us per product
 * faster that way.
 * accumulate != 0 adds into y (a residual stream updated in place).  Shapes it does not take
 * (n % 8, k % 256, unaligned rows, m > 32, another dtype) return DEERS_ROCM_ERR_ARG and
 * launch nothing: the caller then runs the separate entry points.  No counterpart in the
 * reference, whose sampling loop re-runs the whole window
 * (examples/tinystories_train.rs:250-276). */
#define DEERS_ROCM_LINEAR_PLAIN 0
#define DEERS_ROCM_LINEAR_RMS_NORM 1
#define DEERS_ROCM_LINEAR_RELU_SQ 2
#define DEERS_ROCM_LINEAR_W_PACKED (-32)
int deers_rocm_decode_linear(int dtype, int prologue, float eps, const void* x, int64_t ldx,
                             const void* w, int64_t ldw, void* y, int accumulate, int64_t m,
                             int64_t n, int64_t k);

/* Optional hint for the NEXT deers_rocm_decode_linear (or few-rows deers_rocm_matmul) launch:
 * the packed weight (DEERS_ROCM_LINEAR_W_PACKED layout, [ceil(n/32)][k][32] f16) of the product
 * that will follow it.  Workgroups on CUs that launch leaves idle read that weight once, each
 * tile through the L2 of the XCD that will consume it, so the following product finds its
 * weights in L2 instead of HBM.  One-shot: consumed (or dropped) by the next launch; NULL
 * clears it.  Purely a performance hint: results never depend on it, but the hinted buffer is
 * read by that launch, so it must stay allocated until the launch has run (threads that
 * share the library should pair hint and launch under their own lock).  No counterpart in the
 * reference. */
int deers_rocm_decode_linear_hint(const void* next_w_packed, int64_t n, int64_t k);

/* Off by default.  When on, the first matmul of each distinct problem (sizes, strides,
 * transposes, batch) times every kernel the BLAS offers for it on the caller's operands
 * and later calls of that problem use the fastest; the library's own pick is a heuristic
 * and loses up to 2x on tall-skinny products such as the LM head's weight gradient.
 * Costs seconds on the first training step; results are unchanged up to the summation
 * order inside the chosen kernel. */
int deers_rocm_matmul_tune(int on);

/* ---- rotary embedding fused with the head split / merge -----------------------
 * The neighbours of the attention core in CausalSelfAttention::forward
 * (src/models/gpt.rs:115-137): apply_rotary_emb on the [B,T,H,D] projections
 * (src/models/gpt.rs:49-73: narrow, 4 multiplies, 2 adds, cat) followed by
 * permute([0,2,1,3]).  cos and sin are the [1,T,1,D/2] tables of
 * precompute_rotary_embeddings (src/models/gpt.rs:12-47), compact, in the tensor's
 * dtype.  Any even D: rows that are whole aligned 16-byte chunks on both sides take the
 * vectorised kernel, everything else (the reference's GPT test runs head_dim 2,
 * tests/gpt.rs:38-49) one pair per thread; arithmetic is f32 with one rounding. */

/* y [B,H,T,D] = permute(apply_rotary_emb(x)), x logical [B,T,H,D] with element
 * strides x_strides = {b,t,h,d} (NULL = compact, d must be 1).  y is compact, or has
 * element strides y_strides = {b,h,t,d} (d must be 1): with T new positions and a
 * pointer to row `pos` of a [B,H,L_cap,D] KV cache the rotated keys are appended in
 * place (pass cos/sin advanced to row `pos` of the tables). */
int deers_rocm_rope_fwd(int dtype, const void* x, const int64_t* x_strides,
                        const void* cos, const void* sin, void* y, const int64_t* y_strides,
                        int64_t B, int64_t T, int64_t H, int64_t D);

/* One generation step's handling of the new token's q, k, v in one launch: q and k rotated
 * at the step's position (cos_row / sin_row: the D/2 table entries of that position), q to
 * compact q_out [B,H,D], the rotated k and the unrotated v to row `pos` of their caches.
 * q, k, v: [B,H,D] by element strides in_strides = {b, h} (D stride 1; e.g. the thirds of a
 * fused [B, 3C] projection row); caches [B,H,capacity,D] by cache_strides = {b, h, t}.
 * Replaces two deers_rocm_rope_fwd and one deers_rocm_copy_view per block and step.  The
 * reference has no KV cache (examples/tinystories_train.rs:250-276 re-runs the window);
 * the rotation is that of src/models/gpt.rs:49-73. */
int deers_rocm_decode_qkv(int dtype, const void* q, const void* k, const void* v,
                          const int64_t* in_strides, const void* cos_row, const void* sin_row,
                          void* q_out, void* k_cache, void* v_cache, const int64_t* cache_strides,
                          int64_t pos, int64_t capacity, int64_t B, int64_t H, int64_t D);

/* Backward of the above (Permute::backward then the element-wise backward bodies,
 * src/ops.rs:687-727, 130-260): dx (compact [B,T,H,D]) from dy logical [B,H,T,D]
 * with element strides dy_strides = {b,h,t,d} (NULL = compact, d must be 1). */
int deers_rocm_rope_bwd(int dtype, const void* dy, const int64_t* dy_strides,
                        const void* cos, const void* sin, void* dx,
                        int64_t B, int64_t T, int64_t H, int64_t D);

/* ---- testing only: nothing a binding exposes ---- */

/* Test hook for the bounded wait of the single-launch backward: `spin_limit` polls (the
 * default is 2^20) and, when `skip_producers` is non-zero, backward calls launch only the
 * waiting half of the grid, so that every wait runs out, every kernel still exits, and the
 * next deers_rocm_sync returns DEERS_ROCM_ERR_HANDOVER.  (spin_limit 2^20,
 * skip_producers 0) restores normal operation.  No counterpart in the reference. */
int deers_rocm_debug_bwd_wait(int spin_limit, int skip_producers);

#ifdef __cplusplus
}
#endif
#endif /* DEERS_ROCM_H */
