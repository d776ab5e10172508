// Host side of the C ABI declared in include/deers_rocm.h: the process-global
// runtime (device, stream, workspace), memory and timer calls, and the argument
// checks in front of every kernel launch.  The shape of the runtime follows what
// the reference's CUDA backend keeps in its OnceLock (one context, one stream,
// device ordinal fixed at init: src/storage/cuda.rs:462-528).
#define ROCBLAS_BETA_FEATURES_API 1  // solution enumeration for the GEMM tuner
#include <rocblas/rocblas.h>
#include "../../include/deers_rocm.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <unordered_map>
#include <mutex>
#include <string>
#include <vector>

#include "common.h"
#include "storage_ops.h"

namespace deers {
void launch_attn_fwd_f16(const FwdParams& p, int B, int D, hipStream_t stream);
void launch_attn_fwd_f32(const FwdParams& p, int B, int D, hipStream_t stream);
void launch_attn_bwd_f16(const BwdParams& p, int B, int D, int mode, hipStream_t stream);
void launch_attn_bwd_f32(const BwdParams& p, int B, int D, hipStream_t stream);
void launch_attn_decode_f16(const DecodeParams& p, int B, int D, bool append, hipStream_t stream);
int decode_pick_splits(int64_t BH, int64_t L, int* chunk);
void launch_fill(int dtype_f16, void* dst, size_t n, float value, hipStream_t stream);
void launch_add(int dtype_f16, const void* a, const void* b, void* out, size_t n,
                hipStream_t stream);
void launch_neg(int dtype_f16, const void* a, void* out, size_t n, hipStream_t stream);
void launch_copy_strided(int dtype_f16, const void* src, const int64_t* shape,
                         const int64_t* strides, int ndim, void* dst, hipStream_t stream);
bool skinny_gemm_takes(int64_t m, int64_t n, int64_t k, int64_t ldx, int64_t ldw, int64_t ldy,
                       const void* x, const void* w, const void* y);
int skinny_gemm_splits(int64_t n, int64_t k);
size_t skinny_gemm_workspace_bytes(int64_t n, int splits);
void launch_skinny_gemm_f16(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t ldy,
                            int m, int n, int k, bool accumulate, int prologue, float eps, bool packed,
                            int splits, float* partial, int* counters, const SkinnyPrefetch& next,
                            hipStream_t stream);
void launch_decode_qkv(int dtype_f16, const void* q, const void* k, const void* v,
                       const int64_t* in_strides, const void* cos_row, const void* sin_row, void* q_out,
                       void* k_cache, void* v_cache, const int64_t* cache_strides, int64_t pos, int B,
                       int H, int D, hipStream_t stream);
void launch_rope(int dtype_f16, bool inverse, bool vectorised, const void* src,
                 const int64_t* src_strides, const void* cos, const void* sin, void* dst,
                 const int64_t* dst_strides, int B, int T, int H, int D, hipStream_t stream);
void launch_log_softmax_fwd(int dtype_f16, const void* x, void* out, int64_t outer, int64_t inner,
                            hipStream_t stream);
void launch_log_softmax_bwd(int dtype_f16, const void* grad, const void* lsm, void* out,
                            int64_t outer, int64_t inner, hipStream_t stream);
void launch_index_select(int dtype_f16, const void* table, const int64_t* idx, void* out,
                         int64_t n_rows, int64_t n_idx, int width, int* flag, hipStream_t stream);
void launch_index_add(int dtype_f16, const void* src, const int64_t* idx, void* dst, int64_t n_rows,
                      int64_t n_idx, int width, int* flag, hipStream_t stream);
void launch_rms_norm(int dtype_f16, const void* x, const void* dy, const void* addend, void* out, int64_t outer,
                     int width, float eps, int bwd, hipStream_t stream);
void launch_relu_sq(int dtype_f16, const void* x, const void* dy, void* out, int64_t n, int bwd,
                    hipStream_t stream);
void launch_argmax_rows(int dtype_f16, const void* x, int64_t* out, int64_t outer, int width,
                        hipStream_t stream);
void launch_scale_by_device_scalar(int dtype_f16, void* x, int64_t n, const float* factor, hipStream_t stream);
void launch_cross_entropy_fwd(int dtype_f16, const void* logits, const int64_t* targets, float* row_lse,
                              float* row_loss, float* loss, void* dlogits, int64_t n_rows, int width,
                              int* flag, hipStream_t stream);
void launch_cross_entropy_bwd(int dtype_f16, const void* logits, const int64_t* targets,
                              const float* row_lse, const float* upstream, void* dlogits,
                              int64_t n_rows, int width, hipStream_t stream);
int sumsq_partial_count();
void launch_adamw(int dtype_f16, void* w, const void* g, void* m, void* v, int64_t n, double lr,
                  double beta1, double beta2, double eps, double weight_decay, int step,
                  double grad_scale, hipStream_t stream);
void launch_sumsq(int dtype_f16, const void* g, int64_t n, float* partial, float* out,
                  int accumulate, hipStream_t stream);
void launch_scale(int dtype_f16, void* x, int64_t n, double scale, hipStream_t stream);
int multi_max_tensors();
int64_t multi_blocks(int dtype_f16, int64_t n);
void launch_adamw_multi(int dtype_f16, int count, void* const* w, const void* const* g, void* const* m,
                        void* const* v, const int64_t* sizes, double lr, double beta1, double beta2,
                        double eps, double weight_decay, int step, double grad_scale,
                        hipStream_t stream);
int launch_sumsq_multi(int dtype_f16, int count, const void* const* x, const int64_t* sizes,
                       float* partial, hipStream_t stream);
void launch_sumsq_final(const float* partial, int n_partial, float* out, int accumulate,
                        hipStream_t stream);
void launch_copy_view(int dtype_f16, const void* src, const int64_t* src_strides, void* dst,
                      const int64_t* dst_strides, const int64_t* shape, int ndim,
                      hipStream_t stream);
}  // namespace deers

namespace {

struct Runtime {
  bool ready = false;
  int ordinal = -1;
  hipStream_t stream = nullptr;
  void* workspace = nullptr;  // grows on demand, freed never (process lifetime)
  size_t workspace_bytes = 0;
  rocblas_handle blas = nullptr;  // created by the first matmul, bound to `stream`
  // per (head, 128-row query block) publication flags of the single-launch f16
  // backward; a flag equals the current epoch once its rows are published
  int* bwd_ready = nullptr;  // allocation: [error word][flags ...]; kernels get the address of flags[0]
  size_t bwd_ready_len = 0;
  int bwd_epoch = 0;
  bool bwd_error_armed = false;  // a single-launch backward ran since the error word was last read
  // Hand-overs between workgroups inside one launch (the f16 backward's row statistics,
  // the few-rows GEMM's K splits) rely on producer and consumer sharing one XCD's L2,
  // which the kernels get from "workgroup id % 8 is the XCD".  True only on a device where
  // that is known to hold (see handover_policy); otherwise the library takes the forms
  // that need no such hand-over (two launches, unsplit K).
  bool same_xcd_handover = false;
  int handover_forced = -1;   // -1: by policy; 0 / 1: forced by deers_rocm_set_handover_mode
  // test hooks (deers_rocm_debug_bwd_wait): poll bound of the backward's flag wait, and
  // whether the next single-launch backward leaves out the workgroups that publish
  int bwd_spin_limit = 1 << 20;
  int bwd_skip_producers = 0;
  // sticky "an index was out of range" flag that index kernels raise; read back by the
  // next synchronising call after one of them has been launched
  int* index_flag = nullptr;
  bool index_flag_armed = false;
  deers::SkinnyPrefetch skinny_next;  // one-shot hint for the next few-rows product (decode_linear_hint)
  int* skinny_counters = nullptr;  // arrival counters of the few-rows GEMM's K splits (all zero between launches)
  // Block cache behind deers_rocm_alloc / _free.  Every kernel and copy of this library
  // runs on `stream`, in order, so a block handed back by free can be handed out again
  // without waiting for the device: whatever still reads it was enqueued earlier than
  // whatever will write it.  A training step allocates the same sizes every iteration;
  // going to hipMalloc / hipFree each time would serialise the host with the device.
  // GEMM tuner (off by default): the library's own choice of kernel for a problem is a
  // heuristic; with tuning on, the first call of each distinct problem times every
  // kernel the library offers for it and later calls use the fastest.
  bool tune_gemm = false;
  std::map<std::vector<int64_t>, int> gemm_choice;  // problem -> solution index (0 = library default)
  std::unordered_map<size_t, std::vector<void*>> free_blocks;  // by rounded size
  std::unordered_map<void*, size_t> block_size;                // every block handed out
  size_t cached_bytes = 0;
};

Runtime g_rt;
std::mutex g_mu;

// Device memory that exists without any allocation call: the split partials of
// deers_rocm_attn_decode_noalloc live here.  Each GPU the library is loaded on holds its
// own copy until the process ends.  The name below is only a host-side handle: host code
// uses the address hipGetSymbolAddress returns for the current device (g_scratch_ptr,
// resolved once in deers_rocm_init), never the name itself.
constexpr size_t kScratchBytes = 512 * 1024;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
void* g_scratch_ptr = nullptr;  // device address of `scratch` on g_rt.ordinal
thread_local std::string t_err;

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  t_err = buf;
  return code;
}

#define HIP_TRY(expr)                                                                   \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess)                                                               \
      return fail(DEERS_ROCM_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));   \
  } while (0)

#define NEED_INIT()                                                                     \
  do {                                                                                  \
    if (!g_rt.ready)                                                                    \
      return fail(DEERS_ROCM_ERR_NOT_INIT, "deers_rocm_init has not been called");      \
  } while (0)

// The XCD-local hand-overs are taken only on an unpartitioned MI355X with every CU
// enabled: 256 CUs = 8 XCDs x 32, where the dispatcher deals workgroups round-robin to the
// XCDs.  A compute partition (fewer CUs per device) or a CU mask changes which XCD a
// workgroup id lands on.
int handover_policy(int cu_count, int cu_mask_set) {
  return (cu_count == 256 && !cu_mask_set) ? DEERS_ROCM_HANDOVER_SAME_XCD
                                           : DEERS_ROCM_HANDOVER_STREAM_ORDER;
}

bool cu_mask_in_environment() {
  for (const char* name : {"ROC_GLOBAL_CU_MASK", "HSA_CU_MASK", "HSA_CU_MASK_SKIP_INIT"}) {
    const char* v = getenv(name);
    if (v && *v) return true;
  }
  return false;
}

bool device_is_gfx950(int ordinal) {
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, ordinal) != hipSuccess) return false;
  return std::string(prop.gcnArchName).rfind("gfx950", 0) == 0;
}

// Workspace that only grows; callers hold g_mu.
int workspace(size_t bytes, void** out) {
  if (bytes > g_rt.workspace_bytes) {
    if (g_rt.workspace) {
      HIP_TRY(hipStreamSynchronize(g_rt.stream));
      HIP_TRY(hipFree(g_rt.workspace));
      g_rt.workspace = nullptr;
      g_rt.workspace_bytes = 0;
    }
    const size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
    HIP_TRY(hipMalloc(&g_rt.workspace, want));
    g_rt.workspace_bytes = want;
  }
  *out = g_rt.workspace;
  return DEERS_ROCM_OK;
}

// Resolves a [B,H,T,D] stride argument (NULL = compact) and checks what the
// kernels assume: unit D stride and 16-byte aligned rows.
int resolve_strides(const char* name, const void* ptr, const int64_t* strides, int64_t H,
                    int64_t T, int64_t D, size_t elem, deers::Strides3* out) {
  if (!ptr) return fail(DEERS_ROCM_ERR_ARG, "%s: null pointer", name);
  int64_t sb = H * T * D, sh = T * D, st = D, sd = 1;
  if (strides) {
    sb = strides[0];
    sh = strides[1];
    st = strides[2];
    sd = strides[3];
  }
  if (sd != 1)
    return fail(DEERS_ROCM_ERR_LAYOUT,
                "%s: innermost stride is %lld, the kernels need 1 (compact the tensor first)",
                name, (long long)sd);
  const int64_t per16 = 16 / (int64_t)elem;
  if (sb % per16 || sh % per16 || st % per16 || (reinterpret_cast<uintptr_t>(ptr) & 15))
    return fail(DEERS_ROCM_ERR_LAYOUT,
                "%s: rows must be 16-byte aligned (ptr %p, strides %lld,%lld,%lld)", name, ptr,
                (long long)sb, (long long)sh, (long long)st);
  if (sb < 0 || sh < 0 || st < D || T * st >= (int64_t(1) << 30))
    return fail(DEERS_ROCM_ERR_LAYOUT,
                "%s: strides must be non-negative, rows must not overlap and T * row stride "
                "must stay below 2^30 elements (strides %lld,%lld,%lld)",
                name, (long long)sb, (long long)sh, (long long)st);
  out->b = sb;
  out->h = sh;
  out->t = st;
  return DEERS_ROCM_OK;
}

int check_problem(int dtype, int64_t B, int64_t H, int64_t T, int64_t D) {
  if (dtype != DEERS_ROCM_F16 && dtype != DEERS_ROCM_F32)
    return fail(DEERS_ROCM_ERR_ARG, "dtype %d is neither DEERS_ROCM_F16 nor DEERS_ROCM_F32", dtype);
  if (B < 1 || H < 1 || T < 1)
    return fail(DEERS_ROCM_ERR_ARG, "B, H, T must be >= 1 (got %lld, %lld, %lld)", (long long)B,
                (long long)H, (long long)T);
  if (D != 32 && D != 64 && D != 128)
    return fail(DEERS_ROCM_ERR_ARG, "head dim %lld unsupported (32, 64 or 128)", (long long)D);
  if (B * H > 65535 || T > (int64_t(1) << 24))
    return fail(DEERS_ROCM_ERR_ARG, "B*H must be <= 65535 and T <= 2^24");
  return DEERS_ROCM_OK;
}

// The kernels track the running maximum on raw scores and apply the scale inside
// the exponent, which needs scale > 0 (the reference uses 1/sqrt(D)).
int check_scale(float scale) {
  if (!(scale > 0.f) || !std::isfinite(scale))
    return fail(DEERS_ROCM_ERR_ARG, "scale must be positive and finite (got %g)", (double)scale);
  return DEERS_ROCM_OK;
}

struct Timer {
  hipEvent_t start, stop;
};

// Per-kernel profiling records (guarded by g_mu: launches happen under it).
struct LaunchRecord {
  const char* name;
  hipEvent_t start, stop;
};
bool g_prof_on = false;
std::vector<LaunchRecord*> g_prof_records;
struct ProfRow {
  std::string name;
  int64_t calls;
  float total_ms;
};
std::vector<ProfRow> g_prof_rows;

void prof_clear() {
  for (LaunchRecord* r : g_prof_records) {
    (void)hipEventDestroy(r->start);
    (void)hipEventDestroy(r->stop);
    delete r;
  }
  g_prof_records.clear();
  g_prof_rows.clear();
}

}  // namespace

namespace deers {

LaunchScope::LaunchScope(const char* name, hipStream_t stream) : rec_(nullptr), stream_(stream) {
  if (!g_prof_on) return;
  LaunchRecord* r = new LaunchRecord{name, nullptr, nullptr};
  if (hipEventCreate(&r->start) != hipSuccess || hipEventCreate(&r->stop) != hipSuccess ||
      hipEventRecord(r->start, stream) != hipSuccess) {
    delete r;
    return;
  }
  rec_ = r;
}

LaunchScope::~LaunchScope() {
  if (!rec_) return;
  LaunchRecord* r = static_cast<LaunchRecord*>(rec_);
  (void)hipEventRecord(r->stop, stream_);
  g_prof_records.push_back(r);
}

}  // namespace deers

extern "C" {

int deers_rocm_available(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_rt.ready) return 1;
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n < 1) return 0;
  return device_is_gfx950(0) ? 1 : 0;
}

int deers_rocm_init(int ordinal) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (g_rt.ready) {
    if (g_rt.ordinal == ordinal) return DEERS_ROCM_OK;
    return fail(DEERS_ROCM_ERR_ARG, "runtime already initialised on device %d", g_rt.ordinal);
  }
  int n = 0;
  HIP_TRY(hipGetDeviceCount(&n));
  if (ordinal < 0 || ordinal >= n)
    return fail(DEERS_ROCM_ERR_ARG, "device ordinal %d out of range (%d devices)", ordinal, n);
  if (!device_is_gfx950(ordinal))
    return fail(DEERS_ROCM_ERR_ARG, "device %d is not gfx950; this library targets MI355X only",
                ordinal);
  HIP_TRY(hipSetDevice(ordinal));
  HIP_TRY(hipStreamCreateWithFlags(&g_rt.stream, hipStreamNonBlocking));
  HIP_TRY(hipGetSymbolAddress(&g_scratch_ptr, HIP_SYMBOL(scratch)));
  {
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, ordinal));
    g_rt.same_xcd_handover =
        handover_policy(prop.multiProcessorCount, cu_mask_in_environment() ? 1 : 0) ==
        DEERS_ROCM_HANDOVER_SAME_XCD;
  }
  g_rt.ordinal = ordinal;
  g_rt.ready = true;
  return DEERS_ROCM_OK;
}

// Device memory for the index flag, created by the first call that needs it.
int index_flag(int** out) {
  if (!g_rt.index_flag) {
    HIP_TRY(hipMalloc((void**)&g_rt.index_flag, sizeof(int)));
    HIP_TRY(hipMemsetAsync(g_rt.index_flag, 0, sizeof(int), g_rt.stream));
  }
  g_rt.index_flag_armed = true;
  *out = g_rt.index_flag;
  return DEERS_ROCM_OK;
}

// After the stream has drained: reports (once) an out-of-range index seen by any index
// kernel since the last check.  Kernels skip such an index, they never follow it.
int check_index_flag() {
  if (!g_rt.index_flag_armed) return DEERS_ROCM_OK;
  g_rt.index_flag_armed = false;
  int seen = 0;
  HIP_TRY(hipMemcpyAsync(&seen, g_rt.index_flag, sizeof(int), hipMemcpyDeviceToHost, g_rt.stream));
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  if (!seen) return DEERS_ROCM_OK;
  // on the library stream, so that the reset is ordered with the kernels that raise the flag
  HIP_TRY(hipMemsetAsync(g_rt.index_flag, 0, sizeof(int), g_rt.stream));
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  return fail(DEERS_ROCM_ERR_INDEX,
              "an index was out of bounds in an index_select / index_add / cross_entropy call "
              "since the last synchronisation (such rows were skipped)");
}

// After the stream has drained: reports (once) that a dK/dV workgroup of a single-launch
// backward gave up waiting for its row statistics since the last check.
int check_handover_error() {
  if (!g_rt.bwd_error_armed || !g_rt.bwd_ready) return DEERS_ROCM_OK;
  g_rt.bwd_error_armed = false;
  int seen = 0;
  HIP_TRY(hipMemcpyAsync(&seen, g_rt.bwd_ready, sizeof(int), hipMemcpyDeviceToHost, g_rt.stream));
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  if (!seen) return DEERS_ROCM_OK;
  HIP_TRY(hipMemsetAsync(g_rt.bwd_ready, 0, sizeof(int), g_rt.stream));
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  return fail(DEERS_ROCM_ERR_HANDOVER,
              "attn_bwd: a workgroup gave up waiting for another workgroup's row statistics "
              "in a backward pass since the last synchronisation; dK and dV of that call are "
              "not valid (deers_rocm_set_handover_mode(DEERS_ROCM_HANDOVER_STREAM_ORDER) "
              "selects the form without this wait)");
}

int check_device_flags() {
  if (int rc = check_index_flag()) return rc;
  return check_handover_error();
}

int deers_rocm_sync(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  return check_device_flags();
}

int deers_rocm_handover_policy(int cu_count, int cu_mask_set) {
  return handover_policy(cu_count, cu_mask_set);
}

static bool same_xcd_handover_now() {
  return g_rt.handover_forced >= 0 ? g_rt.handover_forced == DEERS_ROCM_HANDOVER_SAME_XCD
                                   : g_rt.same_xcd_handover;
}

int deers_rocm_handover_mode(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!g_rt.ready) return -1;
  return same_xcd_handover_now() ? DEERS_ROCM_HANDOVER_SAME_XCD : DEERS_ROCM_HANDOVER_STREAM_ORDER;
}

int deers_rocm_set_handover_mode(int mode) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (mode != -1 && mode != DEERS_ROCM_HANDOVER_SAME_XCD && mode != DEERS_ROCM_HANDOVER_STREAM_ORDER)
    return fail(DEERS_ROCM_ERR_ARG, "set_handover_mode: mode %d is not -1, 0 or 1", mode);
  if (mode == DEERS_ROCM_HANDOVER_SAME_XCD && !g_rt.same_xcd_handover)
    return fail(DEERS_ROCM_ERR_ARG,
                "set_handover_mode: this device's policy is stream order (partition or CU mask): a hand-over "
                "through one XCD's L2 is not valid here");
  g_rt.handover_forced = mode;
  return DEERS_ROCM_OK;
}

int deers_rocm_debug_bwd_wait(int spin_limit, int skip_producers) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (spin_limit < 1) return fail(DEERS_ROCM_ERR_ARG, "debug_bwd_wait: spin_limit must be >= 1");
  g_rt.bwd_spin_limit = spin_limit;
  g_rt.bwd_skip_producers = skip_producers ? 1 : 0;
  return DEERS_ROCM_OK;
}

const char* deers_rocm_last_error(void) { return t_err.c_str(); }

void* deers_rocm_stream(void) { return g_rt.ready ? (void*)g_rt.stream : nullptr; }

// Returns every cached block to the driver (after the stream has drained).
static int release_cached_blocks() {
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  for (auto& kv : g_rt.free_blocks)
    for (void* p : kv.second) HIP_TRY(hipFree(p));
  g_rt.free_blocks.clear();
  g_rt.cached_bytes = 0;
  return DEERS_ROCM_OK;
}

int deers_rocm_empty_cache(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  return release_cached_blocks();
}

int deers_rocm_alloc(size_t bytes, void** out_ptr) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!out_ptr) return fail(DEERS_ROCM_ERR_ARG, "alloc: null out_ptr");
  *out_ptr = nullptr;
  if (bytes == 0) return DEERS_ROCM_OK;
  const size_t size = (bytes + 255) & ~(size_t)255;
  auto hit = g_rt.free_blocks.find(size);
  if (hit != g_rt.free_blocks.end() && !hit->second.empty()) {
    *out_ptr = hit->second.back();
    hit->second.pop_back();
    g_rt.cached_bytes -= size;
    g_rt.block_size[*out_ptr] = size;
    return DEERS_ROCM_OK;
  }
  HIP_TRY(hipSetDevice(g_rt.ordinal));
  hipError_t e = hipMalloc(out_ptr, size);
  if (e == hipErrorOutOfMemory) {
    (void)hipGetLastError();
    if (int rc = release_cached_blocks()) return rc;
    e = hipMalloc(out_ptr, size);
  }
  HIP_TRY(e);
  g_rt.block_size[*out_ptr] = size;
  return DEERS_ROCM_OK;
}

int deers_rocm_alloc_zeros(size_t bytes, void** out_ptr) {
  int rc = deers_rocm_alloc(bytes, out_ptr);
  if (rc != DEERS_ROCM_OK || bytes == 0) return rc;
  std::lock_guard<std::mutex> lock(g_mu);
  HIP_TRY(hipMemsetAsync(*out_ptr, 0, bytes, g_rt.stream));
  return DEERS_ROCM_OK;
}

int deers_rocm_free(void* ptr) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!ptr) return DEERS_ROCM_OK;
  auto it = g_rt.block_size.find(ptr);
  if (it == g_rt.block_size.end())
    return fail(DEERS_ROCM_ERR_ARG, "free: %p was not allocated by deers_rocm_alloc (or freed twice)", ptr);
  // Work already enqueued may still read the buffer: it stays allocated and goes back
  // to the cache, to be reused by later work on the same stream.
  const size_t size = it->second;
  g_rt.block_size.erase(it);
  g_rt.free_blocks[size].push_back(ptr);
  g_rt.cached_bytes += size;
  return DEERS_ROCM_OK;
}

int deers_rocm_htod(void* dst_device, const void* src_host, size_t bytes) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (bytes == 0) return DEERS_ROCM_OK;
  if (!dst_device || !src_host) return fail(DEERS_ROCM_ERR_ARG, "htod: null pointer");
  HIP_TRY(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, g_rt.stream));
  HIP_TRY(hipStreamSynchronize(g_rt.stream));  // pageable source: safe to reuse on return
  return DEERS_ROCM_OK;
}

int deers_rocm_dtoh(void* dst_host, const void* src_device, size_t bytes) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (bytes == 0) return DEERS_ROCM_OK;
  if (!dst_host || !src_device) return fail(DEERS_ROCM_ERR_ARG, "dtoh: null pointer");
  HIP_TRY(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, g_rt.stream));
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  return check_device_flags();
}

int deers_rocm_dtod(void* dst_device, const void* src_device, size_t bytes) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (bytes == 0) return DEERS_ROCM_OK;
  if (!dst_device || !src_device) return fail(DEERS_ROCM_ERR_ARG, "dtod: null pointer");
  HIP_TRY(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, g_rt.stream));
  return DEERS_ROCM_OK;
}

int deers_rocm_timer_create(void** out_timer) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!out_timer) return fail(DEERS_ROCM_ERR_ARG, "timer_create: null out_timer");
  Timer* t = new Timer;
  hipError_t e = hipEventCreate(&t->start);
  if (e == hipSuccess) e = hipEventCreate(&t->stop);
  if (e != hipSuccess) {
    delete t;
    return fail(DEERS_ROCM_ERR_HIP, "hipEventCreate failed: %s", hipGetErrorString(e));
  }
  *out_timer = t;
  return DEERS_ROCM_OK;
}

int deers_rocm_timer_start(void* timer) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!timer) return fail(DEERS_ROCM_ERR_ARG, "timer_start: null timer");
  HIP_TRY(hipEventRecord(static_cast<Timer*>(timer)->start, g_rt.stream));
  return DEERS_ROCM_OK;
}

int deers_rocm_timer_stop(void* timer) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!timer) return fail(DEERS_ROCM_ERR_ARG, "timer_stop: null timer");
  HIP_TRY(hipEventRecord(static_cast<Timer*>(timer)->stop, g_rt.stream));
  return DEERS_ROCM_OK;
}

int deers_rocm_timer_elapsed_ms(void* timer, float* out_ms) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!timer || !out_ms) return fail(DEERS_ROCM_ERR_ARG, "timer_elapsed_ms: null argument");
  Timer* t = static_cast<Timer*>(timer);
  HIP_TRY(hipEventSynchronize(t->stop));
  HIP_TRY(hipEventElapsedTime(out_ms, t->start, t->stop));
  return DEERS_ROCM_OK;
}

int deers_rocm_timer_destroy(void* timer) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!timer) return DEERS_ROCM_OK;
  Timer* t = static_cast<Timer*>(timer);
  (void)hipEventDestroy(t->start);
  (void)hipEventDestroy(t->stop);
  delete t;
  return DEERS_ROCM_OK;
}

int deers_rocm_profile_enable(int on) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  if (on) prof_clear();
  g_prof_on = on != 0;
  return DEERS_ROCM_OK;
}

int deers_rocm_profile_collect(int* out_rows) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (!out_rows) return fail(DEERS_ROCM_ERR_ARG, "profile_collect: null out_rows");
  HIP_TRY(hipStreamSynchronize(g_rt.stream));
  std::map<std::string, ProfRow> agg;
  for (LaunchRecord* r : g_prof_records) {
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, r->start, r->stop));
    ProfRow& row = agg[r->name];
    row.name = r->name;
    row.calls += 1;
    row.total_ms += ms;
  }
  g_prof_rows.clear();
  for (auto& kv : agg) g_prof_rows.push_back(kv.second);
  *out_rows = (int)g_prof_rows.size();
  return DEERS_ROCM_OK;
}

int deers_rocm_profile_row(int index, const char** out_name, int64_t* out_calls,
                           float* out_total_ms) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (index < 0 || index >= (int)g_prof_rows.size() || !out_name || !out_calls || !out_total_ms)
    return fail(DEERS_ROCM_ERR_ARG, "profile_row: bad index or null argument");
  *out_name = g_prof_rows[index].name.c_str();
  *out_calls = g_prof_rows[index].calls;
  *out_total_ms = g_prof_rows[index].total_ms;
  return DEERS_ROCM_OK;
}

int deers_rocm_attn_fwd(int dtype, const void* q, const int64_t* q_strides, const void* k,
                        const int64_t* k_strides, const void* v, const int64_t* v_strides,
                        void* o, const int64_t* o_strides, float* lse, int64_t B, int64_t H,
                        int64_t T, int64_t D, float scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_problem(dtype, B, H, T, D)) return rc;
  if (int rc = check_scale(scale)) return rc;
  if (!lse) return fail(DEERS_ROCM_ERR_ARG, "attn_fwd: null lse");
  const size_t elem = dtype == DEERS_ROCM_F16 ? 2 : 4;
  deers::FwdParams p{};
  if (int rc = resolve_strides("q", q, q_strides, H, T, D, elem, &p.sq)) return rc;
  if (int rc = resolve_strides("k", k, k_strides, H, T, D, elem, &p.sk)) return rc;
  if (int rc = resolve_strides("v", v, v_strides, H, T, D, elem, &p.sv)) return rc;
  if (int rc = resolve_strides("o", o, o_strides, H, T, D, elem, &p.so)) return rc;
  p.q = q; p.k = k; p.v = v; p.o = o; p.lse = lse;
  p.H = (int)H; p.T = (int)T;
  p.scale_log2 = (float)((double)scale * 1.4426950408889634);
  if (dtype == DEERS_ROCM_F16)
    deers::launch_attn_fwd_f16(p, (int)B, (int)D, g_rt.stream);
  else
    deers::launch_attn_fwd_f32(p, (int)B, (int)D, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_attn_bwd(int dtype, const void* q, const int64_t* q_strides, const void* k,
                        const int64_t* k_strides, const void* v, const int64_t* v_strides,
                        const void* o, const int64_t* o_strides, const float* lse,
                        const void* d_o, const int64_t* do_strides, void* dq,
                        const int64_t* dq_strides, void* dk, const int64_t* dk_strides, void* dv,
                        const int64_t* dv_strides, int64_t B, int64_t H, int64_t T, int64_t D,
                        float scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_problem(dtype, B, H, T, D)) return rc;
  if (int rc = check_scale(scale)) return rc;
  if (!lse) return fail(DEERS_ROCM_ERR_ARG, "attn_bwd: null lse");
  const size_t elem = dtype == DEERS_ROCM_F16 ? 2 : 4;
  deers::BwdParams p{};
  if (int rc = resolve_strides("q", q, q_strides, H, T, D, elem, &p.sq)) return rc;
  if (int rc = resolve_strides("k", k, k_strides, H, T, D, elem, &p.sk)) return rc;
  if (int rc = resolve_strides("v", v, v_strides, H, T, D, elem, &p.sv)) return rc;
  if (int rc = resolve_strides("o", o, o_strides, H, T, D, elem, &p.so)) return rc;
  if (int rc = resolve_strides("d_o", d_o, do_strides, H, T, D, elem, &p.sdo)) return rc;
  if (int rc = resolve_strides("dq", dq, dq_strides, H, T, D, elem, &p.sdq)) return rc;
  if (int rc = resolve_strides("dk", dk, dk_strides, H, T, D, elem, &p.sdk)) return rc;
  if (int rc = resolve_strides("dv", dv, dv_strides, H, T, D, elem, &p.sdv)) return rc;
  // f32: delta[B,H,T].  f16: lse2 and negdelta, rows padded to a multiple of 64 per head.
  const int64_t t_pad = (T + 63) / 64 * 64;
  // f16: + 64 floats, the block-pipelined dK/dV role loads row vectors 64 floats at a time
  const size_t ws_floats = dtype == DEERS_ROCM_F16 ? (size_t)(2 * B * H * t_pad + 64) : (size_t)(B * H * T);
  void* ws = nullptr;
  // f16: behind them the dQ role's scaled queries, [B*H][t_pad][D] f16
  const size_t ws_qs = dtype == DEERS_ROCM_F16 ? (size_t)(B * H * t_pad * D) * 2 : 0;
  if (int rc = workspace(ws_floats * sizeof(float) + ws_qs, &ws)) return rc;
  p.q = q; p.k = k; p.v = v; p.o = o; p.d_o = d_o; p.lse = lse;
  p.delta = static_cast<float*>(ws);
  // A launch that is being captured into a graph gets no fresh epoch on replay: it takes the
  // two-launch form with the flags switched off (epoch 0).  The workspace and the flags must
  // have been grown by an earlier, eager call of the same geometry: capture allows neither
  // the synchronisation nor the allocation.
  bool capturing = false;
  if (dtype == DEERS_ROCM_F16) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    HIP_TRY(hipStreamIsCapturing(g_rt.stream, &cs));
    capturing = cs != hipStreamCaptureStatusNone;
    const size_t n_flags = (size_t)(B * H) * (size_t)((T + 127) / 128);
    if (n_flags > g_rt.bwd_ready_len || g_rt.bwd_epoch == INT32_MAX) {
      if (capturing)
        return fail(DEERS_ROCM_ERR_ARG,
                    "attn_bwd: call once outside stream capture with this geometry first (the "
                    "hand-over flags have to grow)");
      if (g_rt.bwd_ready) {
        HIP_TRY(hipStreamSynchronize(g_rt.stream));
        // an error raised by a launch before this point is reported by this call
        if (int rc = check_handover_error()) return rc;
        HIP_TRY(hipFree(g_rt.bwd_ready));
        g_rt.bwd_ready = nullptr;
      }
      const size_t want = n_flags > g_rt.bwd_ready_len ? n_flags : g_rt.bwd_ready_len;
      HIP_TRY(hipMalloc(&g_rt.bwd_ready, (want + 1) * sizeof(int)));  // [error word][flags]
      HIP_TRY(hipMemsetAsync(g_rt.bwd_ready, 0, (want + 1) * sizeof(int), g_rt.stream));
      g_rt.bwd_ready_len = want;
      g_rt.bwd_epoch = 0;
    }
    p.error = g_rt.bwd_ready;
    p.ready = g_rt.bwd_ready + 1;
    p.epoch = capturing ? 0 : ++g_rt.bwd_epoch;
    p.spin_limit = g_rt.bwd_spin_limit;
  }
  const bool single_launch = !capturing && same_xcd_handover_now();
  p.lse2 = static_cast<float*>(ws);
  p.negdelta = static_cast<float*>(ws) + B * H * t_pad;
  p.qs = static_cast<float*>(ws) + ws_floats;
  p.t_pad = (int)t_pad;
  p.dq = dq; p.dk = dk; p.dv = dv;
  p.H = (int)H; p.T = (int)T;
  p.scale = scale;
  p.scale_log2 = (float)((double)scale * 1.4426950408889634);
  if (dtype == DEERS_ROCM_F16) {
    if (single_launch) g_rt.bwd_error_armed = true;
    const int mode = !single_launch ? 0 : (g_rt.bwd_skip_producers ? 2 : 1);
    deers::launch_attn_bwd_f16(p, (int)B, (int)D, mode, g_rt.stream);
  } else {
    deers::launch_attn_bwd_f32(p, (int)B, (int)D, g_rt.stream);
  }
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// Argument checks and launch shared by deers_rocm_attn_decode (partials in the growing
// workspace) and deers_rocm_attn_decode_noalloc (partials in the static scratch array).
static int attn_decode_impl(const char* what, bool no_alloc, int dtype, const void* q,
                            const void* k_cache, const void* v_cache, const int64_t* kv_strides,
                            void* o, int64_t B, int64_t H, int64_t L, int64_t D, float scale) {
  NEED_INIT();
  if (dtype != DEERS_ROCM_F16)
    return fail(DEERS_ROCM_ERR_ARG, "%s: only DEERS_ROCM_F16 caches are supported", what);
  if (B < 1 || H < 1 || L < 1 || B * H > 65535 || L > (int64_t(1) << 30))
    return fail(DEERS_ROCM_ERR_ARG, "%s: need B,H,L >= 1, B*H <= 65535, L <= 2^30", what);
  if (D != 32 && D != 64 && D != 128)
    return fail(DEERS_ROCM_ERR_ARG, "%s: head dim %lld unsupported (32, 64 or 128)", what,
                (long long)D);
  if (!q || !k_cache || !v_cache || !o) return fail(DEERS_ROCM_ERR_ARG, "%s: null pointer", what);
  if (int rc = check_scale(scale)) return rc;
  deers::DecodeParams p{};
  p.skb = H * L * D; p.skh = L * D; p.skl = D;
  if (kv_strides) { p.skb = kv_strides[0]; p.skh = kv_strides[1]; p.skl = kv_strides[2]; }
  if (p.skb % 8 || p.skh % 8 || p.skl % 8 || (reinterpret_cast<uintptr_t>(k_cache) & 15) ||
      (reinterpret_cast<uintptr_t>(v_cache) & 15) || (reinterpret_cast<uintptr_t>(q) & 15) ||
      (reinterpret_cast<uintptr_t>(o) & 15))
    return fail(DEERS_ROCM_ERR_LAYOUT, "%s: cache rows, q and o must be 16-byte aligned", what);
  int chunk = 0;
  const int splits = deers::decode_pick_splits(B * H, L, &chunk);
  void* ws = nullptr;
  const size_t part_o = (size_t)(B * H) * splits * D * sizeof(float);
  const size_t part_ml = (size_t)(B * H) * splits * 2 * sizeof(float);
  if (no_alloc) {
    // a head that is not split writes its output itself and touches no scratch
    if (splits > 1 && part_o + part_ml > kScratchBytes)
      return fail(DEERS_ROCM_ERR_ARG,
                  "%s: the split partials of this problem need %zu bytes, the static scratch "
                  "holds %zu; use deers_rocm_attn_decode",
                  what, part_o + part_ml, kScratchBytes);
    ws = g_scratch_ptr;
  } else {
    if (int rc = workspace(part_o + part_ml, &ws)) return rc;
  }
  p.q = q; p.k = k_cache; p.v = v_cache; p.o = o;
  p.part_o = static_cast<float*>(ws);
  p.part_ml = reinterpret_cast<float*>(static_cast<char*>(ws) + part_o);
  p.H = (int)H; p.L = (int)L; p.splits = splits; p.chunk = chunk;
  p.scale_log2 = (float)((double)scale * 1.4426950408889634);
  deers::launch_attn_decode_f16(p, (int)B, (int)D, false, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_attn_decode(int dtype, const void* q, const void* k_cache, const void* v_cache,
                           const int64_t* kv_strides, void* o, int64_t B, int64_t H, int64_t L,
                           int64_t D, float scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  return attn_decode_impl("attn_decode", false, dtype, q, k_cache, v_cache, kv_strides, o, B, H, L,
                          D, scale);
}

// The same kernels with the split partials in the file-scope `scratch` array: no
// hipMalloc / hipFree on any path.  Every split slot that the merge kernel reads is
// written by the main kernel of the same call first, so nothing needs clearing.
int deers_rocm_attn_decode_noalloc(int dtype, const void* q, const void* k_cache,
                                   const void* v_cache, const int64_t* kv_strides, void* o,
                                   int64_t B, int64_t H, int64_t L, int64_t D, float scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  return attn_decode_impl("attn_decode_noalloc", true, dtype, q, k_cache, v_cache, kv_strides, o,
                          B, H, L, D, scale);
}

int deers_rocm_attn_decode_append(int dtype, const void* q, const void* k, const void* v,
                                  const int64_t* in_strides, const void* cos_row, const void* sin_row,
                                  void* k_cache, void* v_cache, const int64_t* cache_strides, void* o,
                                  int64_t pos, int64_t capacity, int64_t B, int64_t H, int64_t D,
                                  float scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (dtype != DEERS_ROCM_F16)
    return fail(DEERS_ROCM_ERR_ARG, "attn_decode_append: only DEERS_ROCM_F16 caches are supported");
  if (B < 1 || H < 1 || B * H > 65535 || capacity > (int64_t(1) << 30))
    return fail(DEERS_ROCM_ERR_ARG, "attn_decode_append: need B,H >= 1, B*H <= 65535, capacity <= 2^30");
  if (pos < 0 || pos >= capacity)
    return fail(DEERS_ROCM_ERR_ARG, "attn_decode_append: position %lld outside the cache capacity %lld",
                (long long)pos, (long long)capacity);
  if (D != 32 && D != 64 && D != 128)
    return fail(DEERS_ROCM_ERR_ARG, "attn_decode_append: head dim %lld unsupported (32, 64 or 128)", (long long)D);
  if (!q || !k || !v || !in_strides || !cos_row || !sin_row || !k_cache || !v_cache || !cache_strides || !o)
    return fail(DEERS_ROCM_ERR_ARG, "attn_decode_append: null pointer");
  if (int rc = check_scale(scale)) return rc;
  for (int d = 0; d < 2; ++d)
    if (in_strides[d] < 0 || in_strides[d] % 8)
      return fail(DEERS_ROCM_ERR_LAYOUT, "attn_decode_append: input strides must be non-negative multiples of 16 bytes");
  for (int d = 0; d < 3; ++d)
    if (cache_strides[d] < 0 || cache_strides[d] % 8)
      return fail(DEERS_ROCM_ERR_LAYOUT, "attn_decode_append: cache strides must be non-negative multiples of 16 bytes");
  const void* ptrs[8] = {q, k, v, cos_row, sin_row, k_cache, v_cache, o};
  for (const void* ptr : ptrs)
    if ((uintptr_t)ptr & 15) return fail(DEERS_ROCM_ERR_LAYOUT, "attn_decode_append: pointers must be 16-byte aligned");
  deers::DecodeParams p{};
  p.skb = cache_strides[0]; p.skh = cache_strides[1]; p.skl = cache_strides[2];
  int chunk = 0;
  const int splits = deers::decode_pick_splits(B * H, pos, &chunk);  // over the rows already cached
  void* ws = nullptr;
  const size_t part_o = (size_t)(B * H) * splits * D * sizeof(float);
  const size_t part_ml = (size_t)(B * H) * splits * 2 * sizeof(float);
  if (int rc = workspace(part_o + part_ml, &ws)) return rc;
  p.k = k_cache; p.v = v_cache; p.o = o;
  p.q_in = q; p.k_in = k; p.v_in = v; p.cos_row = cos_row; p.sin_row = sin_row;
  p.in_b = in_strides[0]; p.in_h = in_strides[1];
  p.part_o = static_cast<float*>(ws);
  p.part_ml = reinterpret_cast<float*>(static_cast<char*>(ws) + part_o);
  p.H = (int)H; p.L = (int)pos; p.splits = splits; p.chunk = chunk;
  p.scale_log2 = (float)((double)scale * 1.4426950408889634);
  deers::launch_attn_decode_f16(p, (int)B, (int)D, true, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// ---- element-wise helpers of the storage backend ----

static int check_dtype(int dtype) {
  if (dtype != DEERS_ROCM_F16 && dtype != DEERS_ROCM_F32)
    return fail(DEERS_ROCM_ERR_ARG, "unknown dtype %d", dtype);
  return DEERS_ROCM_OK;
}

int deers_rocm_fill(int dtype, void* dst, size_t n, float value) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n == 0) return DEERS_ROCM_OK;
  if (!dst) return fail(DEERS_ROCM_ERR_ARG, "fill: null pointer");
  deers::launch_fill(dtype == DEERS_ROCM_F16, dst, n, value, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_add(int dtype, const void* a, const void* b, void* out, size_t n) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n == 0) return DEERS_ROCM_OK;
  if (!a || !b || !out) return fail(DEERS_ROCM_ERR_ARG, "add: null pointer");
  deers::launch_add(dtype == DEERS_ROCM_F16, a, b, out, n, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_neg(int dtype, const void* a, void* out, size_t n) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n == 0) return DEERS_ROCM_OK;
  if (!a || !out) return fail(DEERS_ROCM_ERR_ARG, "neg: null pointer");
  deers::launch_neg(dtype == DEERS_ROCM_F16, a, out, n, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_copy_compact(int dtype, const void* src, const int64_t* shape,
                            const int64_t* strides, int ndim, void* dst) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (ndim < 1 || ndim > 6) return fail(DEERS_ROCM_ERR_ARG, "copy_compact: ndim %d not in 1..6", ndim);
  if (!src || !dst || !shape || !strides) return fail(DEERS_ROCM_ERR_ARG, "copy_compact: null pointer");
  for (int d = 0; d < ndim; ++d)
    if (shape[d] < 0 || strides[d] < 0)
      return fail(DEERS_ROCM_ERR_LAYOUT, "copy_compact: negative extent or stride in dim %d", d);
  deers::launch_copy_strided(dtype == DEERS_ROCM_F16, src, shape, strides, ndim, dst, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_copy_view(int dtype, const void* src, const int64_t* src_strides, void* dst,
                         const int64_t* dst_strides, const int64_t* shape, int ndim) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (ndim < 1 || ndim > 6) return fail(DEERS_ROCM_ERR_ARG, "copy_view: ndim %d not in 1..6", ndim);
  if (!src || !dst || !shape || !src_strides || !dst_strides)
    return fail(DEERS_ROCM_ERR_ARG, "copy_view: null pointer");
  for (int d = 0; d < ndim; ++d)
    if (shape[d] < 0 || src_strides[d] < 0 || dst_strides[d] < 0)
      return fail(DEERS_ROCM_ERR_LAYOUT, "copy_view: negative extent or stride in dim %d", d);
  deers::launch_copy_view(dtype == DEERS_ROCM_F16, src, src_strides, dst, dst_strides, shape, ndim,
                          g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// ---- row-wise log-softmax ----

static int lsm_check(const char* what, int dtype, int64_t outer, int64_t inner) {
  if (int rc = check_dtype(dtype)) return rc;
  if (outer < 0 || inner < 1 || outer > INT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "%s: need 0 <= outer < 2^31 rows of inner >= 1 elements", what);
  return DEERS_ROCM_OK;
}

int deers_rocm_log_softmax_fwd(int dtype, const void* x, void* out, int64_t outer, int64_t inner) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = lsm_check("log_softmax_fwd", dtype, outer, inner)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !out) return fail(DEERS_ROCM_ERR_ARG, "log_softmax_fwd: null pointer");
  deers::launch_log_softmax_fwd(dtype == DEERS_ROCM_F16, x, out, outer, inner, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_log_softmax_bwd(int dtype, const void* grad, const void* lsm, void* out,
                               int64_t outer, int64_t inner) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = lsm_check("log_softmax_bwd", dtype, outer, inner)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!grad || !lsm || !out) return fail(DEERS_ROCM_ERR_ARG, "log_softmax_bwd: null pointer");
  deers::launch_log_softmax_bwd(dtype == DEERS_ROCM_F16, grad, lsm, out, outer, inner, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// ---- the other ops of a GPT training step ----

static int rows_check(const char* what, int dtype, int64_t outer, int64_t inner) {
  if (int rc = check_dtype(dtype)) return rc;
  if (outer < 0 || inner < 1 || inner > INT32_MAX || outer > INT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "%s: need 0 <= rows < 2^31 of 1 <= width < 2^31 elements", what);
  return DEERS_ROCM_OK;
}

int deers_rocm_index_select(int dtype, const void* table, const int64_t* indices, void* out,
                            int64_t n_rows, int64_t n_indices, int64_t width) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("index_select", dtype, n_indices, width)) return rc;
  if (n_rows < 0) return fail(DEERS_ROCM_ERR_ARG, "index_select: negative table size");
  if (n_indices == 0) return DEERS_ROCM_OK;
  if (!table || !indices || !out) return fail(DEERS_ROCM_ERR_ARG, "index_select: null pointer");
  int* flag = nullptr;
  if (int rc = index_flag(&flag)) return rc;
  deers::launch_index_select(dtype == DEERS_ROCM_F16, table, indices, out, n_rows, n_indices,
                             (int)width, flag, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_index_add(int dtype, const void* src, const int64_t* indices, void* dst,
                         int64_t n_rows, int64_t n_indices, int64_t width) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("index_add", dtype, n_indices, width)) return rc;
  if (n_rows < 0) return fail(DEERS_ROCM_ERR_ARG, "index_add: negative destination size");
  if (n_indices == 0) return DEERS_ROCM_OK;
  if (!src || !indices || !dst) return fail(DEERS_ROCM_ERR_ARG, "index_add: null pointer");
  int* flag = nullptr;
  if (int rc = index_flag(&flag)) return rc;
  deers::launch_index_add(dtype == DEERS_ROCM_F16, src, indices, dst, n_rows, n_indices,
                          (int)width, flag, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_rms_norm_fwd(int dtype, const void* x, void* y, int64_t outer, int64_t inner,
                            double eps) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("rms_norm_fwd", dtype, outer, inner)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !y) return fail(DEERS_ROCM_ERR_ARG, "rms_norm_fwd: null pointer");
  deers::launch_rms_norm(dtype == DEERS_ROCM_F16, x, nullptr, nullptr, y, outer, (int)inner, (float)eps, 0,
                         g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_rms_norm_bwd(int dtype, const void* x, const void* dy, void* dx, int64_t outer,
                            int64_t inner, double eps) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("rms_norm_bwd", dtype, outer, inner)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !dy || !dx) return fail(DEERS_ROCM_ERR_ARG, "rms_norm_bwd: null pointer");
  deers::launch_rms_norm(dtype == DEERS_ROCM_F16, x, dy, nullptr, dx, outer, (int)inner, (float)eps, 1,
                         g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_rms_norm_bwd_add(int dtype, const void* x, const void* dy, const void* addend, void* dx,
                                int64_t outer, int64_t inner, double eps) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("rms_norm_bwd_add", dtype, outer, inner)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !dy || !addend || !dx) return fail(DEERS_ROCM_ERR_ARG, "rms_norm_bwd_add: null pointer");
  deers::launch_rms_norm(dtype == DEERS_ROCM_F16, x, dy, addend, dx, outer, (int)inner, (float)eps, 1,
                         g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_relu_sq_fwd(int dtype, const void* x, void* y, int64_t n) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n < 0) return fail(DEERS_ROCM_ERR_ARG, "relu_sq_fwd: negative element count");
  if (n == 0) return DEERS_ROCM_OK;
  if (!x || !y) return fail(DEERS_ROCM_ERR_ARG, "relu_sq_fwd: null pointer");
  deers::launch_relu_sq(dtype == DEERS_ROCM_F16, x, nullptr, y, n, 0, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_relu_sq_bwd(int dtype, const void* x, const void* dy, void* dx, int64_t n) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n < 0) return fail(DEERS_ROCM_ERR_ARG, "relu_sq_bwd: negative element count");
  if (n == 0) return DEERS_ROCM_OK;
  if (!x || !dy || !dx) return fail(DEERS_ROCM_ERR_ARG, "relu_sq_bwd: null pointer");
  deers::launch_relu_sq(dtype == DEERS_ROCM_F16, x, dy, dx, n, 1, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_argmax_rows(int dtype, const void* x, int64_t* out, int64_t outer, int64_t inner) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("argmax_rows", dtype, outer, inner)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !out) return fail(DEERS_ROCM_ERR_ARG, "argmax_rows: null pointer");
  deers::launch_argmax_rows(dtype == DEERS_ROCM_F16, x, out, outer, (int)inner, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// the forward, and with dlogits also the gradient for an upstream gradient of one; the caller holds g_mu
static int cross_entropy_fwd_locked(const char* what, int dtype, const void* logits, const int64_t* targets,
                                    float* row_lse, float* loss, void* dlogits, int64_t n_rows,
                                    int64_t n_classes) {
  NEED_INIT();
  if (int rc = rows_check(what, dtype, n_rows, n_classes)) return rc;
  if (n_rows < 1) return fail(DEERS_ROCM_ERR_ARG, "%s: needs at least one row", what);
  if (!logits || !targets || !row_lse || !loss) return fail(DEERS_ROCM_ERR_ARG, "%s: null pointer", what);
  void* ws = nullptr;  // per-row losses
  if (int rc = workspace((size_t)n_rows * sizeof(float), &ws)) return rc;
  int* flag = nullptr;
  if (int rc = index_flag(&flag)) return rc;
  deers::launch_cross_entropy_fwd(dtype == DEERS_ROCM_F16, logits, targets, row_lse, (float*)ws, loss, dlogits,
                                  n_rows, (int)n_classes, flag, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_cross_entropy_fwd(int dtype, const void* logits, const int64_t* targets,
                                 float* row_lse, float* loss, int64_t n_rows, int64_t n_classes) {
  std::lock_guard<std::mutex> lock(g_mu);
  return cross_entropy_fwd_locked("cross_entropy_fwd", dtype, logits, targets, row_lse, loss, nullptr, n_rows,
                                  n_classes);
}

int deers_rocm_cross_entropy_fwd_grad(int dtype, const void* logits, const int64_t* targets, float* row_lse,
                                      float* loss, void* dlogits, int64_t n_rows, int64_t n_classes) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!dlogits) return fail(DEERS_ROCM_ERR_ARG, "cross_entropy_fwd_grad: null pointer");
  return cross_entropy_fwd_locked("cross_entropy_fwd_grad", dtype, logits, targets, row_lse, loss, dlogits,
                                  n_rows, n_classes);
}

int deers_rocm_scale_by_scalar(int dtype, void* x, int64_t n, const float* factor) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n < 0) return fail(DEERS_ROCM_ERR_ARG, "scale_by_scalar: negative element count");
  if (n == 0) return DEERS_ROCM_OK;
  if (!x || !factor) return fail(DEERS_ROCM_ERR_ARG, "scale_by_scalar: null pointer");
  deers::launch_scale_by_device_scalar(dtype == DEERS_ROCM_F16, x, n, factor, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_cross_entropy_bwd(int dtype, const void* logits, const int64_t* targets,
                                 const float* row_lse, const float* upstream, void* dlogits,
                                 int64_t n_rows, int64_t n_classes) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("cross_entropy_bwd", dtype, n_rows, n_classes)) return rc;
  if (n_rows < 1) return fail(DEERS_ROCM_ERR_ARG, "cross_entropy_bwd: needs at least one row");
  if (!logits || !targets || !row_lse || !dlogits)
    return fail(DEERS_ROCM_ERR_ARG, "cross_entropy_bwd: null pointer");
  deers::launch_cross_entropy_bwd(dtype == DEERS_ROCM_F16, logits, targets, row_lse, upstream, dlogits,
                                  n_rows, (int)n_classes, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// ---- the generic BackendStorage kernels ----
static_assert(deers::kUnaryNeg == DEERS_ROCM_UNARY_NEG && deers::kUnaryPowf == DEERS_ROCM_UNARY_POWF &&
                  deers::kUnaryScalarAdd == DEERS_ROCM_UNARY_SCALAR_ADD &&
                  deers::kBinaryAdd == DEERS_ROCM_BINARY_ADD && deers::kBinaryEq == DEERS_ROCM_BINARY_EQ,
              "op codes of the header and of storage_ops.h must agree");

// Collapses (shape, strides) into a StridedView: dimensions of extent 1 dropped, a
// dimension merged into its inner neighbour where the two are contiguous with each
// other.  Returns false if the view is compact (no StridedView needed).
static bool make_view(int ndim, const int64_t* shape, const int64_t* strides, deers::StridedView* v) {
  v->ndim = 0;
  if (!strides) return false;
  int64_t s[deers::kMaxViewDims], t[deers::kMaxViewDims];
  int n = 0;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] == 1) continue;
    if (n > 0 && t[n - 1] == strides[d] * shape[d]) {  // outer stride spans the inner dimension
      s[n - 1] *= shape[d];
      t[n - 1] = strides[d];
    } else {
      s[n] = shape[d];
      t[n] = strides[d];
      ++n;
    }
  }
  if (n == 0 || (n == 1 && t[0] == 1)) return false;
  v->ndim = n;
  for (int d = 0; d < n; ++d) {
    v->shape[d] = (uint32_t)s[d];
    v->stride[d] = t[d];
  }
  return true;
}

// element count of `shape`, or -1 if a dimension is negative or the view is too large
static int64_t view_elements(const char* what, int ndim, const int64_t* shape) {
  if (ndim < 1 || ndim > deers::kMaxViewDims) {
    fail(DEERS_ROCM_ERR_ARG, "%s: ndim %d not in 1..%d", what, ndim, deers::kMaxViewDims);
    return -1;
  }
  if (!shape) {
    fail(DEERS_ROCM_ERR_ARG, "%s: null shape", what);
    return -1;
  }
  int64_t n = 1;
  for (int d = 0; d < ndim; ++d) {
    if (shape[d] < 0) {
      fail(DEERS_ROCM_ERR_LAYOUT, "%s: negative extent in dim %d", what, d);
      return -1;
    }
    if (shape[d] > 0 && n > INT64_MAX / shape[d]) {
      fail(DEERS_ROCM_ERR_ARG, "%s: element count overflows", what);
      return -1;
    }
    n *= shape[d];
  }
  return n;
}

int deers_rocm_unary(int dtype, int op, const void* x, int ndim, const int64_t* shape,
                     const int64_t* strides, double param, void* out) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (op < 0 || op >= deers::kUnaryCount) return fail(DEERS_ROCM_ERR_ARG, "unary: unknown op %d", op);
  const int64_t n = view_elements("unary", ndim, shape);
  if (n < 0) return DEERS_ROCM_ERR_ARG;
  if (n == 0) return DEERS_ROCM_OK;
  if (!x || !out) return fail(DEERS_ROCM_ERR_ARG, "unary: null pointer");
  deers::StridedView view;
  const bool strided = make_view(ndim, shape, strides, &view);
  if ((strided || ((uintptr_t)x & 15) || ((uintptr_t)out & 15)) && n > (int64_t)UINT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "unary: a strided or unaligned operand is limited to 2^32 - 1 elements");
  deers::launch_unary(dtype == DEERS_ROCM_F16, op, x, strided ? &view : nullptr, out, n, param, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_binary(int dtype, int op, const void* a, const int64_t* a_strides, const void* b,
                      const int64_t* b_strides, int ndim, const int64_t* shape, void* out) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (op < 0 || op >= deers::kBinaryCount) return fail(DEERS_ROCM_ERR_ARG, "binary: unknown op %d", op);
  const int64_t n = view_elements("binary", ndim, shape);
  if (n < 0) return DEERS_ROCM_ERR_ARG;
  if (n == 0) return DEERS_ROCM_OK;
  if (!a || !b || !out) return fail(DEERS_ROCM_ERR_ARG, "binary: null pointer");
  deers::StridedView va, vb;
  const bool sa = make_view(ndim, shape, a_strides, &va), sb = make_view(ndim, shape, b_strides, &vb);
  const bool vector_path = !sa && !sb && !((uintptr_t)a & 15) && !((uintptr_t)b & 15) && !((uintptr_t)out & 15);
  if (!vector_path && n > (int64_t)UINT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "binary: strided or unaligned operands are limited to 2^32 - 1 elements");
  deers::launch_binary(dtype == DEERS_ROCM_F16, op, a, sa ? &va : nullptr, b, sb ? &vb : nullptr, out, n,
                       g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_reduce(int dtype, int op, const void* x, void* out, int64_t outer, int64_t reduce_size) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("reduce", dtype, outer, reduce_size)) return rc;
  if (op != DEERS_ROCM_REDUCE_SUM && op != DEERS_ROCM_REDUCE_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "reduce: unknown op %d", op);
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !out) return fail(DEERS_ROCM_ERR_ARG, "reduce: null pointer");
  deers::launch_reduce(dtype == DEERS_ROCM_F16, op == DEERS_ROCM_REDUCE_MAX, x, out, outer, reduce_size,
                       g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_log_sum_exp(int dtype, const void* x, void* out, int64_t outer, int64_t reduce_size) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = rows_check("log_sum_exp", dtype, outer, reduce_size)) return rc;
  if (outer == 0) return DEERS_ROCM_OK;
  if (!x || !out) return fail(DEERS_ROCM_ERR_ARG, "log_sum_exp: null pointer");
  deers::launch_log_sum_exp(dtype == DEERS_ROCM_F16, x, out, outer, reduce_size, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

static int dim_check(const char* what, int64_t left, int64_t dim, int64_t index_len, int64_t right) {
  if (left < 0 || dim < 0 || index_len < 0 || right < 0)
    return fail(DEERS_ROCM_ERR_ARG, "%s: negative extent", what);
  const int64_t lim = (int64_t)1 << 40;
  if (left > lim || dim > lim || index_len > lim || right > lim ||
      (double)left * (double)right * (double)(dim > index_len ? dim : index_len) > 9.0e18)
    return fail(DEERS_ROCM_ERR_ARG, "%s: element count overflows", what);
  return DEERS_ROCM_OK;
}

int deers_rocm_gather(int dtype, const void* src, const int64_t* indices, void* out, int64_t left,
                      int64_t src_dim, int64_t index_len, int64_t right) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (dtype != DEERS_ROCM_F16 && dtype != DEERS_ROCM_F32 && dtype != DEERS_ROCM_I64)
    return fail(DEERS_ROCM_ERR_ARG, "gather: unknown dtype %d", dtype);
  if (int rc = dim_check("gather", left, src_dim, index_len, right)) return rc;
  if (left * index_len * right == 0) return DEERS_ROCM_OK;
  if (!src || !indices || !out) return fail(DEERS_ROCM_ERR_ARG, "gather: null pointer");
  int* flag = nullptr;
  if (int rc = index_flag(&flag)) return rc;
  const int bytes = dtype == DEERS_ROCM_F16 ? 2 : dtype == DEERS_ROCM_F32 ? 4 : 8;
  deers::launch_gather(bytes, src, indices, out, left, src_dim, index_len, right, flag, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_scatter_add(int dtype, const void* src, const int64_t* indices, void* dst, int64_t left,
                           int64_t dst_dim, int64_t index_len, int64_t right) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (int rc = dim_check("scatter_add", left, dst_dim, index_len, right)) return rc;
  if (left * index_len * right == 0) return DEERS_ROCM_OK;
  if (!src || !indices || !dst) return fail(DEERS_ROCM_ERR_ARG, "scatter_add: null pointer");
  if (left * right > (int64_t)INT32_MAX * 256)
    return fail(DEERS_ROCM_ERR_ARG, "scatter_add: too many columns for one call");
  int* flag = nullptr;
  if (int rc = index_flag(&flag)) return rc;
  deers::launch_scatter_add(dtype == DEERS_ROCM_F16, src, indices, dst, left, dst_dim, index_len, right,
                            flag, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// ---- optimizer step ----

int deers_rocm_adamw_step(int dtype, void* w, const void* grad, void* m, void* v, int64_t n,
                          double lr, double beta1, double beta2, double eps, double weight_decay,
                          int64_t step, double grad_scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n < 0) return fail(DEERS_ROCM_ERR_ARG, "adamw_step: negative element count");
  if (step < 1 || step > INT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "adamw_step: step counts from 1 (got %lld)", (long long)step);
  if (n == 0) return DEERS_ROCM_OK;
  if (!w || !grad || !m || !v) return fail(DEERS_ROCM_ERR_ARG, "adamw_step: null pointer");
  deers::launch_adamw(dtype == DEERS_ROCM_F16, w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay,
                      (int)step, grad_scale, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_sum_squares(int dtype, const void* x, int64_t n, float* total, int accumulate) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n < 0) return fail(DEERS_ROCM_ERR_ARG, "sum_squares: negative element count");
  if (!total || (n > 0 && !x)) return fail(DEERS_ROCM_ERR_ARG, "sum_squares: null pointer");
  void* ws = nullptr;
  if (int rc = workspace(deers::sumsq_partial_count() * sizeof(float), &ws)) return rc;
  deers::launch_sumsq(dtype == DEERS_ROCM_F16, x, n, (float*)ws, total, accumulate, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// Tensors the multi-tensor kernels take: non-empty and 16-byte aligned.
static bool multi_ok(const void* p, int64_t n) { return n > 0 && ((uintptr_t)p & 15) == 0; }

int deers_rocm_adamw_step_multi(int dtype, int n_tensors, void* const* w, const void* const* grad,
                                void* const* m, void* const* v, const int64_t* sizes, double lr,
                                double beta1, double beta2, double eps, double weight_decay,
                                int64_t step, double grad_scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n_tensors < 0) return fail(DEERS_ROCM_ERR_ARG, "adamw_step_multi: negative tensor count");
  if (step < 1 || step > INT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "adamw_step_multi: step counts from 1 (got %lld)", (long long)step);
  if (n_tensors == 0) return DEERS_ROCM_OK;
  if (!w || !grad || !m || !v || !sizes) return fail(DEERS_ROCM_ERR_ARG, "adamw_step_multi: null table");
  const int f16 = dtype == DEERS_ROCM_F16;
  for (int i = 0; i < n_tensors; ++i) {
    if (sizes[i] < 0) return fail(DEERS_ROCM_ERR_ARG, "adamw_step_multi: tensor %d has a negative size", i);
    if (sizes[i] > 0 && (!w[i] || !grad[i] || !m[i] || !v[i]))
      return fail(DEERS_ROCM_ERR_ARG, "adamw_step_multi: tensor %d has a null pointer", i);
  }
  // groups of aligned tensors go out together; an unaligned one takes the single-tensor kernels
  const int cap = deers::multi_max_tensors();
  std::vector<void*> gw, gm, gv;
  std::vector<const void*> gg;
  std::vector<int64_t> gn;
  int64_t group_blocks = 0;
  auto flush = [&]() {
    if (gw.empty()) return;
    deers::launch_adamw_multi(f16, (int)gw.size(), gw.data(), gg.data(), gm.data(), gv.data(), gn.data(), lr,
                              beta1, beta2, eps, weight_decay, (int)step, grad_scale, g_rt.stream);
    gw.clear(); gg.clear(); gm.clear(); gv.clear(); gn.clear();
    group_blocks = 0;
  };
  for (int i = 0; i < n_tensors; ++i) {
    if (sizes[i] == 0) continue;
    if (multi_ok(w[i], sizes[i]) && multi_ok(grad[i], sizes[i]) && multi_ok(m[i], sizes[i]) &&
        multi_ok(v[i], sizes[i])) {
      const int64_t nb = deers::multi_blocks(f16, sizes[i]);
      if ((int)gw.size() == cap || group_blocks + nb > INT32_MAX / 2) flush();
      gw.push_back(w[i]); gg.push_back(grad[i]); gm.push_back(m[i]); gv.push_back(v[i]); gn.push_back(sizes[i]);
      group_blocks += nb;
    } else {
      deers::launch_adamw(f16, w[i], grad[i], m[i], v[i], sizes[i], lr, beta1, beta2, eps, weight_decay,
                          (int)step, grad_scale, g_rt.stream);
    }
  }
  flush();
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_sum_squares_multi(int dtype, int n_tensors, const void* const* x, const int64_t* sizes,
                                 float* total, int accumulate) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n_tensors < 0) return fail(DEERS_ROCM_ERR_ARG, "sum_squares_multi: negative tensor count");
  if (!total) return fail(DEERS_ROCM_ERR_ARG, "sum_squares_multi: null total");
  if (n_tensors > 0 && (!x || !sizes)) return fail(DEERS_ROCM_ERR_ARG, "sum_squares_multi: null table");
  const int f16 = dtype == DEERS_ROCM_F16;
  int64_t blocks = 0;
  for (int i = 0; i < n_tensors; ++i) {
    if (sizes[i] < 0) return fail(DEERS_ROCM_ERR_ARG, "sum_squares_multi: tensor %d has a negative size", i);
    if (sizes[i] > 0 && !x[i]) return fail(DEERS_ROCM_ERR_ARG, "sum_squares_multi: tensor %d is null", i);
    if (sizes[i] > 0 && ((uintptr_t)x[i] & 15))
      return fail(DEERS_ROCM_ERR_LAYOUT, "sum_squares_multi: tensor %d is not 16-byte aligned; use "
                  "deers_rocm_sum_squares for it", i);
    blocks += deers::multi_blocks(f16, sizes[i]);
  }
  if (blocks > INT32_MAX / 2) return fail(DEERS_ROCM_ERR_ARG, "sum_squares_multi: too many elements for one call");
  void* ws = nullptr;  // one partial per block of every tensor, then one fixed-order sum
  if (int rc = workspace((size_t)(blocks > 0 ? blocks : 1) * sizeof(float), &ws)) return rc;
  float* partial = (float*)ws;
  const int cap = deers::multi_max_tensors();
  int written = 0;
  std::vector<const void*> gx;
  std::vector<int64_t> gn;
  auto flush = [&]() {
    if (gx.empty()) return;
    written += deers::launch_sumsq_multi(f16, (int)gx.size(), gx.data(), gn.data(), partial + written, g_rt.stream);
    gx.clear(); gn.clear();
  };
  for (int i = 0; i < n_tensors; ++i) {
    if (sizes[i] == 0) continue;
    if ((int)gx.size() == cap) flush();
    gx.push_back(x[i]); gn.push_back(sizes[i]);
  }
  flush();
  deers::launch_sumsq_final(partial, written, total, accumulate, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_scale(int dtype, void* x, int64_t n, double scale) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (n < 0) return fail(DEERS_ROCM_ERR_ARG, "scale: negative element count");
  if (n == 0) return DEERS_ROCM_OK;
  if (!x) return fail(DEERS_ROCM_ERR_ARG, "scale: null pointer");
  deers::launch_scale(dtype == DEERS_ROCM_F16, x, n, scale, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// ---- batched matrix product (library GEMM) ----

// the solution-enumeration calls are tagged "beta, subject to change" by their header
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Wdeprecated-declarations"

#define HIP_TRY_BOOL(expr)              \
  do {                                  \
    if ((expr) != hipSuccess) {         \
      (void)hipGetLastError();          \
      return false;                     \
    }                                   \
  } while (0)

int deers_rocm_matmul_tune(int on) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  g_rt.tune_gemm = on != 0;
  return DEERS_ROCM_OK;
}

constexpr size_t kTuneScratchMax = (size_t)256 << 20;  // largest output a tuned product with an addend may have
constexpr int kSkinnyCounters = 4096;  // column blocks a K-split launch of the few-rows GEMM may have

// The few-rows GEMM on operands skinny_gemm_takes() accepted; prologue 0 none, 1 rms_norm
// of x's rows, 2 relu(x)^2.  The caller holds g_mu.
static int skinny_locked(const void* x, int64_t ldx, const void* w, int64_t ldw, void* y, int64_t m,
                         int64_t n, int64_t k, bool accumulate, int prologue, float eps, bool packed) {
  // row sums of squares need all of K; the split sum's hand-over needs the splits of a
  // column block on one XCD
  int splits = (prologue == 1 || !same_xcd_handover_now()) ? 1 : deers::skinny_gemm_splits(n, k);
  void* ws = nullptr;
  if (splits > 1 && (n + 31) / 32 > kSkinnyCounters) splits = 1;
  if (splits > 1) {
    if (int rc = workspace(deers::skinny_gemm_workspace_bytes(n, splits), &ws)) return rc;
    if (!g_rt.skinny_counters) {  // zero once; the kernel leaves every counter at zero
      HIP_TRY(hipMalloc(&g_rt.skinny_counters, kSkinnyCounters * sizeof(int)));
      HIP_TRY(hipMemsetAsync(g_rt.skinny_counters, 0, kSkinnyCounters * sizeof(int), g_rt.stream));
    }
  }
  const deers::SkinnyPrefetch next = g_rt.skinny_next;
  g_rt.skinny_next = deers::SkinnyPrefetch{};  // a hint serves one launch
  deers::LaunchScope scope("matmul", g_rt.stream);
  deers::launch_skinny_gemm_f16(x, ldx, w, ldw, y, n, (int)m, (int)n, (int)k, accumulate, prologue, eps, packed,
                                splits, (float*)ws, g_rt.skinny_counters, next, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

// c = a @ b (addend null) or c = a @ b + addend (compact like c; may be c itself); the
// caller holds g_mu
static int matmul_locked(int dtype, const void* a, int64_t a_rs, int64_t a_cs, int64_t a_bs,
                         const void* b, int64_t b_rs, int64_t b_cs, int64_t b_bs, const void* addend,
                         void* c, int64_t batch, int64_t m, int64_t n, int64_t k) {
  NEED_INIT();
  const bool accumulate = addend != nullptr;
  if (int rc = check_dtype(dtype)) return rc;
  if (batch < 0 || m < 0 || n < 0 || k < 0 || m > INT32_MAX || n > INT32_MAX || k > INT32_MAX ||
      batch > INT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "matmul: sizes must be in [0, 2^31)");
  if (batch == 0 || m == 0 || n == 0) return DEERS_ROCM_OK;
  if (!a || !b || !c) return fail(DEERS_ROCM_ERR_ARG, "matmul: null pointer");
  const size_t c_bytes = (size_t)(batch * m * n) * (dtype == DEERS_ROCM_F16 ? 2 : 4);
  if (k == 0) {  // empty sum
    if (accumulate) {
      if (addend != c) HIP_TRY(hipMemcpyAsync(c, addend, c_bytes, hipMemcpyDeviceToDevice, g_rt.stream));
      return DEERS_ROCM_OK;
    }
    deers::launch_fill(dtype == DEERS_ROCM_F16, c, (size_t)(batch * m * n), 0.f, g_rt.stream);
    HIP_TRY(hipGetLastError());
    return DEERS_ROCM_OK;
  }
  // A matrix the BLAS can take needs a unit stride along rows or along columns
  // (a dimension of extent 1 has no stride to speak of).
  auto unit = [](int64_t rows, int64_t cols, int64_t rs, int64_t cs, bool* transposed,
                 int64_t* ld) {
    if (cs == 1 || cols == 1) { *transposed = false; *ld = rows == 1 ? (rs > cols ? rs : cols) : rs; return rs >= cols || rows == 1; }
    if (rs == 1 || rows == 1) { *transposed = true; *ld = cols == 1 ? (cs > rows ? cs : rows) : cs; return cs >= rows || cols == 1; }
    return false;
  };
  bool a_t = false, b_t = false;
  int64_t lda = 0, ldb = 0;
  if (!unit(m, k, a_rs, a_cs, &a_t, &lda) || !unit(k, n, b_rs, b_cs, &b_t, &ldb) || a_bs < 0 ||
      b_bs < 0)
    return fail(DEERS_ROCM_ERR_LAYOUT,
                "matmul: each operand needs a unit row or column stride and non-overlapping "
                "lines (a %lld,%lld b %lld,%lld); compact the tensor first",
                (long long)a_rs, (long long)a_cs, (long long)b_rs, (long long)b_cs);
  // a few rows against a weight matrix (a generation step's projections): one streaming
  // pass over the weights instead of a library GEMM
  if (dtype == DEERS_ROCM_F16 && batch == 1 && !a_t && !b_t && (!accumulate || addend == c) &&
      deers::skinny_gemm_takes(m, n, k, lda, ldb, n, a, b, c))
    return skinny_locked(a, lda, b, ldb, c, m, n, k, accumulate, 0, 0.f, false);
  g_rt.skinny_next = deers::SkinnyPrefetch{};  // a pending prefetch hint does not outlive this product
  if (!g_rt.blas) {
    if (rocblas_create_handle(&g_rt.blas) != rocblas_status_success)
      return fail(DEERS_ROCM_ERR_HIP, "rocblas_create_handle failed");
    if (rocblas_set_stream(g_rt.blas, g_rt.stream) != rocblas_status_success)
      return fail(DEERS_ROCM_ERR_HIP, "rocblas_set_stream failed");
  }
  // Row-major C = A B is column-major C^T = B^T A^T: the BLAS sees B first.  A
  // row-major [rows x cols] matrix with unit column stride is, read column-major, its
  // own transpose with leading dimension = row stride.
  const rocblas_datatype ty = dtype == DEERS_ROCM_F16 ? rocblas_datatype_f16_r : rocblas_datatype_f32_r;
  const float alpha = 1.f, beta = accumulate ? 1.f : 0.f;
  const rocblas_operation op_b = b_t ? rocblas_operation_transpose : rocblas_operation_none;
  const rocblas_operation op_a = a_t ? rocblas_operation_transpose : rocblas_operation_none;
  const void* c_in = accumulate ? addend : c;
  auto run_into = [&](int solution, void* out) {
    return rocblas_gemm_strided_batched_ex(
        g_rt.blas, op_b, op_a, (rocblas_int)n, (rocblas_int)m, (rocblas_int)k, &alpha, b, ty,
        (rocblas_int)ldb, b_bs, a, ty, (rocblas_int)lda, a_bs, &beta, c_in, ty, (rocblas_int)n, m * n, out,
        ty, (rocblas_int)n, m * n, (rocblas_int)batch, rocblas_datatype_f32_r,
        solution ? rocblas_gemm_algo_solution_index : rocblas_gemm_algo_standard, solution, 0);
  };
  auto run = [&](int solution) { return run_into(solution, c); };
  int solution = 0;
  if (g_rt.tune_gemm) {
    const std::vector<int64_t> key{dtype, (int64_t)b_t, (int64_t)a_t, n, m, k, ldb, lda, b_bs, a_bs, batch};
    auto hit = g_rt.gemm_choice.find(key);
    if (hit != g_rt.gemm_choice.end()) {
      solution = hit->second;
    } else if (!accumulate || c_bytes <= kTuneScratchMax) {
      // Times the default and every listed kernel on the caller's own operands: one
      // warm-up and one timed run each, a second timed run for those within 20 % of the
      // best so far.  A plain product's trial runs write the output the real call below
      // overwrites; a product with an addend writes its trials into the workspace, since
      // the addend may be the output itself.
      void* trial_out = c;
      if (accumulate)
        if (int rc = workspace(c_bytes, &trial_out)) return rc;
      rocblas_int count = 0;
      std::vector<rocblas_int> list;
      if (rocblas_gemm_strided_batched_ex_get_solutions(
              g_rt.blas, op_b, op_a, (rocblas_int)n, (rocblas_int)m, (rocblas_int)k, &alpha, b, ty,
              (rocblas_int)ldb, b_bs, a, ty, (rocblas_int)lda, a_bs, &beta, c_in, ty, (rocblas_int)n,
              m * n, c, ty, (rocblas_int)n, m * n, (rocblas_int)batch, rocblas_datatype_f32_r,
              rocblas_gemm_algo_solution_index, 0, nullptr, &count) == rocblas_status_success &&
          count > 0) {
        list.resize(count);
        if (rocblas_gemm_strided_batched_ex_get_solutions(
                g_rt.blas, op_b, op_a, (rocblas_int)n, (rocblas_int)m, (rocblas_int)k, &alpha, b, ty,
                (rocblas_int)ldb, b_bs, a, ty, (rocblas_int)lda, a_bs, &beta, c_in, ty, (rocblas_int)n,
                m * n, c, ty, (rocblas_int)n, m * n, (rocblas_int)batch, rocblas_datatype_f32_r,
                rocblas_gemm_algo_solution_index, 0, list.data(), &count) != rocblas_status_success)
          list.clear();
      }
      hipEvent_t e0, e1;
      HIP_TRY(hipEventCreate(&e0));
      HIP_TRY(hipEventCreate(&e1));
      auto time_runs = [&](int sol, int runs, float* ms) -> bool {  // mean of back-to-back launches
        HIP_TRY_BOOL(hipEventRecord(e0, g_rt.stream));
        for (int i = 0; i < runs; ++i)
          if (run_into(sol, trial_out) != rocblas_status_success) return false;
        HIP_TRY_BOOL(hipEventRecord(e1, g_rt.stream));
        HIP_TRY_BOOL(hipEventSynchronize(e1));
        HIP_TRY_BOOL(hipEventElapsedTime(ms, e0, e1));
        *ms /= (float)runs;
        return true;
      };
      auto time_one = [&](int sol, float* ms) -> bool { return time_runs(sol, 1, ms); };
      float best = 0.f;
      float t = 0.f;
      if (!time_one(0, &t) || !time_one(0, &best)) best = 1e30f;  // warm-up, then the default
      list.insert(list.begin(), 0);
      std::vector<std::pair<float, int>> close{{best, 0}};  // (time, kernel) of the contenders
      for (size_t i = 1; i < list.size(); ++i) {
        float t1 = 0.f, t2 = 0.f;
        if (!time_one(list[i], &t1) || !time_one(list[i], &t1)) continue;  // warm-up, timed
        if (t1 > 1.2f * best) continue;
        if (!time_one(list[i], &t2)) continue;
        const float tt = t1 < t2 ? t1 : t2;
        close.emplace_back(tt, (int)list[i]);
        if (tt < best) best = tt;
      }
      // a single run's time wanders by a few percent, as much as the best kernels differ: the
      // four fastest go again, eight back-to-back launches between one pair of events, three
      // times over, and the smallest mean decides
      std::sort(close.begin(), close.end());
      if (close.size() > 4) close.resize(4);
      best = 1e30f;
      for (int round = 0; round < 3; ++round)
        for (const auto& cand : close)
          if (time_runs(cand.second, 8, &t) && t < best) {
            best = t;
            solution = cand.second;
          }
      (void)hipEventDestroy(e0);
      (void)hipEventDestroy(e1);
      g_rt.gemm_choice[key] = solution;
    }
  }
  deers::LaunchScope scope("matmul", g_rt.stream);
  rocblas_status st = run(solution);
  if (st != rocblas_status_success && solution) st = run(0);
  if (st != rocblas_status_success)
    return fail(DEERS_ROCM_ERR_HIP, "rocblas_gemm_strided_batched_ex failed: %s",
                rocblas_status_to_string(st));
  return DEERS_ROCM_OK;
}

int deers_rocm_matmul(int dtype, const void* a, int64_t a_rs, int64_t a_cs, int64_t a_bs,
                      const void* b, int64_t b_rs, int64_t b_cs, int64_t b_bs, void* c,
                      int64_t batch, int64_t m, int64_t n, int64_t k) {
  std::lock_guard<std::mutex> lock(g_mu);
  return matmul_locked(dtype, a, a_rs, a_cs, a_bs, b, b_rs, b_cs, b_bs, nullptr, c, batch, m, n, k);
}

int deers_rocm_matmul_acc(int dtype, const void* a, int64_t a_rs, int64_t a_cs, int64_t a_bs,
                          const void* b, int64_t b_rs, int64_t b_cs, int64_t b_bs, void* c,
                          int64_t batch, int64_t m, int64_t n, int64_t k) {
  std::lock_guard<std::mutex> lock(g_mu);
  return matmul_locked(dtype, a, a_rs, a_cs, a_bs, b, b_rs, b_cs, b_bs, c, c, batch, m, n, k);
}

int deers_rocm_matmul_add(int dtype, const void* a, int64_t a_rs, int64_t a_cs, int64_t a_bs,
                          const void* b, int64_t b_rs, int64_t b_cs, int64_t b_bs, const void* addend,
                          void* c, int64_t batch, int64_t m, int64_t n, int64_t k) {
  std::lock_guard<std::mutex> lock(g_mu);
  if (!addend && batch > 0 && m > 0 && n > 0) return fail(DEERS_ROCM_ERR_ARG, "matmul_add: null addend");
  return matmul_locked(dtype, a, a_rs, a_cs, a_bs, b, b_rs, b_cs, b_bs, addend, c, batch, m, n, k);
}

int deers_rocm_decode_linear(int dtype, int prologue, float eps, const void* x, int64_t ldx, const void* w,
                             int64_t ldw, void* y, int accumulate, int64_t m, int64_t n, int64_t k) {
  const bool packed = ldw == DEERS_ROCM_LINEAR_W_PACKED;
  if (packed) ldw = n;  // for the shape rules below
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (prologue < DEERS_ROCM_LINEAR_PLAIN || prologue > DEERS_ROCM_LINEAR_RELU_SQ)
    return fail(DEERS_ROCM_ERR_ARG, "decode_linear: unknown prologue %d", prologue);
  if (!x || !w || !y) return fail(DEERS_ROCM_ERR_ARG, "decode_linear: null pointer");
  if (dtype != DEERS_ROCM_F16 || !deers::skinny_gemm_takes(m, n, k, ldx, ldw, n, x, w, y))
    return fail(DEERS_ROCM_ERR_ARG,
                "decode_linear: f16, 1 <= m <= 32, n %% 8 == 0, k %% 256 == 0, row strides multiples of "
                "8 elements and 16-byte aligned pointers (m %lld n %lld k %lld)",
                (long long)m, (long long)n, (long long)k);
  return skinny_locked(x, ldx, w, ldw, y, m, n, k, accumulate != 0, prologue, eps, packed);
}

int deers_rocm_decode_linear_hint(const void* next_w_packed, int64_t n, int64_t k) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  g_rt.skinny_next = deers::SkinnyPrefetch{};
  if (!next_w_packed) return DEERS_ROCM_OK;
  if (n < 1 || k < 256 || k % 256 || k * 64 > INT32_MAX || (n + 31) / 32 * (k / 256) > 65536 ||
      ((uintptr_t)next_w_packed & 15))
    return fail(DEERS_ROCM_ERR_ARG, "decode_linear_hint: bad shape or unaligned pointer");
  g_rt.skinny_next.w = next_w_packed;
  g_rt.skinny_next.n = n;
  g_rt.skinny_next.k = k;
  return DEERS_ROCM_OK;
}
#pragma clang diagnostic pop

// ---- rotary embedding fused with the head split / merge ----

// Checks shared by rope_fwd / rope_bwd.  *vectorised: every row of the strided side is a
// whole number of aligned 16-byte chunks (the fast kernel); any other even D, stride or
// alignment takes the kernel that moves one pair per thread.
static int rope_common(const char* what, int dtype, const void* src, const int64_t* strides,
                       const void* cos, const void* sin, void* dst, int64_t B, int64_t T,
                       int64_t H, int64_t D, int64_t* resolved, bool inverse, bool* vectorised) {
  if (int rc = check_dtype(dtype)) return rc;
  if (!src || !cos || !sin || !dst) return fail(DEERS_ROCM_ERR_ARG, "%s: null pointer", what);
  const int64_t per16 = dtype == DEERS_ROCM_F16 ? 8 : 4;
  if (B < 1 || T < 1 || H < 1 || D < 2 || D % 2 ||
      B * T * H * D >= (int64_t(1) << 40) || B > INT32_MAX || T > INT32_MAX || H > INT32_MAX)
    return fail(DEERS_ROCM_ERR_ARG, "%s: need B,T,H >= 1 and an even D >= 2", what);
  // compact defaults: forward input [B,T,H,D], backward input [B,H,T,D]
  resolved[0] = T * H * D;
  resolved[1] = inverse ? T * D : H * D;
  resolved[2] = D;
  int64_t last = 1;
  if (strides) {
    resolved[0] = strides[0]; resolved[1] = strides[1]; resolved[2] = strides[2];
    last = strides[3];
  }
  if (last != 1)
    return fail(DEERS_ROCM_ERR_LAYOUT, "%s: innermost stride is %lld, need 1", what, (long long)last);
  *vectorised = (D / 2) % per16 == 0;
  for (int d = 0; d < 3; ++d) {
    if (resolved[d] < 0)
      return fail(DEERS_ROCM_ERR_LAYOUT, "%s: strides must be non-negative", what);
    if (resolved[d] % per16) *vectorised = false;
  }
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) |
       reinterpret_cast<uintptr_t>(cos) | reinterpret_cast<uintptr_t>(sin)) & 15)
    *vectorised = false;
  return DEERS_ROCM_OK;
}

int deers_rocm_rope_fwd(int dtype, const void* x, const int64_t* x_strides, const void* cos,
                        const void* sin, void* y, const int64_t* y_strides, int64_t B, int64_t T,
                        int64_t H, int64_t D) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  int64_t st[3];
  bool vectorised = false;
  if (int rc = rope_common("rope_fwd", dtype, x, x_strides, cos, sin, y, B, T, H, D, st, false,
                           &vectorised))
    return rc;
  if (y_strides) {
    const int64_t per16 = dtype == DEERS_ROCM_F16 ? 8 : 4;
    if (y_strides[3] != 1)
      return fail(DEERS_ROCM_ERR_LAYOUT, "rope_fwd: innermost output stride must be 1");
    for (int d = 0; d < 3; ++d) {
      if (y_strides[d] < 0)
        return fail(DEERS_ROCM_ERR_LAYOUT, "rope_fwd: output strides must be non-negative");
      if (y_strides[d] % per16) vectorised = false;
    }
  }
  deers::launch_rope(dtype == DEERS_ROCM_F16, false, vectorised, x, st, cos, sin, y, y_strides,
                     (int)B, (int)T, (int)H, (int)D, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_decode_qkv(int dtype, const void* q, const void* k, const void* v,
                          const int64_t* in_strides, const void* cos_row, const void* sin_row,
                          void* q_out, void* k_cache, void* v_cache, const int64_t* cache_strides,
                          int64_t pos, int64_t capacity, int64_t B, int64_t H, int64_t D) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  if (int rc = check_dtype(dtype)) return rc;
  if (D != 32 && D != 64 && D != 128) return fail(DEERS_ROCM_ERR_ARG, "decode_qkv: head width %lld not in {32, 64, 128}", (long long)D);
  if (B < 0 || H < 0 || B * H > (int64_t)1 << 24) return fail(DEERS_ROCM_ERR_ARG, "decode_qkv: bad batch or head count");
  if (pos < 0 || pos >= capacity) return fail(DEERS_ROCM_ERR_ARG, "decode_qkv: position %lld outside the cache capacity %lld", (long long)pos, (long long)capacity);
  if (B == 0 || H == 0) return DEERS_ROCM_OK;
  if (!q || !k || !v || !in_strides || !cos_row || !sin_row || !q_out || !k_cache || !v_cache || !cache_strides)
    return fail(DEERS_ROCM_ERR_ARG, "decode_qkv: null pointer");
  const int64_t per16 = dtype == DEERS_ROCM_F16 ? 8 : 4;
  for (int d = 0; d < 2; ++d)
    if (in_strides[d] < 0 || in_strides[d] % per16)
      return fail(DEERS_ROCM_ERR_LAYOUT, "decode_qkv: input strides must be non-negative multiples of 16 bytes");
  for (int d = 0; d < 3; ++d)
    if (cache_strides[d] < 0 || cache_strides[d] % per16)
      return fail(DEERS_ROCM_ERR_LAYOUT, "decode_qkv: cache strides must be non-negative multiples of 16 bytes");
  const void* ptrs[8] = {q, k, v, cos_row, sin_row, q_out, k_cache, v_cache};
  for (const void* ptr : ptrs)
    if ((uintptr_t)ptr & 15) return fail(DEERS_ROCM_ERR_LAYOUT, "decode_qkv: pointers must be 16-byte aligned");
  deers::launch_decode_qkv(dtype == DEERS_ROCM_F16, q, k, v, in_strides, cos_row, sin_row, q_out, k_cache,
                           v_cache, cache_strides, pos, (int)B, (int)H, (int)D, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

int deers_rocm_rope_bwd(int dtype, const void* dy, const int64_t* dy_strides, const void* cos,
                        const void* sin, void* dx, int64_t B, int64_t T, int64_t H, int64_t D) {
  std::lock_guard<std::mutex> lock(g_mu);
  NEED_INIT();
  int64_t st[3];
  bool vectorised = false;
  if (int rc = rope_common("rope_bwd", dtype, dy, dy_strides, cos, sin, dx, B, T, H, D, st, true,
                           &vectorised))
    return rc;
  deers::launch_rope(dtype == DEERS_ROCM_F16, true, vectorised, dy, st, cos, sin, dx, nullptr,
                     (int)B, (int)T, (int)H, (int)D, g_rt.stream);
  HIP_TRY(hipGetLastError());
  return DEERS_ROCM_OK;
}

}  // extern "C"
