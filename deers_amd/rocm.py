"""Python binding of the C ABI in include/deers_rocm.h (ctypes, no torch).

This is host-side plumbing for tests and the benchmark: device buffers, copies,
timers and the three attention entry points, called exactly the way a
`Device::Rocm` storage backend in deers would call them over `extern "C"`.
There is no CPU fallback: if the HIP library is missing or no gfx950 device is
present, every call raises.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

F16, F32 = 0, 1
_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("DEERS_ROCM_LIB") or os.path.join(_HERE, "libdeers_rocm.so")

_lib = None
_inited = False


class RocmError(RuntimeError):
    """A non-zero return code from the library (the role of deers' backend error variant)."""


def load() -> ctypes.CDLL:
    """Loads libdeers_rocm.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RocmError(
                f"{LIB_PATH} is missing: build it with `make -C deers_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback path")
        lib = ctypes.CDLL(LIB_PATH)
        lib.deers_rocm_last_error.restype = ctypes.c_char_p
        lib.deers_rocm_stream.restype = ctypes.c_void_p
        _lib = lib
    return _lib


def _check(rc: int):
    if rc != 0:
        raise RocmError(f"deers_rocm error {rc}: {load().deers_rocm_last_error().decode()}")


def available() -> bool:
    return bool(load().deers_rocm_available())


def init(ordinal: int = 0):
    global _inited
    if not _inited:
        _check(load().deers_rocm_init(ctypes.c_int(ordinal)))
        _inited = True


def sync():
    _check(load().deers_rocm_sync())


HANDOVER_STREAM_ORDER, HANDOVER_SAME_XCD = 0, 1


def handover_policy(cu_count: int, cu_mask_set: bool) -> int:
    """deers_rocm_handover_policy: the rule alone, no device needed."""
    return int(load().deers_rocm_handover_policy(ctypes.c_int(cu_count), ctypes.c_int(int(cu_mask_set))))


def handover_mode() -> int:
    """Mode in force: HANDOVER_SAME_XCD / HANDOVER_STREAM_ORDER, -1 before init."""
    return int(load().deers_rocm_handover_mode())


def set_handover_mode(mode: int):
    _check(load().deers_rocm_set_handover_mode(ctypes.c_int(mode)))


def debug_bwd_wait(spin_limit: int = 1 << 20, skip_producers: bool = False):
    """Test hook of the single-launch backward's bounded wait (see the header)."""
    _check(load().deers_rocm_debug_bwd_wait(ctypes.c_int(spin_limit), ctypes.c_int(int(skip_producers))))


def dtype_code(dtype) -> int:
    dtype = np.dtype(dtype)
    if dtype == np.float16:
        return F16
    if dtype == np.float32:
        return F32
    raise TypeError(f"unsupported dtype {dtype}")


class DeviceBuffer:
    """An owned device allocation with a shape and dtype (compact row-major)."""

    def __init__(self, shape, dtype, zeros: bool = False):
        init()
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        ptr = ctypes.c_void_p()
        fn = load().deers_rocm_alloc_zeros if zeros else load().deers_rocm_alloc
        _check(fn(ctypes.c_size_t(self.nbytes), ctypes.byref(ptr)))
        self.ptr = ptr

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.shape, a.dtype)
        _check(load().deers_rocm_htod(buf.ptr, a.ctypes.data_as(ctypes.c_void_p),
                                      ctypes.c_size_t(buf.nbytes)))
        return buf

    def numpy(self) -> np.ndarray:
        out = np.empty(self.shape, dtype=self.dtype)
        _check(load().deers_rocm_dtoh(out.ctypes.data_as(ctypes.c_void_p), self.ptr,
                                      ctypes.c_size_t(self.nbytes)))
        return out

    def free(self):
        if self.ptr is not None and self.ptr.value:
            _check(load().deers_rocm_free(self.ptr))
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Timer:
    """hipEvent pair on the library stream."""

    def __init__(self):
        init()
        self.h = ctypes.c_void_p()
        _check(load().deers_rocm_timer_create(ctypes.byref(self.h)))

    def start(self):
        _check(load().deers_rocm_timer_start(self.h))

    def stop(self):
        _check(load().deers_rocm_timer_stop(self.h))

    def elapsed_ms(self) -> float:
        ms = ctypes.c_float()
        _check(load().deers_rocm_timer_elapsed_ms(self.h, ctypes.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            load().deers_rocm_timer_destroy(self.h)
        except Exception:
            pass


def profile_enable(on: bool = True):
    """Switch per-kernel event timing on (clears earlier records) or off."""
    init()
    _check(load().deers_rocm_profile_enable(ctypes.c_int(1 if on else 0)))


def matmul_tune(on: bool):
    _check(load().deers_rocm_matmul_tune(ctypes.c_int(1 if on else 0)))


def empty_cache():
    _check(load().deers_rocm_empty_cache())


def profile_collect() -> dict:
    """{kernel name: (calls, total_ms)} for launches since profile_enable(True)."""
    n = ctypes.c_int()
    _check(load().deers_rocm_profile_collect(ctypes.byref(n)))
    out = {}
    for i in range(n.value):
        name, calls, ms = ctypes.c_char_p(), ctypes.c_int64(), ctypes.c_float()
        _check(load().deers_rocm_profile_row(ctypes.c_int(i), ctypes.byref(name),
                                             ctypes.byref(calls), ctypes.byref(ms)))
        out[name.value.decode()] = (int(calls.value), float(ms.value))
    return out


def _strides(s):
    if s is None:
        return None
    return (ctypes.c_int64 * 4)(*[int(x) for x in s])


def attn_fwd_raw(dtype, q, k, v, o, lse, B, H, T, D, scale, q_strides=None, k_strides=None,
                 v_strides=None, o_strides=None):
    """deers_rocm_attn_fwd on raw device pointers (DeviceBuffer.ptr)."""
    _check(load().deers_rocm_attn_fwd(
        ctypes.c_int(dtype_code(dtype)), q, _strides(q_strides), k, _strides(k_strides), v,
        _strides(v_strides), o, _strides(o_strides), lse, ctypes.c_int64(B), ctypes.c_int64(H),
        ctypes.c_int64(T), ctypes.c_int64(D), ctypes.c_float(scale)))


def attn_bwd_raw(dtype, q, k, v, o, lse, do, dq, dk, dv, B, H, T, D, scale, strides=None):
    """deers_rocm_attn_bwd on raw device pointers; `strides` maps tensor name -> 4 strides."""
    s = strides or {}
    g = lambda n: _strides(s.get(n))  # noqa: E731
    _check(load().deers_rocm_attn_bwd(
        ctypes.c_int(dtype_code(dtype)), q, g("q"), k, g("k"), v, g("v"), o, g("o"), lse, do,
        g("do"), dq, g("dq"), dk, g("dk"), dv, g("dv"), ctypes.c_int64(B), ctypes.c_int64(H),
        ctypes.c_int64(T), ctypes.c_int64(D), ctypes.c_float(scale)))


def attn_decode_raw(dtype, q, k_cache, v_cache, o, B, H, L, D, scale, kv_strides=None):
    ks = None if kv_strides is None else (ctypes.c_int64 * 3)(*[int(x) for x in kv_strides])
    _check(load().deers_rocm_attn_decode(
        ctypes.c_int(dtype_code(dtype)), q, k_cache, v_cache, ks, o, ctypes.c_int64(B),
        ctypes.c_int64(H), ctypes.c_int64(L), ctypes.c_int64(D), ctypes.c_float(scale)))


def attn_decode_noalloc_raw(dtype, q, k_cache, v_cache, o, B, H, L, D, scale, kv_strides=None):
    """deers_rocm_attn_decode_noalloc: attn_decode with the split partials in static device memory."""
    ks = None if kv_strides is None else (ctypes.c_int64 * 3)(*[int(x) for x in kv_strides])
    _check(load().deers_rocm_attn_decode_noalloc(
        ctypes.c_int(dtype_code(dtype)), q, k_cache, v_cache, ks, o, ctypes.c_int64(B),
        ctypes.c_int64(H), ctypes.c_int64(L), ctypes.c_int64(D), ctypes.c_float(scale)))


def attn_decode_append_raw(dtype, q, k, v, in_strides, cos_row, sin_row, k_cache, v_cache, cache_strides,
                           o, pos, capacity, B, H, D, scale):
    """deers_rocm_attn_decode_append: rotate q, k at `pos`, append k, v as cache row pos, attend over [0,pos]."""
    i64 = ctypes.c_int64
    _check(load().deers_rocm_attn_decode_append(
        ctypes.c_int(dtype_code(dtype)), q, k, v, (i64 * 2)(*[int(x) for x in in_strides]), cos_row,
        sin_row, k_cache, v_cache, (i64 * 3)(*[int(x) for x in cache_strides]), o, i64(pos),
        i64(capacity), i64(B), i64(H), i64(D), ctypes.c_float(scale)))


def fill_raw(dtype, dst, n, value):
    _check(load().deers_rocm_fill(ctypes.c_int(dtype_code(dtype)), dst, ctypes.c_size_t(n),
                                  ctypes.c_float(value)))


def add_raw(dtype, a, b, out, n):
    _check(load().deers_rocm_add(ctypes.c_int(dtype_code(dtype)), a, b, out, ctypes.c_size_t(n)))


def neg_raw(dtype, a, out, n):
    _check(load().deers_rocm_neg(ctypes.c_int(dtype_code(dtype)), a, out, ctypes.c_size_t(n)))


def copy_compact_raw(dtype, src, shape, strides, dst):
    """dst (compact over `shape`) <- src read through element `strides`."""
    nd = len(shape)
    sh = (ctypes.c_int64 * nd)(*[int(x) for x in shape])
    st = (ctypes.c_int64 * nd)(*[int(x) for x in strides])
    _check(load().deers_rocm_copy_compact(ctypes.c_int(dtype_code(dtype)), src, sh, st,
                                          ctypes.c_int(nd), dst))


def log_softmax_fwd_raw(dtype, x, out, outer, inner):
    _check(load().deers_rocm_log_softmax_fwd(ctypes.c_int(dtype_code(dtype)), x, out,
                                             ctypes.c_int64(outer), ctypes.c_int64(inner)))


def log_softmax_bwd_raw(dtype, grad, lsm, out, outer, inner):
    _check(load().deers_rocm_log_softmax_bwd(ctypes.c_int(dtype_code(dtype)), grad, lsm, out,
                                             ctypes.c_int64(outer), ctypes.c_int64(inner)))


def index_select_raw(dtype, table, indices, out, n_rows, n_indices, width):
    _check(load().deers_rocm_index_select(ctypes.c_int(dtype_code(dtype)), table, indices, out,
                                          ctypes.c_int64(n_rows), ctypes.c_int64(n_indices),
                                          ctypes.c_int64(width)))


def index_add_raw(dtype, src, indices, dst, n_rows, n_indices, width):
    _check(load().deers_rocm_index_add(ctypes.c_int(dtype_code(dtype)), src, indices, dst,
                                       ctypes.c_int64(n_rows), ctypes.c_int64(n_indices),
                                       ctypes.c_int64(width)))


def rms_norm_fwd_raw(dtype, x, y, outer, inner, eps):
    _check(load().deers_rocm_rms_norm_fwd(ctypes.c_int(dtype_code(dtype)), x, y, ctypes.c_int64(outer),
                                          ctypes.c_int64(inner), ctypes.c_double(eps)))


def rms_norm_bwd_raw(dtype, x, dy, dx, outer, inner, eps):
    _check(load().deers_rocm_rms_norm_bwd(ctypes.c_int(dtype_code(dtype)), x, dy, dx,
                                          ctypes.c_int64(outer), ctypes.c_int64(inner),
                                          ctypes.c_double(eps)))


def rms_norm_bwd_add_raw(dtype, x, dy, addend, dx, outer, inner, eps):
    _check(load().deers_rocm_rms_norm_bwd_add(ctypes.c_int(dtype_code(dtype)), x, dy, addend, dx,
                                              ctypes.c_int64(outer), ctypes.c_int64(inner),
                                              ctypes.c_double(eps)))


def relu_sq_fwd_raw(dtype, x, y, n):
    _check(load().deers_rocm_relu_sq_fwd(ctypes.c_int(dtype_code(dtype)), x, y, ctypes.c_int64(n)))


def relu_sq_bwd_raw(dtype, x, dy, dx, n):
    _check(load().deers_rocm_relu_sq_bwd(ctypes.c_int(dtype_code(dtype)), x, dy, dx, ctypes.c_int64(n)))


def argmax_rows_raw(dtype, x, out, outer, inner):
    _check(load().deers_rocm_argmax_rows(ctypes.c_int(dtype_code(dtype)), x, out, ctypes.c_int64(outer),
                                         ctypes.c_int64(inner)))


def cross_entropy_fwd_raw(dtype, logits, targets, row_lse, loss, n_rows, n_classes):
    _check(load().deers_rocm_cross_entropy_fwd(ctypes.c_int(dtype_code(dtype)), logits, targets, row_lse,
                                               loss, ctypes.c_int64(n_rows), ctypes.c_int64(n_classes)))


def cross_entropy_fwd_grad_raw(dtype, logits, targets, row_lse, loss, dlogits, n_rows, n_classes):
    _check(load().deers_rocm_cross_entropy_fwd_grad(ctypes.c_int(dtype_code(dtype)), logits, targets, row_lse,
                                                    loss, dlogits, ctypes.c_int64(n_rows),
                                                    ctypes.c_int64(n_classes)))


def scale_by_scalar_raw(dtype, x, n, factor):
    _check(load().deers_rocm_scale_by_scalar(ctypes.c_int(dtype_code(dtype)), x, ctypes.c_int64(n), factor))


def cross_entropy_bwd_raw(dtype, logits, targets, row_lse, upstream, dlogits, n_rows, n_classes):
    _check(load().deers_rocm_cross_entropy_bwd(ctypes.c_int(dtype_code(dtype)), logits, targets, row_lse,
                                               upstream, dlogits, ctypes.c_int64(n_rows),
                                               ctypes.c_int64(n_classes)))


# op codes of deers_rocm_unary / deers_rocm_binary / deers_rocm_reduce (include/deers_rocm.h)
UNARY_OPS = {"neg": 0, "exp": 1, "log": 2, "sin": 3, "cos": 4, "tanh": 5, "relu": 6,
             "relu_backward": 7, "scalar_add": 8, "scalar_mul": 9, "scalar_div": 10, "powf": 11}
BINARY_OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3, "pow": 4, "eq": 5}
REDUCE_OPS = {"sum": 0, "max": 1}
I64 = 2


def _i64_array(values):
    if values is None:
        return None
    return (ctypes.c_int64 * len(values))(*[int(x) for x in values])


def unary_raw(dtype, op, x, shape, strides, param, out):
    """out (compact over `shape`) = op(x read through element `strides`; None = compact)."""
    _check(load().deers_rocm_unary(ctypes.c_int(dtype_code(dtype)), ctypes.c_int(UNARY_OPS[op]), x,
                                   ctypes.c_int(len(shape)), _i64_array(shape), _i64_array(strides),
                                   ctypes.c_double(param), out))


def binary_raw(dtype, op, a, a_strides, b, b_strides, shape, out):
    _check(load().deers_rocm_binary(ctypes.c_int(dtype_code(dtype)), ctypes.c_int(BINARY_OPS[op]), a,
                                    _i64_array(a_strides), b, _i64_array(b_strides),
                                    ctypes.c_int(len(shape)), _i64_array(shape), out))


def reduce_raw(dtype, op, x, out, outer, reduce_size):
    _check(load().deers_rocm_reduce(ctypes.c_int(dtype_code(dtype)), ctypes.c_int(REDUCE_OPS[op]), x, out,
                                    ctypes.c_int64(outer), ctypes.c_int64(reduce_size)))


def log_sum_exp_raw(dtype, x, out, outer, reduce_size):
    _check(load().deers_rocm_log_sum_exp(ctypes.c_int(dtype_code(dtype)), x, out, ctypes.c_int64(outer),
                                         ctypes.c_int64(reduce_size)))


def gather_raw(dtype, src, indices, out, left, src_dim, index_len, right):
    code = I64 if np.dtype(dtype) == np.int64 else dtype_code(dtype)
    _check(load().deers_rocm_gather(ctypes.c_int(code), src, indices, out, ctypes.c_int64(left),
                                    ctypes.c_int64(src_dim), ctypes.c_int64(index_len),
                                    ctypes.c_int64(right)))


def scatter_add_raw(dtype, src, indices, dst, left, dst_dim, index_len, right):
    _check(load().deers_rocm_scatter_add(ctypes.c_int(dtype_code(dtype)), src, indices, dst,
                                         ctypes.c_int64(left), ctypes.c_int64(dst_dim),
                                         ctypes.c_int64(index_len), ctypes.c_int64(right)))


def adamw_step_raw(dtype, w, grad, m, v, n, lr, beta1, beta2, eps, weight_decay, step,
                   grad_scale=1.0):
    _check(load().deers_rocm_adamw_step(
        ctypes.c_int(dtype_code(dtype)), w, grad, m, v, ctypes.c_int64(n), ctypes.c_double(lr),
        ctypes.c_double(beta1), ctypes.c_double(beta2), ctypes.c_double(eps),
        ctypes.c_double(weight_decay), ctypes.c_int64(step), ctypes.c_double(grad_scale)))


def sum_squares_raw(dtype, x, n, total, accumulate=False):
    _check(load().deers_rocm_sum_squares(ctypes.c_int(dtype_code(dtype)), x, ctypes.c_int64(n),
                                         total, ctypes.c_int(1 if accumulate else 0)))


def _ptr_table(ptrs):
    return (ctypes.c_void_p * len(ptrs))(*[p.value if isinstance(p, ctypes.c_void_p) else p for p in ptrs])


def adamw_step_multi_raw(dtype, w, grad, m, v, sizes, lr, beta1, beta2, eps, weight_decay, step,
                         grad_scale=1.0):
    n = len(sizes)
    _check(load().deers_rocm_adamw_step_multi(
        ctypes.c_int(dtype_code(dtype)), ctypes.c_int(n), _ptr_table(w), _ptr_table(grad), _ptr_table(m),
        _ptr_table(v), (ctypes.c_int64 * n)(*sizes), ctypes.c_double(lr), ctypes.c_double(beta1),
        ctypes.c_double(beta2), ctypes.c_double(eps), ctypes.c_double(weight_decay), ctypes.c_int64(step),
        ctypes.c_double(grad_scale)))


def sum_squares_multi_raw(dtype, x, sizes, total, accumulate=False):
    n = len(sizes)
    _check(load().deers_rocm_sum_squares_multi(ctypes.c_int(dtype_code(dtype)), ctypes.c_int(n),
                                               _ptr_table(x), (ctypes.c_int64 * n)(*sizes), total,
                                               ctypes.c_int(1 if accumulate else 0)))


def scale_raw(dtype, x, n, scale):
    _check(load().deers_rocm_scale(ctypes.c_int(dtype_code(dtype)), x, ctypes.c_int64(n),
                                   ctypes.c_double(scale)))


def matmul_raw(dtype, a, a_strides, b, b_strides, c, batch, m, n, k):
    """deers_rocm_matmul: c[batch,m,n] = a @ b; strides are (row, col, batch) in elements."""
    i64 = ctypes.c_int64
    _check(load().deers_rocm_matmul(
        ctypes.c_int(dtype_code(dtype)), a, i64(a_strides[0]), i64(a_strides[1]), i64(a_strides[2]),
        b, i64(b_strides[0]), i64(b_strides[1]), i64(b_strides[2]), c, i64(batch), i64(m), i64(n),
        i64(k)))


def matmul_acc_raw(dtype, a, a_strides, b, b_strides, c, batch, m, n, k):
    """deers_rocm_matmul_acc: c[batch,m,n] += a @ b; strides are (row, col, batch) in elements."""
    i64 = ctypes.c_int64
    _check(load().deers_rocm_matmul_acc(
        ctypes.c_int(dtype_code(dtype)), a, i64(a_strides[0]), i64(a_strides[1]), i64(a_strides[2]),
        b, i64(b_strides[0]), i64(b_strides[1]), i64(b_strides[2]), c, i64(batch), i64(m), i64(n),
        i64(k)))


def matmul_add_raw(dtype, a, a_strides, b, b_strides, addend, c, batch, m, n, k):
    """deers_rocm_matmul_add: c[batch,m,n] = a @ b + addend; strides are (row, col, batch) in elements."""
    i64 = ctypes.c_int64
    _check(load().deers_rocm_matmul_add(
        ctypes.c_int(dtype_code(dtype)), a, i64(a_strides[0]), i64(a_strides[1]), i64(a_strides[2]),
        b, i64(b_strides[0]), i64(b_strides[1]), i64(b_strides[2]), addend, c, i64(batch), i64(m), i64(n),
        i64(k)))


LINEAR_PROLOGUES = {"plain": 0, "rms_norm": 1, "relu_sq": 2}
LINEAR_W_PACKED = -32  # DEERS_ROCM_LINEAR_W_PACKED: pass as ldw for a [n/32][k][32] weight


def decode_linear_raw(dtype, prologue, eps, x, ldx, w, ldw, y, accumulate, m, n, k):
    """deers_rocm_decode_linear: y[m,n] (+)= f(x)[m,k] @ w[k,n], m <= 32, f one of LINEAR_PROLOGUES."""
    i64 = ctypes.c_int64
    _check(load().deers_rocm_decode_linear(
        ctypes.c_int(dtype_code(dtype)), ctypes.c_int(LINEAR_PROLOGUES[prologue]), ctypes.c_float(eps), x,
        i64(ldx), w, i64(ldw), y, ctypes.c_int(1 if accumulate else 0), i64(m), i64(n), i64(k)))


def decode_linear_hint_raw(next_w_packed, n, k):
    """deers_rocm_decode_linear_hint: the packed weight of the product after the next one (None clears)."""
    _check(load().deers_rocm_decode_linear_hint(next_w_packed, ctypes.c_int64(n), ctypes.c_int64(k)))


def decode_qkv_raw(dtype, q, k, v, in_strides, cos_row, sin_row, q_out, k_cache, v_cache, cache_strides,
                   pos, capacity, B, H, D):
    """deers_rocm_decode_qkv: rotate q, k at `pos`; q -> q_out [B,H,D]; k, v -> row pos of the caches."""
    i64 = ctypes.c_int64
    _check(load().deers_rocm_decode_qkv(
        ctypes.c_int(dtype_code(dtype)), q, k, v, (i64 * 2)(*[int(x) for x in in_strides]), cos_row,
        sin_row, q_out, k_cache, v_cache, (i64 * 3)(*[int(x) for x in cache_strides]), i64(pos),
        i64(capacity), i64(B), i64(H), i64(D)))


def rope_fwd_raw(dtype, x, cos, sin, y, B, T, H, D, x_strides=None, y_strides=None):
    """deers_rocm_rope_fwd: x logical [B,T,H,D] -> y [B,H,T,D] (compact unless y_strides)."""
    _check(load().deers_rocm_rope_fwd(
        ctypes.c_int(dtype_code(dtype)), x, _strides(x_strides), cos, sin, y, _strides(y_strides),
        ctypes.c_int64(B), ctypes.c_int64(T), ctypes.c_int64(H), ctypes.c_int64(D)))


def copy_view_raw(dtype, src, src_strides, dst, dst_strides, shape):
    nd = len(shape)
    arr = lambda v: (ctypes.c_int64 * nd)(*[int(x) for x in v])  # noqa: E731
    _check(load().deers_rocm_copy_view(ctypes.c_int(dtype_code(dtype)), src, arr(src_strides), dst,
                                       arr(dst_strides), arr(shape), ctypes.c_int(nd)))


def rope_bwd_raw(dtype, dy, cos, sin, dx, B, T, H, D, dy_strides=None):
    """deers_rocm_rope_bwd: dy logical [B,H,T,D] -> dx compact [B,T,H,D]."""
    _check(load().deers_rocm_rope_bwd(
        ctypes.c_int(dtype_code(dtype)), dy, _strides(dy_strides), cos, sin, dx, ctypes.c_int64(B),
        ctypes.c_int64(T), ctypes.c_int64(H), ctypes.c_int64(D)))


def default_scale(D: int) -> float:
    """1/sqrt(D) in double, narrowed to f32 (src/models/gpt.rs:139, src/storage.rs:115-117)."""
    return float(np.float32(1.0 / np.sqrt(float(D))))


# ---- numpy-in / numpy-out conveniences (copy to the device, run, copy back) ----

def attn_fwd(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float | None = None):
    """Returns (o, lse) for compact [B,H,T,D] numpy inputs of one dtype (f16 or f32)."""
    B, H, T, D = q.shape
    scale = default_scale(D) if scale is None else scale
    dq_, dk_, dv_ = (DeviceBuffer.from_numpy(a) for a in (q, k, v))
    o = DeviceBuffer(q.shape, q.dtype)
    lse = DeviceBuffer((B, H, T), np.float32)
    attn_fwd_raw(q.dtype, dq_.ptr, dk_.ptr, dv_.ptr, o.ptr, lse.ptr, B, H, T, D, scale)
    return o.numpy(), lse.numpy()


def attn_fwd_composed_raw(dtype, q, k, v, mask, o, lse, s, p, B, H, T, D, scale):
    """The reference's own op chain for the attention core (src/models/gpt.rs:139-144,
    softmax of src/tensor.rs:456-458) on the device, one storage kernel per tensor op:
    matmul, scalar_mul, add of the [B,1,T,T] mask broadcast over the heads, log_sum_exp,
    sub of the [B,H,T,1] statistic broadcast over the keys, exp, matmul.  What a
    Device::Rocm backend executes where the fused op does not apply (any head width).
    `s`, `p`: two [B,H,T,T] scratch buffers of `dtype`; `lse`: [B,H,T] of `dtype`."""
    BH, shape = B * H, (B, H, T, T)
    matmul_raw(dtype, q, (D, 1, T * D), k, (1, D, T * D), s, BH, T, T, D)            # q @ k^T
    unary_raw(dtype, "scalar_mul", s, shape, None, scale, p)                          # * scale
    binary_raw(dtype, "add", p, None, mask, [T * T, 0, T, 1], shape, s)               # + mask
    log_sum_exp_raw(dtype, s, lse, BH * T, T)
    binary_raw(dtype, "sub", s, None, lse, [H * T, T, 1, 0], shape, p)                # - lse
    unary_raw(dtype, "exp", p, shape, None, 0.0, s)
    matmul_raw(dtype, s, (T, 1, T * T), v, (D, 1, T * D), o, BH, T, D, T)             # @ v


def causal_mask_host(B: int, T: int, dtype) -> np.ndarray:
    """Additive mask [B,1,T,T]: -inf above the diagonal, as src/nn/functional.rs:12-55 builds it
    on the host before every forward."""
    m = np.where(np.triu(np.ones((T, T), bool), 1), -np.inf, 0.0).astype(dtype)
    return np.ascontiguousarray(np.broadcast_to(m, (B, 1, T, T)))


def attn_fwd_composed(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float | None = None):
    """Returns (o, lse) computed by the unfused chain; compact [B,H,T,D] inputs of one dtype."""
    B, H, T, D = q.shape
    scale = default_scale(D) if scale is None else scale
    bq, bk, bv = (DeviceBuffer.from_numpy(a) for a in (q, k, v))
    mask = DeviceBuffer.from_numpy(causal_mask_host(B, T, q.dtype))
    o = DeviceBuffer(q.shape, q.dtype)
    lse = DeviceBuffer((B, H, T), q.dtype)
    s, p = DeviceBuffer((B, H, T, T), q.dtype), DeviceBuffer((B, H, T, T), q.dtype)
    attn_fwd_composed_raw(q.dtype, bq.ptr, bk.ptr, bv.ptr, mask.ptr, o.ptr, lse.ptr, s.ptr, p.ptr,
                          B, H, T, D, scale)
    return o.numpy(), lse.numpy()


def attn_fwd_bwd(q, k, v, do, scale: float | None = None):
    """Returns (o, lse, dq, dk, dv): forward then backward through the C ABI."""
    B, H, T, D = q.shape
    scale = default_scale(D) if scale is None else scale
    bq, bk, bv, bdo = (DeviceBuffer.from_numpy(a) for a in (q, k, v, do))
    o = DeviceBuffer(q.shape, q.dtype)
    lse = DeviceBuffer((B, H, T), np.float32)
    gq, gk, gv = (DeviceBuffer(q.shape, q.dtype) for _ in range(3))
    attn_fwd_raw(q.dtype, bq.ptr, bk.ptr, bv.ptr, o.ptr, lse.ptr, B, H, T, D, scale)
    attn_bwd_raw(q.dtype, bq.ptr, bk.ptr, bv.ptr, o.ptr, lse.ptr, bdo.ptr, gq.ptr, gk.ptr, gv.ptr,
                 B, H, T, D, scale)
    return o.numpy(), lse.numpy(), gq.numpy(), gk.numpy(), gv.numpy()


def attn_decode(q: np.ndarray, k_cache: np.ndarray, v_cache: np.ndarray,
                scale: float | None = None, length: int | None = None):
    """q [B,H,D], caches [B,H,Lcap,D] (f16); attends to the first `length` cache rows."""
    B, H, D = q.shape
    Lcap = k_cache.shape[2]
    L = Lcap if length is None else length
    scale = default_scale(D) if scale is None else scale
    bq, bk, bv = (DeviceBuffer.from_numpy(a) for a in (q, k_cache, v_cache))
    o = DeviceBuffer((B, H, D), q.dtype)
    attn_decode_raw(q.dtype, bq.ptr, bk.ptr, bv.ptr, o.ptr, B, H, L, D, scale,
                    kv_strides=(H * Lcap * D, Lcap * D, D))
    return o.numpy()
