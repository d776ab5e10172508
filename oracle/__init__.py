"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE, not product code).

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import
this package; the shipped library never does.  The arithmetic lives in
``attention_ref.cc`` (a restatement of the reference's CPU attention,
src/models/gpt.rs:139-144 and its autograd backward); this module moves numpy
arrays across the C boundary and restates the rotary embedding around the core
(src/models/gpt.rs:12-73), the loss's row-wise log-softmax
(src/storage/cpu.rs:793-888) and the AdamW step with gradient clipping
(src/optim.rs:214-296) directly in numpy.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile liboracle.so with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_max_threads.restype = ctypes.c_int
    return _lib


def max_threads() -> int:
    return int(lib().oracle_max_threads())


_I64 = ctypes.c_int64


def _suffix(dtype) -> str:
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(f"oracle supports float32/float64 arrays, got {dtype}")


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def causal_mask(batch: int, tgt_len: int, seqlen_offset: int, dtype=np.float32) -> np.ndarray:
    """Additive mask [batch,1,tgt,tgt+offset] (src/nn/functional.rs:12-55)."""
    out = np.empty((batch, 1, tgt_len, tgt_len + seqlen_offset), dtype=dtype)
    getattr(lib(), f"oracle_causal_mask_{_suffix(dtype)}")(
        _I64(batch), _I64(tgt_len), _I64(seqlen_offset), _ptr(out))
    return out


def matmul(a: np.ndarray, b: np.ndarray, nthreads: int = 1) -> np.ndarray:
    """Batched matmul of two equal-rank arrays; views (transposes) are passed by stride,
    the way the reference's CPU backend consumes them (src/storage/cpu.rs:688-753)."""
    assert a.dtype == b.dtype and a.ndim == b.ndim >= 2
    suf = _suffix(a.dtype)
    m, k = a.shape[-2:]
    k2, n = b.shape[-2:]
    assert k == k2 and a.shape[:-2] == b.shape[:-2]
    batch_shape = a.shape[:-2]
    batch = int(np.prod(batch_shape)) if batch_shape else 1
    # Flatten the batch dims.  numpy keeps the last-two-dims strides when the batch
    # dims collapse without a copy; otherwise it copies (same values, compact strides).
    def prep(x):
        if x.ndim == 2:
            return x, 0
        x3 = x.reshape((batch,) + x.shape[-2:])
        return x3, x3.strides[0] // x3.itemsize
    a3, a_bs = prep(a)
    b3, b_bs = prep(b)
    isz = a.itemsize
    out = np.empty(batch_shape + (m, n), dtype=a.dtype)
    getattr(lib(), f"oracle_matmul_{suf}")(
        _ptr(a3), _I64(a_bs), _I64(a3.strides[-2] // isz), _I64(a3.strides[-1] // isz),
        _ptr(b3), _I64(b_bs), _I64(b3.strides[-2] // isz), _I64(b3.strides[-1] // isz),
        _ptr(out), _I64(batch), _I64(m), _I64(n), _I64(k), ctypes.c_int(nthreads))
    return out


def scalar_mul(x: np.ndarray, s: float) -> np.ndarray:
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    getattr(lib(), f"oracle_scalar_mul_{_suffix(x.dtype)}")(
        _ptr(x), _I64(x.size), ctypes.c_double(s), _ptr(out))
    return out


def log_sum_exp(x: np.ndarray) -> np.ndarray:
    """Row-wise log-sum-exp over the last axis (src/storage/cpu.rs:755-771)."""
    x = np.ascontiguousarray(x)
    cols = x.shape[-1]
    rows = x.size // cols
    out = np.empty(x.shape[:-1], dtype=x.dtype)
    getattr(lib(), f"oracle_log_sum_exp_{_suffix(x.dtype)}")(
        _ptr(x), _I64(rows), _I64(cols), _ptr(out))
    return out


def softmax(x: np.ndarray) -> np.ndarray:
    """exp(x - lse(x)) over the last axis (src/tensor.rs:408-425, 456-458)."""
    x = np.ascontiguousarray(x)
    cols = x.shape[-1]
    out = np.empty_like(x)
    getattr(lib(), f"oracle_softmax_{_suffix(x.dtype)}")(
        _ptr(x), _I64(x.size // cols), _I64(cols), _ptr(out))
    return out


def attn_fwd(q, k, v, scale: float | None = None, dtype=np.float32, nthreads: int = 0,
             return_lse: bool = False, return_attn: bool = False, heads_per_call: int = 0):
    """softmax(q k^T * scale + causal_mask) v for q [B,H,Tq,D], k,v [B,H,Tk,D].

    Inputs are converted to ``dtype`` (float32 follows the reference's f32 path;
    f16 configurations pass the f16-rounded values here).  ``scale`` defaults to
    1/sqrt(D) computed in double (src/models/gpt.rs:139).  ``heads_per_call`` bounds
    memory by evaluating that many batch entries at a time (0 = everything at
    once, the way the reference materialises it).
    """
    q, k, v = _c(q, dtype), _c(k, dtype), _c(v, dtype)
    B, H, tq, D = q.shape
    tk = k.shape[2]
    assert k.shape == (B, H, tk, D) and v.shape == (B, H, tk, D) and tk >= tq
    if scale is None:
        scale = 1.0 / np.sqrt(float(D))
    y = np.empty((B, H, tq, D), dtype=dtype)
    lse = np.empty((B, H, tq), dtype=dtype) if return_lse else None
    attn = np.empty((B, H, tq, tk), dtype=dtype) if return_attn else None
    fn = getattr(lib(), f"oracle_attn_fwd_{_suffix(dtype)}")
    step = heads_per_call if heads_per_call > 0 else B
    for b0 in range(0, B, step):
        b1 = min(B, b0 + step)
        fn(_ptr(q[b0:b1]), _ptr(k[b0:b1]), _ptr(v[b0:b1]), _I64(b1 - b0), _I64(H), _I64(tq),
           _I64(tk), _I64(D), ctypes.c_double(scale), _ptr(y[b0:b1]),
           _ptr(lse[b0:b1]) if lse is not None else None,
           _ptr(attn[b0:b1]) if attn is not None else None, ctypes.c_int(nthreads))
    res = (y,)
    if return_lse:
        res += (lse,)
    if return_attn:
        res += (attn,)
    return res if len(res) > 1 else y


def attn_bwd(q, k, v, dy, scale: float | None = None, dtype=np.float32, nthreads: int = 0,
             heads_per_call: int = 0):
    """Gradients (dq, dk, dv) of attn_fwd for upstream gradient dy [B,H,Tq,D]."""
    q, k, v, dy = _c(q, dtype), _c(k, dtype), _c(v, dtype), _c(dy, dtype)
    B, H, tq, D = q.shape
    tk = k.shape[2]
    if scale is None:
        scale = 1.0 / np.sqrt(float(D))
    dq, dk, dv = np.empty_like(q), np.empty_like(k), np.empty_like(v)
    fn = getattr(lib(), f"oracle_attn_bwd_{_suffix(dtype)}")
    step = heads_per_call if heads_per_call > 0 else B
    for b0 in range(0, B, step):
        b1 = min(B, b0 + step)
        fn(_ptr(q[b0:b1]), _ptr(k[b0:b1]), _ptr(v[b0:b1]), _ptr(dy[b0:b1]), _I64(b1 - b0),
           _I64(H), _I64(tq), _I64(tk), _I64(D), ctypes.c_double(scale), _ptr(dq[b0:b1]),
           _ptr(dk[b0:b1]), _ptr(dv[b0:b1]), ctypes.c_int(nthreads))
    return dq, dk, dv


# ---- rotary embedding (numpy restatement; byte/float arithmetic in the reference's order) ----

def rope_tables(seq_len: int, head_dim: int, base: float = 10000.0, dtype=np.float32):
    """cos, sin [seq_len, head_dim/2] as precompute_rotary_embeddings builds them
    (src/models/gpt.rs:12-47): inv_freq_i = 1 / base^(2i/D) in f32, angle = t * inv_freq
    in f32, cos/sin in f32, then cast to `dtype`."""
    assert head_dim % 2 == 0, "RoPE requires an even head dimension"
    half = head_dim // 2
    channel = (2 * np.arange(half)).astype(np.float32)
    inv_freq = (np.float32(1.0) / np.power(np.float32(base), channel / np.float32(head_dim))
                ).astype(np.float32)
    t = np.arange(seq_len, dtype=np.float32)[:, None]
    freqs = (t * inv_freq[None, :]).astype(np.float32)
    return np.cos(freqs).astype(dtype), np.sin(freqs).astype(dtype)


def rope_apply(x: np.ndarray, cos: np.ndarray, sin: np.ndarray, dtype=np.float32) -> np.ndarray:
    """apply_rotary_emb on x [B,T,H,D] (src/models/gpt.rs:49-73):
    y1 = x1*cos + x2*sin, y2 = x1*(sin*-1) + x2*cos, cat along D; evaluated in `dtype`
    (float32 for the f32 path and as the oracle of the f16 path on rounded inputs)."""
    x = np.asarray(x, dtype=dtype)
    half = x.shape[3] // 2
    c = np.asarray(cos, dtype=dtype)[None, :, None, :]
    s = np.asarray(sin, dtype=dtype)[None, :, None, :]
    x1, x2 = x[..., :half], x[..., half:]
    y1 = x1 * c + x2 * s
    y2 = x1 * (s * dtype(-1.0)) + x2 * c
    return np.concatenate([y1, y2], axis=3)


def rope_apply_bwd(dy: np.ndarray, cos: np.ndarray, sin: np.ndarray, dtype=np.float32) -> np.ndarray:
    """Gradient of rope_apply w.r.t. x for upstream dy [B,T,H,D], from the backward
    bodies of cat / add / mul (src/ops.rs:130-260): dx1 = dy1*cos + dy2*(-sin),
    dx2 = dy1*sin + dy2*cos."""
    dy = np.asarray(dy, dtype=dtype)
    half = dy.shape[3] // 2
    c = np.asarray(cos, dtype=dtype)[None, :, None, :]
    s = np.asarray(sin, dtype=dtype)[None, :, None, :]
    d1, d2 = dy[..., :half], dy[..., half:]
    return np.concatenate([d1 * c + d2 * (s * dtype(-1.0)), d1 * s + d2 * c], axis=3)


# ---- row-wise log-softmax (numpy restatement) ----

def _lsm_compute_type(dtype):
    # f16 and f32 rows accumulate in f32 as the reference does; float64 is accepted so
    # that tests can difference the same formula without rounding noise.
    return np.float64 if np.dtype(dtype) == np.float64 else np.float32


def log_softmax_fwd(x: np.ndarray, dtype=np.float32) -> np.ndarray:
    """log_softmax_fwd over the last axis of compact [outer, inner] data
    (src/storage/cpu.rs:793-840): per row max, sum of exp(x - max) in f32,
    lse = ln(sum) + max, out = x - lse; f16 rows convert each element to f32 and round
    the result once."""
    ct = _lsm_compute_type(dtype)
    xf = np.asarray(x, dtype=dtype).astype(ct)
    mx = xf.max(axis=-1, keepdims=True)
    s = np.exp(xf - mx, dtype=ct).sum(axis=-1, keepdims=True, dtype=ct)
    lse = np.log(s, dtype=ct) + mx
    return (xf - lse).astype(dtype)


def log_softmax_bwd(grad: np.ndarray, lsm: np.ndarray, dtype=np.float32) -> np.ndarray:
    """log_softmax_bwd (src/storage/cpu.rs:842-888): per row s = sum(grad) in f32,
    out = grad - exp(lsm) * s."""
    ct = _lsm_compute_type(dtype)
    g = np.asarray(grad, dtype=dtype).astype(ct)
    l = np.asarray(lsm, dtype=dtype).astype(ct)
    s = g.sum(axis=-1, keepdims=True, dtype=ct)
    return (g - np.exp(l, dtype=ct) * s).astype(dtype)


# ---- optimizer step (numpy restatement; every tensor op rounds to the tensor's dtype) ----

def _powi(a: float, b: int) -> float:
    """f64 power by repeated squaring, what Rust's f64::powi lowers to."""
    recip = b < 0
    b = abs(b)
    r = 1.0
    while True:
        if b & 1:
            r *= a
        b //= 2
        if b == 0:
            break
        a *= a
    return 1.0 / r if recip else r


def _scalar(x: float, dtype):
    """A host f64 scalar as storage::ScalarMul / ScalarAdd see it (src/storage.rs:108-123):
    cast to f32, then for f16 tensors to f16."""
    return np.dtype(dtype).type(np.float32(x))


def adamw_step(w, g, m, v, step: int, lr: float, betas=(0.9, 0.999), eps: float = 1e-8,
               weight_decay: float = 0.0, dtype=np.float32):
    """One AdamW::step_with_grads body for one parameter (src/optim.rs:214-251) as the
    same chain of element-wise ops, each rounding to `dtype`; `step` is the count after
    the increment at line 215.  Returns the new (w, m, v)."""
    T = np.dtype(dtype).type
    w, g, m, v = (np.asarray(a, dtype=dtype) for a in (w, g, m, v))
    beta1, beta2 = betas
    bc1 = 1.0 - _powi(beta1, step)
    bc2 = 1.0 - _powi(beta2, step)
    S = lambda x: _scalar(x, dtype)
    with np.errstate(all="ignore"):
        m = (m * S(beta1)).astype(T) + (g * S(1.0 - beta1)).astype(T)
        v = (v * S(beta2)).astype(T) + ((g * g).astype(T) * S(1.0 - beta2)).astype(T)
        m_hat = m * S(1.0 / bc1)
        v_hat = v * S(1.0 / bc2)
        decayed = w * S(1.0 - lr * weight_decay) if weight_decay > 0.0 else w
        update = m_hat / (np.sqrt(v_hat) + S(eps))
        w = decayed - update * S(lr)
    return w.astype(T), m.astype(T), v.astype(T)


def clip_grad_norm(grads, max_norm: float, dtype=np.float32):
    """clip_grad_norm (src/optim.rs:258-296) over a list of gradient arrays: returns
    (norm before clipping as f32, the list of possibly rescaled gradients)."""
    assert max_norm > 0.0, "max_norm must be positive"
    T = np.dtype(dtype).type
    if not grads:
        return np.float32(0.0), []
    grads = [np.asarray(g, dtype=dtype) for g in grads]
    total = T(0.0)
    with np.errstate(all="ignore"):
        for g in grads:
            total = T(total + (g * g).astype(T).sum(dtype=T))
        norm = np.float32(np.sqrt(total))
    if not np.isfinite(norm) or norm <= np.float32(max_norm):
        return norm, grads
    scale = max_norm / (float(norm) + 1e-6)
    return norm, [(g * _scalar(scale, dtype)).astype(T) for g in grads]


# ---- the other ops of a GPT training step (numpy restatements) ----

def index_select(table: np.ndarray, indices: np.ndarray) -> np.ndarray:
    """index_select along dim 0 (src/storage/cpu.rs:555-610, 936-952): rows of `table`
    picked by `indices`; an index out of range is an error there and here."""
    indices = np.asarray(indices, dtype=np.int64)
    if indices.size and (indices.min() < 0 or indices.max() >= table.shape[0]):
        raise IndexError("index_select: index out of bounds")
    return np.ascontiguousarray(table[indices])


def index_add(n_rows: int, src: np.ndarray, indices: np.ndarray) -> np.ndarray:
    """index_add along dim 0 into zeros [n_rows, width] (src/storage/cpu.rs:612-660,
    954-975): out[indices[i]] += src[i] for i ascending, each `+=` in the storage type."""
    indices = np.asarray(indices, dtype=np.int64)
    if indices.size and (indices.min() < 0 or indices.max() >= n_rows):
        raise IndexError("index_add: index out of bounds")
    out = np.zeros((n_rows,) + src.shape[1:], dtype=src.dtype)
    for i, r in enumerate(indices):  # the reference's loop order
        out[r] = out[r] + src[i]
    return out


def rms_norm_fwd(x: np.ndarray, eps: float, dtype=np.float32) -> np.ndarray:
    """RMSNorm::forward (src/nn.rs:244-251) as its chain of ops in `dtype`:
    mean_sq = sum(x*x, last) * (1/n); inv = (mean_sq + eps)^-0.5; y = x * inv."""
    T = np.dtype(dtype).type
    x = np.asarray(x, dtype=dtype)
    n = x.shape[-1]
    sq = (x * x).astype(T)
    mean_sq = (sq.sum(axis=-1, keepdims=True, dtype=T) * _scalar_any(1.0 / n, dtype)).astype(T)
    inv = np.power((mean_sq + _scalar_any(eps, dtype)).astype(T), T(-0.5)).astype(T)
    return (x * inv).astype(T)


def rms_norm_bwd(x: np.ndarray, dy: np.ndarray, eps: float, dtype=np.float32) -> np.ndarray:
    """Gradient of rms_norm_fwd w.r.t. x, what the reference's autograd yields through
    mul / scalar_powf / scalar_add / mean / mul (src/ops.rs): with inv as above,
    dx = dy*inv - x * inv^3 * sum(dy*x, last) / n."""
    T = np.dtype(dtype).type
    x = np.asarray(x, dtype=dtype)
    dy = np.asarray(dy, dtype=dtype)
    n = x.shape[-1]
    inv = np.power((x * x).sum(axis=-1, keepdims=True, dtype=T) / T(n) + T(eps), T(-0.5))
    dot = (dy * x).sum(axis=-1, keepdims=True, dtype=T)
    return (dy * inv - x * (inv ** 3) * dot / T(n)).astype(T)


def _scalar_any(x: float, dtype):
    """Like _scalar, but passes float64 through for finite-difference checks."""
    return np.float64(x) if np.dtype(dtype) == np.float64 else _scalar(x, dtype)


def relu_sq_fwd(x: np.ndarray) -> np.ndarray:
    """`y.relu(); &y * &y` (src/models/gpt.rs:196-197; Relu at src/storage.rs:77-88)."""
    r = np.maximum(x, x.dtype.type(0))
    return (r * r).astype(x.dtype)


def relu_sq_bwd(x: np.ndarray, dy: np.ndarray) -> np.ndarray:
    """Backward of relu_sq_fwd through EWiseMul (both operands are r = relu(x): the two
    contributions dy*r are accumulated) and Relu (mask x > 0, src/storage.rs:90-102)."""
    r = np.maximum(x, x.dtype.type(0))
    g = (dy * r).astype(x.dtype)
    return ((g + g) * (x > 0)).astype(x.dtype)


def cross_entropy_fwd(logits: np.ndarray, targets: np.ndarray, dtype=np.float32):
    """loss::cross_entropy (src/loss.rs:11-24): log_softmax(1), gather the target column,
    sum, times -1/N.  Returns the scalar loss in `dtype`."""
    T = np.dtype(dtype).type
    lsm = log_softmax_fwd(logits, dtype=dtype)
    targets = np.asarray(targets, dtype=np.int64)
    n = lsm.shape[0]
    picked = lsm[np.arange(n), targets]
    return T(picked.sum(dtype=T) * _scalar_any(-1.0 / n, dtype))


def cross_entropy_bwd(logits: np.ndarray, targets: np.ndarray, upstream: float = 1.0,
                      dtype=np.float32) -> np.ndarray:
    """Gradient of cross_entropy_fwd w.r.t. the logits through ScalarMul, Sum, Gather
    (scatter of the upstream gradient into zeros) and log_softmax_bwd."""
    T = np.dtype(dtype).type
    lsm = log_softmax_fwd(logits, dtype=dtype)
    n = lsm.shape[0]
    g = np.zeros_like(lsm)
    g[np.arange(n), np.asarray(targets, dtype=np.int64)] = T(upstream) * _scalar_any(-1.0 / n, dtype)
    return log_softmax_bwd(g, lsm, dtype=dtype)
