"""CPU restatement of the reference's generic storage kernels (TEST INFRASTRUCTURE).

Only tests and the smoke check import this module; the shipped library never does.
Each function follows the reference's CPU backend operation by operation, in its
element order and with its roundings:

  unary / ewise_powf   src/storage.rs:32-123, src/storage/cpu.rs:203-265
  binary               src/storage.rs:126-190, src/storage/cpu.rs:267-321
  reduce               src/storage/cpu.rs:323-357 (left to right, accumulator of the storage type)
  log_sum_exp          src/storage/cpu.rs:755-791
  gather               src/storage/cpu.rs:398-462, 891-912
  scatter_add          src/storage/cpu.rs:464-553, 914-934
  cat                  src/storage/cpu.rs:47-90

Pinned in tests/test_oracle_storage.py by the literal inputs of the reference's own tests
(tests/tensor.rs:515-538, 625-648, 1885-1909, 2226-2257) evaluated with numpy / scipy /
torch library routines, by closed forms and by brute force on small shapes.
"""
from __future__ import annotations

import numpy as np

UNARY = ("neg", "exp", "log", "sin", "cos", "tanh", "relu", "relu_backward", "scalar_add",
         "scalar_mul", "scalar_div", "powf")
BINARY = ("add", "sub", "mul", "div", "pow", "eq")


def _f32(x):
    return np.asarray(x).astype(np.float32)


def unary(op: str, x: np.ndarray, param: float = 0.0) -> np.ndarray:
    """UnaryOp::f32 / ::f16 applied element-wise (src/storage.rs:32-123); output compact, dtype of x.

    f16: convert to f32, operate, convert back (the unary_op! macro); a scalar is cast
    f64 -> f32 -> f16 first (scalar_op! macro), the exponent of powf f64 -> f32 only
    (src/storage/cpu.rs:203-235).
    """
    dt = x.dtype
    v = _f32(np.ascontiguousarray(x))
    with np.errstate(all="ignore"):
        if op == "neg":
            r = -v
        elif op == "exp":
            r = np.exp(v)
        elif op == "log":
            r = np.log(v)
        elif op == "sin":
            r = np.sin(v)
        elif op == "cos":
            r = np.cos(v)
        elif op == "tanh":
            r = np.tanh(v)
        elif op == "relu":
            r = np.fmax(v, np.float32(0))  # f32::max ignores a NaN operand
        elif op == "relu_backward":
            r = (v > 0).astype(np.float32)
        elif op in ("scalar_add", "scalar_mul", "scalar_div"):
            s = np.float32(param)
            if dt == np.float16:
                s = np.float32(np.float16(s))
            r = v + s if op == "scalar_add" else v * s if op == "scalar_mul" else v / s
        elif op == "powf":
            r = np.power(v, np.float32(param))
        else:
            raise ValueError(op)
    with np.errstate(over="ignore"):
        return r.astype(np.float32).astype(dt)


def binary(op: str, a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """BinaryOp::f32 / ::f16 (src/storage.rs:126-190) over two views of one shape; output compact."""
    assert a.shape == b.shape and a.dtype == b.dtype
    dt = a.dtype
    x, y = _f32(a), _f32(b)
    with np.errstate(all="ignore"):
        if op == "add":
            r = x + y
        elif op == "sub":
            r = x - y
        elif op == "mul":
            r = x * y
        elif op == "div":
            r = x / y
        elif op == "pow":
            r = np.power(x, y)
        elif op == "eq":
            r = (x == y).astype(np.float32)
        else:
            raise ValueError(op)
    with np.errstate(over="ignore"):
        return np.ascontiguousarray(r.astype(np.float32).astype(dt))


def reduce(op: str, x: np.ndarray) -> np.ndarray:
    """x: [outer, reduce_size] compact; each row folded left to right with an accumulator of
    the storage type (`chunk.iter().copied().reduce(O::f16 | O::f32)`, src/storage/cpu.rs:337-346)."""
    dt = x.dtype
    acc = x[:, 0].copy()
    with np.errstate(all="ignore"):
        for i in range(1, x.shape[1]):
            if op == "sum":
                acc = (acc.astype(np.float32) + x[:, i].astype(np.float32)).astype(dt)
            elif op == "max":
                acc = np.fmax(acc, x[:, i])  # f32::max / f16::max ignore a NaN operand
            else:
                raise ValueError(op)
    return acc


def log_sum_exp(x: np.ndarray) -> np.ndarray:
    """x: [outer, reduce_size]; max = fold(-inf, f32::max), sum of exp(x - max) left to right in
    f32, ln(sum) + max, rounded to the storage type (src/storage/cpu.rs:755-791)."""
    dt = x.dtype
    v = _f32(x)
    with np.errstate(all="ignore"):
        mx = np.fmax.reduce(v, axis=1, initial=-np.inf).astype(np.float32)
        s = np.zeros(v.shape[0], np.float32)
        for i in range(v.shape[1]):
            s = (s + np.exp(v[:, i] - mx).astype(np.float32)).astype(np.float32)
        r = (np.log(s).astype(np.float32) + mx).astype(np.float32)
    return r.astype(dt)


def gather(src: np.ndarray, dim: int, indices: np.ndarray) -> np.ndarray:
    """out[l, i, r] = src[l, indices[l, i, r], r] (gather_into, src/storage/cpu.rs:891-912)."""
    left = int(np.prod(indices.shape[:dim], dtype=np.int64))
    right = int(np.prod(indices.shape[dim + 1:], dtype=np.int64))
    s = np.ascontiguousarray(src).reshape(left, src.shape[dim], right)
    ix = np.ascontiguousarray(indices).reshape(left, indices.shape[dim], right)
    out = np.empty(ix.shape, src.dtype)
    for i in range(ix.shape[1]):
        k = ix[:, i, :]
        out[:, i, :] = s[np.arange(left)[:, None], k, np.arange(right)[None, :]]
    return out.reshape(indices.shape)


def scatter_add(src: np.ndarray, dim: int, indices: np.ndarray, dst_shape) -> np.ndarray:
    """dst zero-initialised; dst[l, indices[l, i, r], r] += src[l, i, r] in the order l, i, r with
    the storage type's addition (scatter_add_into, src/storage/cpu.rs:914-934)."""
    left = int(np.prod(indices.shape[:dim], dtype=np.int64))
    right = int(np.prod(indices.shape[dim + 1:], dtype=np.int64))
    s = np.ascontiguousarray(src).reshape(left, indices.shape[dim], right)
    ix = np.ascontiguousarray(indices).reshape(left, indices.shape[dim], right)
    out = np.zeros((left, int(dst_shape[dim]), right), src.dtype)
    li, ri = np.arange(left)[:, None], np.arange(right)[None, :]
    for i in range(ix.shape[1]):  # within one i the (l, r) targets are distinct
        k = ix[:, i, :]
        cur = out[li, k, ri].astype(np.float32)
        out[li, k, ri] = (cur + s[:, i, :].astype(np.float32)).astype(src.dtype)
    return out.reshape(tuple(dst_shape))


def cat(parts) -> np.ndarray:
    """Compact buffers one after the other (CpuStorage::cat, src/storage/cpu.rs:47-90)."""
    return np.concatenate([np.ascontiguousarray(p).reshape(-1) for p in parts])


def index_select_dim(x: np.ndarray, dim: int, indices) -> np.ndarray:
    """index_select along any dimension: for every leading slab, the rows named by `indices`
    in their order (index_select_into, src/storage/cpu.rs:936-952)."""
    indices = np.asarray(indices, dtype=np.int64)
    if indices.size and (indices.min() < 0 or indices.max() >= x.shape[dim]):
        raise IndexError("index_select: index out of bounds")
    left = int(np.prod(x.shape[:dim], dtype=np.int64))
    right = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    s = np.ascontiguousarray(x).reshape(left, x.shape[dim], right)
    out = np.empty((left, indices.size, right), x.dtype)
    for l in range(left):
        for i, r in enumerate(indices):
            out[l, i, :] = s[l, r, :]
    return out.reshape(x.shape[:dim] + (indices.size,) + x.shape[dim + 1:])


def index_add_dim(src: np.ndarray, dim: int, indices, dst_shape) -> np.ndarray:
    """index_add along any dimension into zeros of `dst_shape`: for every leading slab,
    dst[l, indices[i], :] += src[l, i, :] for i ascending, each `+=` in the storage type
    (index_add_into, src/storage/cpu.rs:954-975)."""
    indices = np.asarray(indices, dtype=np.int64)
    if indices.size and (indices.min() < 0 or indices.max() >= dst_shape[dim]):
        raise IndexError("index_add: index out of bounds")
    left = int(np.prod(dst_shape[:dim], dtype=np.int64))
    right = int(np.prod(dst_shape[dim + 1:], dtype=np.int64))
    s = np.ascontiguousarray(src).reshape(left, indices.size, right)
    out = np.zeros((left, int(dst_shape[dim]), right), src.dtype)
    for l in range(left):
        for i, r in enumerate(indices):
            out[l, r, :] = out[l, r, :] + s[l, i, :]
    return out.reshape(tuple(dst_shape))
