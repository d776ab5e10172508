"""Seeded synthetic inputs for the attention path.

A counter-based generator so any element of any tensor can be produced
independently: element ``i`` of a tensor draws two 64-bit words
``splitmix64(seed + 2i)`` and ``splitmix64(seed + 2i + 1)``, maps them to
uniforms in (0,1] and [0,1), and applies Box-Muller.  The per-tensor seed is
``splitmix64`` folded over (base seed, configuration name, tensor name), so the
same (seed, config, name) triple gives the same values on every machine.
Layout is compact row-major ``[B,H,T,D]``.  f16 configurations round the f32
draw to nearest-even; the CPU oracle consumes those rounded values in f32.
"""
from __future__ import annotations

import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)
GENERATOR_VERSION = 1


def _splitmix64(x: np.ndarray) -> np.ndarray:
    """One splitmix64 output step applied to each uint64 counter in ``x``."""
    with np.errstate(over="ignore"):
        z = (x + np.uint64(0x9E3779B97F4A7C15)) & _MASK
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
        return z ^ (z >> np.uint64(31))


def tensor_seed(base_seed: int, config: str, name: str) -> int:
    """Fold (base_seed, config, name) into one 64-bit seed."""
    h = np.array([base_seed & 0xFFFFFFFFFFFFFFFF], dtype=np.uint64)
    for byte in (config + "\x00" + name).encode():
        h = _splitmix64(h ^ np.uint64(byte))
    return int(h[0])


def normal(shape, seed: int, sigma: float = 1.0, chunk: int = 1 << 22) -> np.ndarray:
    """N(0, sigma) float32 array of ``shape`` from the counter-based stream ``seed``."""
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    s = np.uint64(seed & 0xFFFFFFFFFFFFFFFF)
    for lo in range(0, n, chunk):
        hi = min(n, lo + chunk)
        with np.errstate(over="ignore"):
            ctr = (np.arange(lo, hi, dtype=np.uint64) * np.uint64(2) + s) & _MASK
            a = _splitmix64(ctr)
            b = _splitmix64((ctr + np.uint64(1)) & _MASK)
        # 53-bit mantissas: u1 in (0,1], u2 in [0,1)
        u1 = ((a >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)
        u2 = (b >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
        out[lo:hi] = (z * sigma).astype(np.float32)
    return out.reshape(shape)


def attention_inputs(config: str, B: int, H: int, T: int, D: int, dtype, base_seed: int = 0,
                     sigma: float = 1.0, names=("q", "k", "v", "do"), kv_len: int | None = None):
    """Dict of tensors for one configuration.  ``q``/``do`` are [B,H,T,D]; ``k``/``v`` are
    [B,H,kv_len or T,D].  Values are drawn in f32 and cast to ``dtype`` (RNE for f16)."""
    out = {}
    for name in names:
        t = (kv_len if (kv_len is not None and name in ("k", "v")) else T)
        x = normal((B, H, t, D), tensor_seed(base_seed, config, name), sigma)
        out[name] = x.astype(dtype)
    return out


def rotary_tables(seq_len: int, head_dim: int, base: float = 10000.0, dtype=np.float32):
    """cos, sin [seq_len, head_dim/2] of the rotary embedding, the host-side table a model
    uploads once (the reference builds it on the CPU in f32 and moves it to the device,
    src/models/gpt.rs:12-47): inv_freq_i = base^(-2i/D), angle = t * inv_freq."""
    half = head_dim // 2
    inv_freq = (np.float32(1.0) / np.power(np.float32(base),
                                           (2 * np.arange(half)).astype(np.float32) / np.float32(head_dim))
                ).astype(np.float32)
    ang = (np.arange(seq_len, dtype=np.float32)[:, None] * inv_freq[None, :]).astype(np.float32)
    return np.cos(ang).astype(dtype), np.sin(ang).astype(dtype)
