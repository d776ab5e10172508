"""Writes the small attention fixtures in this directory.

Inputs come from the seeded generator in deers_amd.synth; expected outputs come
from a LIBRARY routine, torch.nn.functional.scaled_dot_product_attention with
is_causal=True (or an explicit offset mask when kv_len > T) evaluated in float64
on the CPU, with gradients from torch autograd.  The reference (Rust) is not
imported, run or copied by this script.  Each fixture is one .npz holding the
inputs (as the dtype the kernel will see), y, lse, dq, dk, dv (float64 results
rounded to float32) and the shape / seed header.

Usage: python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from deers_amd import synth  # noqa: E402

# name, B, H, T, D, kv_len, dtype, sigma
CASES = [
    ("f32_b1h2t8d32", 1, 2, 8, 32, None, np.float32, 1.0),
    ("f32_b2h3t33d32", 2, 3, 33, 32, None, np.float32, 1.0),
    ("f32_b1h1t130d64", 1, 1, 130, 64, None, np.float32, 1.0),
    ("f16_b2h3t33d64", 2, 3, 33, 64, None, np.float16, 1.0),
    ("f16_b1h2t200d64", 1, 2, 200, 64, None, np.float16, 1.0),
    ("f16_b1h1t130d128", 1, 1, 130, 128, None, np.float16, 0.5),
    ("f16_decode_b3h2l77d64", 3, 2, 1, 64, 77, np.float16, 1.0),
]


def torch_reference(q, k, v, do):
    tq, tk = q.shape[2], k.shape[2]
    qt, kt, vt = (torch.tensor(a.astype(np.float64), requires_grad=True) for a in (q, k, v))
    off = tk - tq
    i = torch.arange(tq)[:, None]
    j = torch.arange(tk)[None, :]
    allowed = ~((j >= off) & (j - off > i))
    y = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=allowed)
    y.backward(torch.tensor(do.astype(np.float64)))
    scores = (qt @ kt.transpose(2, 3)) / np.sqrt(q.shape[3])
    lse = torch.logsumexp(scores.masked_fill(~allowed, float("-inf")), dim=3)
    return [t.detach().numpy().astype(np.float32) for t in (y, lse, qt.grad, kt.grad, vt.grad)]


def main():
    for name, B, H, T, D, kv_len, dtype, sigma in CASES:
        x = synth.attention_inputs(name, B, H, T, D, dtype, base_seed=1234, sigma=sigma,
                                   kv_len=kv_len)
        y, lse, dq, dk, dv = torch_reference(x["q"], x["k"], x["v"], x["do"])
        np.savez_compressed(os.path.join(HERE, name + ".npz"), q=x["q"], k=x["k"], v=x["v"],
                            do=x["do"], y=y, lse=lse, dq=dq, dk=dk, dv=dv,
                            header=np.array([B, H, T, D, kv_len or T, 1234,
                                             synth.GENERATOR_VERSION], dtype=np.int64))
        print(name, "ok")


if __name__ == "__main__":
    main()
