"""BASELINE configs[4] at its real size: the f32 attention kernels at B=8 H=12 T=1024 D=64 and
the whole GPT training step at 12 layers x 12 heads x 768, vocabulary 50257, T=1024, B=8.

The reference's counterpart is its training loop (examples/tinystories_train.rs:188-218) and
its end-to-end test against a second implementation (tests/gpt.rs:295-343); at this size the
CPU oracle is run on two of the eight sequences for the attention kernels, and the step as a
whole is held to size-independent properties of a freshly initialised model."""
import json
import math
import os
import subprocess

import numpy as np
import pytest

import oracle
from deers_amd import rocm, synth

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GPT_STEP = os.path.join(ROOT, "deers_amd", "host", "gpt_step")


def max_err(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))))


def test_f32_attention_at_config5_size_matches_oracle_and_is_reproducible():
    B, H, T, D = 8, 12, 1024, 64
    rocm.init(0)
    x = synth.attention_inputs("c5-attn", B, H, T, D, np.float32, base_seed=0)
    q, k, v, do = x["q"], x["k"], x["v"], x["do"]
    print(f"case c5-attn f32 B={B} H={H} T={T} D={D}", flush=True)
    o, lse, dq, dk, dv = rocm.attn_fwd_bwd(q, k, v, do)
    for a in (o, lse, dq, dk, dv):
        assert np.isfinite(a).all()
    # the oracle on two (batch, head) pairs at opposite corners of the launch grid
    for b, h in ((0, 0), (7, 11)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        ro, rlse = oracle.attn_fwd(q[sl], k[sl], v[sl], return_lse=True)
        rdq, rdk, rdv = oracle.attn_bwd(q[sl], k[sl], v[sl], do[sl])
        errs = {"o": max_err(o[sl], ro), "lse": max_err(lse[sl], rlse), "dq": max_err(dq[sl], rdq),
                "dk": max_err(dk[sl], rdk), "dv": max_err(dv[sl], rdv)}
        print(f"  (b={b}, h={h}): " + " ".join(f"{n}={e:.2e}" for n, e in errs.items()), flush=True)
        for n, e in errs.items():
            assert e <= 1e-4, f"(b={b}, h={h}) {n}: max abs err {e:.3e} > 1e-4"
    # size-independent properties over the whole launch
    np.testing.assert_array_equal(o[:, :, 0], v[:, :, 0])  # the first query sees only itself
    assert np.max(np.abs(dq[:, :, 0])) <= 1e-5             # ... so dS = P (dP - delta) cancels to rounding
    o2, lse2, dq2, dk2, dv2 = rocm.attn_fwd_bwd(q, k, v, do)
    for a, b_ in ((o, o2), (lse, lse2), (dk, dk2), (dv, dv2)):
        np.testing.assert_array_equal(a, b_)               # bit-reproducible
    # dQ adds the contributions of its (up to 8) key blocks with f32 atomics in arrival order:
    # reproducible to f32 rounding of that sum
    assert np.max(np.abs(dq - dq2)) <= 1e-6


def test_f32_attention_with_ragged_heads_and_several_tiles_per_workgroup():
    """45 heads (not a multiple of the 8 XCDs) x 12 query tiles = 540 tiles, more than the
    device holds at once: the f32 forward's workgroups walk lists of several tiles, with list
    entries of the three padding heads skipped; T is not a multiple of any tile size."""
    B, H, T, D = 5, 9, 1500, 64
    rocm.init(0)
    x = synth.attention_inputs("c5-ragged", B, H, T, D, np.float32, base_seed=3)
    q, k, v, do = x["q"], x["k"], x["v"], x["do"]
    print(f"case c5-ragged f32 B={B} H={H} T={T} D={D}", flush=True)
    o, lse, dq, dk, dv = rocm.attn_fwd_bwd(q, k, v, do)
    for a in (o, lse, dq, dk, dv):
        assert np.isfinite(a).all()
    for b, h in ((0, 0), (2, 4), (4, 8)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        ro, rlse = oracle.attn_fwd(q[sl], k[sl], v[sl], return_lse=True)
        rdq, rdk, rdv = oracle.attn_bwd(q[sl], k[sl], v[sl], do[sl])
        errs = {"o": max_err(o[sl], ro), "lse": max_err(lse[sl], rlse), "dq": max_err(dq[sl], rdq),
                "dk": max_err(dk[sl], rdk), "dv": max_err(dv[sl], rdv)}
        print(f"  (b={b}, h={h}): " + " ".join(f"{n}={e:.2e}" for n, e in errs.items()), flush=True)
        for n, e in errs.items():
            assert e <= 1e-4, f"(b={b}, h={h}) {n}: max abs err {e:.3e} > 1e-4"
    np.testing.assert_array_equal(o[:, :, 0], v[:, :, 0])
    o2, lse2, _, dk2, dv2 = rocm.attn_fwd_bwd(q, k, v, do)
    for a, b_ in ((o, o2), (lse, lse2), (dk, dk2), (dv, dv2)):
        np.testing.assert_array_equal(a, b_)


def test_gpt_training_step_at_baseline_geometry_learns():
    if not os.path.exists(GPT_STEP):
        pytest.fail("deers_amd/host/gpt_step is not built (run __graft_entry__.build())")
    vocab = 50257
    # vocab seq n_layer n_head n_embd mlp_hidden batch steps warmup
    args = [str(a) for a in (vocab, 1024, 12, 12, 768, 3072, 8, 3, 1)]
    print("gpt_step " + " ".join(args), flush=True)
    r = subprocess.run([GPT_STEP] + args, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout + r.stderr
    out = json.loads(r.stdout.strip().splitlines()[-1])
    losses, norms = out["losses"], out["grad_norms"]
    print(f"losses {losses} grad norms {norms}", flush=True)
    assert out["parameters"] == 162129408 and out["batch"] == 8 and out["seq_len"] == 1024
    assert len(losses) >= 4 and all(math.isfinite(x) for x in losses + norms)
    assert all(n > 0 for n in norms)
    # A fresh model predicts nearly uniformly: the loss starts at ln(vocab) plus half the
    # variance of a logit.  The final RMSNorm leaves rows of mean square 1 and the LM head is
    # uniform in +-1/sqrt(768) (variance 1/(3*768)), so a logit has variance 1/3.
    expect = math.log(vocab) + 1.0 / 6.0
    assert abs(losses[0] - expect) <= 0.1, f"initial loss {losses[0]:.4f}, expected about {expect:.4f}"
    assert abs(losses[0] - math.log(vocab)) <= 0.3
    # same batch every step: clipped AdamW steps must drive the loss down
    assert losses[3] < losses[0] - 1e-3 and losses[-1] < losses[0]
