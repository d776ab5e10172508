"""The C++ host side (deers_amd/host): tensor / autograd slice and the fused attention op.

The graph cases are the reference's own autograd tests (src/backprop.rs:142-201)
restated in C++ and run on unbacked tensors, so they need no GPU.  The GPU case
drives the op the way src/models/gpt.rs:135-147 does (projections [B,T,H,D],
permuted views in, reshape copy out, reverse sweep through Permute / Compact /
FusedCausalAttention) and is checked here against the CPU oracle.
"""
import os
import subprocess

import numpy as np
import pytest

from deers_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_TEST = os.path.join(ROOT, "deers_amd", "host", "host_test")


def _run(*args):
    if not os.path.exists(HOST_TEST):
        pytest.fail("deers_amd/host/host_test is not built (run __graft_entry__.build())")
    return subprocess.run([HOST_TEST, *args], capture_output=True, text=True, timeout=300)


def test_host_graph_contract():
    r = _run("graph")
    assert r.returncode == 0, r.stdout + r.stderr
    for name in ("layout", "sorted_nodes_linear_chain", "sorted_nodes_diamond",
                 "sorted_nodes_skips_no_grad", "graph_of_attention_views"):
        assert f"ok {name}" in r.stdout
    assert "all passed" in r.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,B,H,T,D,L,tol", [
    (np.float16, 2, 3, 200, 64, 300, 5e-3),
    (np.float32, 1, 2, 130, 32, 0, 1e-4),
])
def test_host_fused_attention_matches_oracle(tmp_path, dtype, B, H, T, D, L, tol):
    import oracle
    x = synth.attention_inputs("host", B, H, T, D, dtype, base_seed=3)
    bthd = lambda a: np.ascontiguousarray(a.transpose(0, 2, 1, 3))
    for name in ("q", "k", "v", "do"):
        bthd(x[name]).tofile(tmp_path / f"{name}.bin")
    if L:
        d = synth.attention_inputs("hostdec", B, H, 1, D, dtype, base_seed=4, kv_len=L,
                                   names=("q", "k", "v"))
        d["q"][:, :, 0].tofile(tmp_path / "dec_q.bin")
        d["k"].tofile(tmp_path / "dec_k.bin")
        d["v"].tofile(tmp_path / "dec_v.bin")
    (tmp_path / "case.txt").write_text(f"{0 if dtype == np.float16 else 1} {B} {H} {T} {D} {L}\n")

    r = _run("gpu", str(tmp_path))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok backward_accumulates_diamond_grads" in r.stdout and "all passed" in r.stdout
    assert "ok matmul_add_matches_matmul_then_add" in r.stdout

    def out(name, shape=(B, T, H, D)):
        return np.fromfile(tmp_path / name, dtype=dtype).reshape(shape).astype(np.float64)

    f32 = {n: x[n].astype(np.float32) for n in ("q", "k", "v", "do")}
    want_o = oracle.attn_fwd(f32["q"], f32["k"], f32["v"])
    want = oracle.attn_bwd(f32["q"], f32["k"], f32["v"], f32["do"])
    err = lambda got, ref: float(np.max(np.abs(got - bthd(ref))))
    assert err(out("y.bin"), want_o) <= tol
    for name, ref in zip(("dq.bin", "dk.bin", "dv.bin"), want):
        assert err(out(name), ref) <= tol, name
    # RoPE on q and k around the core, against the composed oracle
    cos, sin = oracle.rope_tables(T, D, dtype=dtype)
    c32, s32 = cos.astype(np.float32), sin.astype(np.float32)
    hd = lambda a: a.transpose(0, 2, 1, 3)  # [B,T,H,D] <-> [B,H,T,D]
    qr = hd(oracle.rope_apply(bthd(f32["q"]), c32, s32))
    kr = hd(oracle.rope_apply(bthd(f32["k"]), c32, s32))
    want_yr = oracle.attn_fwd(qr, kr, f32["v"])
    gq, gk, gv = oracle.attn_bwd(qr, kr, f32["v"], f32["do"])
    want_r = (oracle.rope_apply_bwd(bthd(gq), c32, s32), oracle.rope_apply_bwd(bthd(gk), c32, s32),
              bthd(gv))
    assert float(np.max(np.abs(out("y_rope.bin") - bthd(want_yr)))) <= tol
    for name, ref in zip(("dq_rope.bin", "dk_rope.bin", "dv_rope.bin"), want_r):
        assert float(np.max(np.abs(out(name) - ref))) <= tol, name
    if dtype == np.float16:
        # two ops on the same inputs give the same bits, and x + x is exact in f16
        assert np.array_equal(out("dv_twice.bin"), 2 * out("dv.bin"))
    if L:
        got = np.fromfile(tmp_path / "dec_o.bin", dtype=dtype).reshape(B, H, D).astype(np.float64)
        ref = oracle.attn_fwd(d["q"].astype(np.float32), d["k"].astype(np.float32),
                              d["v"].astype(np.float32))[:, :, 0]
        assert float(np.max(np.abs(got - ref))) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,B,T,C,H,tol", [
    (np.float32, 2, 70, 128, 4, 2e-4),
    (np.float16, 2, 200, 256, 4, 5e-3),
])
def test_host_attention_module_matches_composed_oracle(tmp_path, dtype, B, T, C, H, tol):
    """x -> q/k/v projections -> RoPE -> causal attention -> head merge -> out projection
    (src/models/gpt.rs:101-147) and its backward, against the same chain on the CPU oracle
    (rounded to f16 where the device rounds).  Tolerance: the path's 5e-3 (f16) per unit of
    the tensor's largest value (weight gradients sum over B*T rows and reach tens)."""
    import oracle
    rng = np.random.default_rng(41)
    D = C // H
    x = rng.standard_normal((B, T, C)).astype(dtype)
    ws = [(rng.standard_normal((C, C)) / np.sqrt(C)).astype(dtype) for _ in range(4)]
    dy = rng.standard_normal((B, T, C)).astype(dtype)
    for name, a in zip(("x", "wq", "wk", "wv", "wo", "dy"), (x, *ws, dy)):
        a.tofile(tmp_path / f"{name}.bin")
    (tmp_path / "module.txt").write_text(f"{0 if dtype == np.float16 else 1} {B} {T} {C} {H}\n")
    r = _run("module", str(tmp_path))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok module" in r.stdout and "all passed" in r.stdout

    f = lambda a: a.astype(np.float32)
    xf, (wq, wk, wv, wo), dyf = f(x).reshape(B * T, C), [f(w) for w in ws], f(dy).reshape(B * T, C)
    mm = lambda a, b: oracle.matmul(a[None], b[None])[0]
    rnd = (lambda a: a.astype(np.float16).astype(np.float32)) if dtype == np.float16 else (lambda a: a)
    cos, sin = oracle.rope_tables(T, D, dtype=dtype)
    c32, s32 = f(cos), f(sin)
    hd = lambda a: np.ascontiguousarray(a.transpose(0, 2, 1, 3))
    q, k, v = (rnd(mm(xf, w)).reshape(B, T, H, D) for w in (wq, wk, wv))
    qh, kh, vh = hd(rnd(oracle.rope_apply(q, c32, s32))), hd(rnd(oracle.rope_apply(k, c32, s32))), hd(v)
    o = rnd(oracle.attn_fwd(qh, kh, vh))
    o_flat = hd(o).reshape(B * T, C)
    want_y = mm(o_flat, wo)
    # backward by hand, in the order the reverse sweep runs it
    d_o_flat = rnd(mm(dyf, wo.T))
    want_dwo = mm(o_flat.T, dyf)
    gq, gk, gv = (rnd(g) for g in oracle.attn_bwd(qh, kh, vh, hd(d_o_flat.reshape(B, T, H, D))))
    dq = rnd(oracle.rope_apply_bwd(hd(gq), c32, s32)).reshape(B * T, C)
    dk = rnd(oracle.rope_apply_bwd(hd(gk), c32, s32)).reshape(B * T, C)
    dv = hd(gv).reshape(B * T, C)
    want = {"dwq": mm(xf.T, dq), "dwk": mm(xf.T, dk), "dwv": mm(xf.T, dv), "dwo": want_dwo,
            "dx": mm(dq, wq.T) + mm(dk, wk.T) + mm(dv, wv.T)}
    got = lambda name, shape: np.fromfile(tmp_path / f"{name}.bin", dtype=dtype).reshape(shape).astype(np.float64)
    ytol = tol * max(1.0, float(np.max(np.abs(want_y))))
    assert np.max(np.abs(got("y", (B * T, C)) - want_y)) <= ytol
    if dtype == np.float16:
        # token-by-token generation through the KV cache reproduces the full forward's rows
        assert np.max(np.abs(got("y_decode", (B * T, C)) - want_y)) <= ytol
        assert np.max(np.abs(got("y_decode", (B * T, C)) - got("y", (B * T, C)))) <= ytol
    for name, ref in want.items():
        g = got(name, ref.shape)
        scale = max(1.0, float(np.max(np.abs(ref))))
        assert np.max(np.abs(g - ref)) <= tol * scale, name


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,outer,inner", [(np.float32, 6, 777), (np.float16, 5, 1000),
                                               (np.float32, 2, 3)])
def test_host_fused_log_softmax_matches_oracle(tmp_path, dtype, outer, inner):
    import oracle
    if (outer, inner) == (2, 3):  # the reference's literal, tests/tensor.rs:296
        x = np.array([[1.0, 2.0, 3.0], [1.5, 0.5, -1.0]], dtype=dtype)
    else:
        x = synth.normal((outer, inner), synth.tensor_seed(41, "hostlsm", "x"), 3.0).astype(dtype)
    g = synth.normal((outer, inner), synth.tensor_seed(41, "hostlsm", "g"), 1.0).astype(dtype)
    x.tofile(tmp_path / "x.bin")
    g.tofile(tmp_path / "g.bin")
    (tmp_path / "case.txt").write_text(f"{0 if dtype == np.float16 else 1} {outer} {inner}\n")
    r = _run("lsm", str(tmp_path))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok log_softmax" in r.stdout and "all passed" in r.stdout

    def out(name, shape):
        return np.fromfile(tmp_path / name, dtype=dtype).reshape(shape)

    x32 = x.astype(np.float32)
    tol = lambda want: (5e-3 + np.abs(want).max() * 2 ** -11) if dtype == np.float16 else 1e-4
    y = out("y.bin", (outer, inner))
    want = oracle.log_softmax_fwd(x32)
    assert np.abs(y.astype(np.float32) - want).max() <= tol(want)
    want_dx = oracle.log_softmax_bwd(g.astype(np.float32), y.astype(np.float32))
    assert np.abs(out("dx.bin", (outer, inner)).astype(np.float32) - want_dx).max() <= tol(want_dx)
    # transposed view: rows are the columns of x; loss = sum, so d = 1 - n * softmax
    yt = out("yt.bin", (inner, outer))
    want_t = oracle.log_softmax_fwd(np.ascontiguousarray(x32.T))
    assert np.abs(yt.astype(np.float32) - want_t).max() <= tol(want_t)
    want_dxt = oracle.log_softmax_bwd(np.ones_like(want_t), yt.astype(np.float32)).T
    assert np.abs(out("dxt.bin", (outer, inner)).astype(np.float32) - want_dxt).max() <= tol(want_dxt)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,max_norm", [(np.float32, 0.75), (np.float32, 1e9), (np.float16, 0.75)])
def test_host_adamw_and_clip_grad_norm_match_oracle(tmp_path, dtype, max_norm):
    import oracle
    n0, n1, steps, lr, wd = 5003, 640, 6, 3e-3, 0.1
    w0 = synth.normal((n0,), synth.tensor_seed(61, "hostopt", "w0"), 1.0).astype(dtype)
    w1 = synth.normal((n1,), synth.tensor_seed(61, "hostopt", "w1"), 1.0).astype(dtype)
    w0.tofile(tmp_path / "w0.bin")
    w1.tofile(tmp_path / "w1.bin")
    gs = []
    for t in range(1, steps + 1):
        g0 = synth.normal((n0,), synth.tensor_seed(61, "hostopt", f"g0_{t}"), 0.02).astype(dtype)
        g1 = synth.normal((n1,), synth.tensor_seed(61, "hostopt", f"g1_{t}"), 0.02).astype(dtype)
        g0.tofile(tmp_path / f"g0_{t}.bin")
        g1.tofile(tmp_path / f"g1_{t}.bin")
        gs.append((g0, g1))
    dt = 0 if dtype == np.float16 else 1
    (tmp_path / "case.txt").write_text(f"{dt} {n0} {n1} {steps} {lr} {wd} {max_norm}\n")
    r = _run("optim", str(tmp_path))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok optim" in r.stdout and "all passed" in r.stdout

    norms = np.fromfile(tmp_path / "norms.bin", dtype=np.float32)
    assert norms.shape == (steps,)
    m0 = np.zeros(n0, dtype)
    v0 = np.zeros(n0, dtype)
    m1 = np.zeros(n1, dtype)
    v1 = np.zeros(n1, dtype)
    eps = 1e-8
    for t, (g0, g1) in enumerate(gs, start=1):
        want_norm = np.sqrt((g0.astype(np.float64) ** 2).sum() + (g1.astype(np.float64) ** 2).sum())
        assert abs(norms[t - 1] - want_norm) <= 1e-6 * want_norm
        # rescale with the norm the device computed (summation order differs from numpy's
        # in the last bit), exactly as src/optim.rs:285-293 does; the rest is bit for bit
        if np.isfinite(norms[t - 1]) and norms[t - 1] > np.float32(max_norm):
            s = oracle._scalar(max_norm / (float(norms[t - 1]) + 1e-6), dtype)
            g0, g1 = (g0 * s).astype(dtype), (g1 * s).astype(dtype)
        w0, m0, v0 = oracle.adamw_step(w0, g0, m0, v0, t, lr, (0.9, 0.95), eps, wd, dtype=dtype)
        w1, m1, v1 = oracle.adamw_step(w1, g1, m1, v1, t, lr, (0.9, 0.95), eps, wd, dtype=dtype)
    if max_norm < 1:
        assert (norms > max_norm).all()  # the case does clip
    out = lambda name: np.fromfile(tmp_path / name, dtype=dtype)
    for name, want in (("w0_out.bin", w0), ("w1_out.bin", w1), ("m0_out.bin", m0), ("v0_out.bin", v0)):
        assert np.array_equal(out(name), want, equal_nan=True), name


REFERENCE_TEST_CFG = dict(vocab_size=8, sequence_len=4, n_layer=1, n_head=2, n_embd=4, mlp_hidden_dim=8,
                          rms_norm_eps=1e-5, rope_base=10000.0)  # tests/gpt.rs:38-49: head_dim 2


@pytest.mark.gpu
@pytest.mark.parametrize("cfg,B,T", [
    (dict(vocab_size=37, sequence_len=16, n_layer=2, n_head=2, n_embd=64, mlp_hidden_dim=96,
          rms_norm_eps=1e-5, rope_base=10000.0), 3, 11),
    (dict(vocab_size=300, sequence_len=160, n_layer=3, n_head=3, n_embd=192, mlp_hidden_dim=256,
          rms_norm_eps=1e-5, rope_base=10000.0), 2, 130),
    (REFERENCE_TEST_CFG, 2, 3),
    (dict(vocab_size=50, sequence_len=40, n_layer=2, n_head=2, n_embd=12, mlp_hidden_dim=20,
          rms_norm_eps=1e-5, rope_base=10000.0), 3, 37),  # head_dim 6
], ids=["d32", "d64", "reference-test-geometry-d2", "d6"])
def test_host_gpt_training_step_matches_oracle(tmp_path, cfg, B, T):
    """GPT forward, cross-entropy, backward and AdamW steps of the C++ host (f32) against
    the composed numpy oracle, the way tests/gpt.rs compares the reference with a library
    model.  Head widths 32 and 64 run the fused attention kernels; the reference's own test
    geometry (head_dim 2, its token ids and targets, tests/gpt.rs:38-65) and a head_dim 6
    model run the same op through the unfused device chain and the per-pair RoPE kernel."""
    import oracle
    from oracle import gpt as ogpt
    from test_oracle_gpt import make_weights
    rng = np.random.default_rng(17)
    if cfg is REFERENCE_TEST_CFG:
        ids = np.array([[1, 2, 3], [4, 3, 2]], np.int64)
        targets = np.array([2, 3, 4, 3, 2, 1], np.int64)
    else:
        ids = rng.integers(0, cfg["vocab_size"], (B, T)).astype(np.int64)
        ids[1, 2:6] = ids[0, 0]
        targets = rng.integers(0, cfg["vocab_size"], B * T).astype(np.int64)
    w = make_weights(cfg, 19, dtype=np.float32)
    for i, a in enumerate(w):
        a.tofile(tmp_path / f"w{i}.bin")
    ids.tofile(tmp_path / "ids.bin")
    targets.tofile(tmp_path / "targets.bin")
    steps, lr, wd, max_norm = 3, 1e-2, 0.01, 1.0
    (tmp_path / "case.txt").write_text(
        f"{cfg['vocab_size']} {cfg['sequence_len']} {cfg['n_layer']} {cfg['n_head']} {cfg['n_embd']} "
        f"{cfg['mlp_hidden_dim']} {cfg['rms_norm_eps']} {cfg['rope_base']} {B} {T} {steps} {lr} {wd} "
        f"{max_norm}\n")
    r = _run("gpt", str(tmp_path))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok gpt" in r.stdout and "all passed" in r.stdout

    out = lambda name, shape: np.fromfile(tmp_path / name, dtype=np.float32).reshape(shape)
    V = cfg["vocab_size"]
    want_logits = ogpt.gpt_forward(cfg, w, ids)
    assert np.abs(out("logits.bin", (B, T, V)) - want_logits).max() <= 1e-4
    want_loss, want_grads = ogpt.gpt_loss_and_grads(cfg, w, ids, targets)
    assert abs(float(out("loss.bin", (1,))[0]) - float(want_loss)) <= 1e-5
    for i, g in enumerate(want_grads):
        assert np.abs(out(f"g{i}.bin", g.shape) - g).max() <= 1e-4, i
    # training steps: same losses, norms and parameters
    losses, norms = out("losses.bin", (steps,)), out("norms.bin", (steps,))
    mom = [(np.zeros_like(a), np.zeros_like(a)) for a in w]
    cur = w
    for t in range(1, steps + 1):
        loss, norm, cur, mom = ogpt.train_step(cfg, cur, mom, t, ids, targets, lr, (0.9, 0.95), 1e-8, wd,
                                               max_norm)
        assert abs(float(losses[t - 1]) - float(loss)) <= 1e-4, t
        assert abs(float(norms[t - 1]) - float(norm)) <= 1e-4 * max(1.0, float(norm)), t
    assert losses[-1] < losses[0]
    for i, a in enumerate(cur):
        # Adam's first steps move every weight by about lr whatever the gradient's size, so
        # a gradient entry near zero may pick either sign: compare where the step is decided
        d = np.abs(out(f"w{i}_out.bin", a.shape) - a)
        assert np.quantile(d, 0.999) <= 1e-4 and d.max() <= 2.5 * steps * lr, i


@pytest.mark.gpu
@pytest.mark.parametrize("T,n_new,seq_len,C,H", [(24, 10, 48, 128, 2), (300, 6, 320, 128, 2), (40, 8, 64, 192, 6)])
def test_host_gpt_generation_with_kv_caches(tmp_path, T, n_new, seq_len, C, H):
    """An f16 GPT generating through per-block KV caches: every decode step's logits equal
    the matching row of the full causal forward (device) and the f32 oracle on the same
    f16 weights; a prompt taken through prefill leaves the same logits and caches as its tokens
    one by one; the greedy continuation picks the teacher-forced argmax at every position."""
    from oracle import gpt as ogpt
    from test_oracle_gpt import make_weights
    cfg = dict(vocab_size=300, sequence_len=seq_len, n_layer=2, n_head=H, n_embd=C, mlp_hidden_dim=2 * C,
               rms_norm_eps=1e-5, rope_base=10000.0)
    # T = 300: the prefilled half spans two 128-row tiles of the fused forward; C = 192 with 6
    # heads is the width of the reference's TinyStories model (head width 32; its products do
    # not fit the few-rows kernel and take the separate norm / GEMM / activation launches)
    B = 3
    rng = np.random.default_rng(23)
    ids = rng.integers(0, cfg["vocab_size"], (B, T)).astype(np.int64)
    w = [a.astype(np.float16) for a in make_weights(cfg, 29, dtype=np.float32)]
    for i, a in enumerate(w):
        a.tofile(tmp_path / f"w{i}.bin")
    ids.tofile(tmp_path / "ids.bin")
    (tmp_path / "case.txt").write_text(
        f"{cfg['vocab_size']} {cfg['sequence_len']} {cfg['n_layer']} {cfg['n_head']} {cfg['n_embd']} "
        f"{cfg['mlp_hidden_dim']} {cfg['rms_norm_eps']} {cfg['rope_base']} {B} {T} {n_new}\n")
    r = _run("generate", str(tmp_path))
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok generate" in r.stdout and "all passed" in r.stdout
    V = cfg["vocab_size"]
    full = np.fromfile(tmp_path / "logits_full.bin", dtype=np.float16).reshape(B, T, V).astype(np.float32)
    steps = np.fromfile(tmp_path / "logits_steps.bin", dtype=np.float16).reshape(B, T, V).astype(np.float32)
    want = ogpt.gpt_forward(cfg, [a.astype(np.float32) for a in w], ids)
    scale = np.abs(want).max()
    assert np.abs(full - want).max() <= 2e-2 * scale
    assert np.abs(steps - want).max() <= 2e-2 * scale
    assert np.abs(steps - full).max() <= 2e-2 * scale
    # the first half through prefill, the second half step by step from its caches
    t0 = T // 2
    pre = np.fromfile(tmp_path / "logits_prefill.bin", dtype=np.float16).reshape(B, V).astype(np.float32)
    assert np.abs(pre - want[:, t0 - 1]).max() <= 2e-2 * scale
    assert np.abs(pre - full[:, t0 - 1]).max() <= 2e-2 * scale
    rest = np.fromfile(tmp_path / "logits_after_prefill.bin", dtype=np.float16).reshape(B, T - t0, V)
    assert np.abs(rest.astype(np.float32) - want[:, t0:]).max() <= 2e-2 * scale
    H, D = cfg["n_head"], cfg["n_embd"] // cfg["n_head"]
    for name in ("k", "v"):
        a = np.fromfile(tmp_path / f"{name}_cache_prefill.bin", dtype=np.float16).reshape(B, H, T, D)
        b = np.fromfile(tmp_path / f"{name}_cache_steps.bin", dtype=np.float16).reshape(B, H, T, D)
        a, b = a.astype(np.float32), b.astype(np.float32)
        assert np.abs(a[:, :, :t0] - b[:, :, :t0]).max() <= 2e-2 * max(1.0, np.abs(b).max()), name
        assert np.abs(b[:, :, :t0]).max() > 0
    # greedy continuation
    gen = np.fromfile(tmp_path / "generated.bin", dtype=np.int64).reshape(B, t0 + n_new)
    assert np.array_equal(gen[:, :t0], ids[:, :t0])
    assert gen.min() >= 0 and gen.max() < V
    forced = np.fromfile(tmp_path / "logits_generated.bin", dtype=np.float16).reshape(B, t0 + n_new, V)
    forced = forced.astype(np.float32)
    for t in range(t0 - 1, t0 + n_new - 1):
        row = forced[:, t]
        picked = row[np.arange(B), gen[:, t + 1]]
        # the generated token is the teacher-forced maximum up to f16 rounding of the logits
        assert (row.max(axis=1) - picked <= 2e-2 * scale).all(), t
