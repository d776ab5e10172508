#!/usr/bin/env python3
"""Benchmark of the MI355X causal-attention path (one GPU).

A "step" is one fused forward + backward of causal self-attention over one batch
of synthetic, seeded inputs that are already resident in HBM:
f16, B=8 H=12 T=1024 D=64 (GPT-2-small geometry).  The headline value is
TFLOP/s with the FlashAttention FLOP convention, fwd+bwd = 7*B*H*T^2*D
(causal-halved; the backward counted as 2.5x the forward however many tile
GEMMs the kernels really execute).  The decode kernel (B=32 H=12 L=4096 D=64,
f16) is timed in the same run and reported as achieved HBM GB/s.

Prints ONE JSON line.  `roofline` describes the dominant kernel of the step from
a pass of its own: one hipEvent pair around K back-to-back launches of that
kernel; `cpu_baseline` is the CPU oracle (a restatement of the reference's
materialised CPU path) timed on this box's host cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from deers_amd import rocm, synth  # noqa: E402

PEAK_F16_TFLOPS = 2500.0  # MI355X dense f16 MFMA, published
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, published

KERNEL_PASS_MIN_STEPS = 200  # launches per kernel behind `kernels` and `roofline`

C2 = dict(B=8, H=12, T=1024, D=64)
C4 = dict(B=32, H=12, L=4096, D=64)


def attn_flops(B, H, T, D):
    fwd = 4.0 * B * H * T * T * D / 2.0
    return fwd, 2.5 * fwd


def bench_train(steps: int, warmup: int, only: str = "all"):
    B, H, T, D = C2["B"], C2["H"], C2["T"], C2["D"]
    x = synth.attention_inputs("c2", B, H, T, D, np.float16, base_seed=0)
    q, k, v, do = (rocm.DeviceBuffer.from_numpy(x[n]) for n in ("q", "k", "v", "do"))
    o = rocm.DeviceBuffer((B, H, T, D), np.float16)
    lse = rocm.DeviceBuffer((B, H, T), np.float32)
    dq, dk, dv = (rocm.DeviceBuffer((B, H, T, D), np.float16) for _ in range(3))
    scale = rocm.default_scale(D)

    def fwd():
        rocm.attn_fwd_raw(np.float16, q.ptr, k.ptr, v.ptr, o.ptr, lse.ptr, B, H, T, D, scale)

    def bwd():
        rocm.attn_bwd_raw(np.float16, q.ptr, k.ptr, v.ptr, o.ptr, lse.ptr, do.ptr, dq.ptr, dk.ptr,
                          dv.ptr, B, H, T, D, scale)

    fwd()  # the backward needs a forward's O and LSE whatever is timed

    def step():
        if only in ("all", "fwd"):
            fwd()
        if only in ("all", "bwd"):
            bwd()

    # first pass: as many untimed steps as the per-kernel pass has launches, so that the timed
    # passes see the device in the state a long job keeps it in: from idle, the first few
    # milliseconds of launches run 5-8 % slower while the clocks settle, and K = 20 steps are
    # 2 ms in all.
    ksteps = max(steps, KERNEL_PASS_MIN_STEPS)
    for _ in range(ksteps):
        step()
    rocm.sync()
    # second pass: per-kernel device time, one event pair around `ksteps` back-to-back launches
    # of that kernel (`roofline` is computed from this pass; a kernel trace of the same command
    # gives the same average from the dispatch records)
    kernels = {}
    for name, fn in (("attn_fwd_f16", fwd), ("attn_bwd_f16", bwd)):
        if only not in ("all", name[5:8]):
            continue
        for _ in range(10):
            fn()
        rocm.sync()
        t = rocm.Timer()
        t.start()
        for _ in range(ksteps):
            fn()
        t.stop()
        rocm.sync()
        kernels[name] = {"calls": ksteps, "avg_us": 1e3 * t.elapsed_ms() / ksteps}

    # the timed region: `warmup` untimed steps, then exactly `steps` steps between two events
    # (and two host clock reads), synchronised on both sides
    for _ in range(warmup):
        step()
    rocm.sync()
    timer = rocm.Timer()
    t0 = time.perf_counter()
    timer.start()
    for _ in range(steps):
        step()
    timer.stop()
    rocm.sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    dev_ms = timer.elapsed_ms()

    # third pass: every step between its own pair of events (median and minimum of a step)
    timers = [rocm.Timer() for _ in range(steps)]
    for t in timers:
        t.start()
        step()
        t.stop()
    rocm.sync()
    per_step = sorted(1e3 * t.elapsed_ms() for t in timers)
    step_us = {"median": per_step[len(per_step) // 2], "min": per_step[0]}
    return dict(wall_ms=wall_ms, dev_ms=dev_ms, kernels=kernels, step_us=step_us,
                warmup_effective=warmup + 2 * ksteps + 10 * len(kernels))


PEAK_F32_TFLOPS = 157.3  # MI355X dense f32 MFMA, published


def bench_attention_config(dtype, B, H, T, D, launches=50, sigma=1.0):
    """Forward, backward and fwd+bwd step of one more attention geometry: each from one event
    pair around `launches` back-to-back launches, after as many untimed ones."""
    x = synth.attention_inputs(f"bench-{B}-{H}-{T}-{D}", B, H, T, D, dtype, base_seed=1)
    if sigma != 1.0:
        x = {n: (a.astype(np.float32) * sigma).astype(dtype) for n, a in x.items()}
    q, k, v, do = (rocm.DeviceBuffer.from_numpy(x[n]) for n in ("q", "k", "v", "do"))
    o = rocm.DeviceBuffer((B, H, T, D), dtype)
    lse = rocm.DeviceBuffer((B, H, T), np.float32)
    dq, dk, dv = (rocm.DeviceBuffer((B, H, T, D), dtype) for _ in range(3))
    scale = rocm.default_scale(D)

    def fwd():
        rocm.attn_fwd_raw(dtype, q.ptr, k.ptr, v.ptr, o.ptr, lse.ptr, B, H, T, D, scale)

    def bwd():
        rocm.attn_bwd_raw(dtype, q.ptr, k.ptr, v.ptr, o.ptr, lse.ptr, do.ptr, dq.ptr, dk.ptr, dv.ptr,
                          B, H, T, D, scale)

    def both():
        fwd()
        bwd()

    us = {}
    for name, fn in (("fwd", fwd), ("bwd", bwd), ("step", both)):
        for _ in range(launches):
            fn()
        rocm.sync()
        t = rocm.Timer()
        t.start()
        for _ in range(launches):
            fn()
        t.stop()
        rocm.sync()
        us[name] = 1e3 * t.elapsed_ms() / launches
    fwd_f, bwd_f = attn_flops(B, H, T, D)
    peak = PEAK_F16_TFLOPS if np.dtype(dtype) == np.float16 else PEAK_F32_TFLOPS
    tf = {"fwd": fwd_f / (us["fwd"] * 1e-6) / 1e12, "bwd": bwd_f / (us["bwd"] * 1e-6) / 1e12,
          "step": (fwd_f + bwd_f) / (us["step"] * 1e-6) / 1e12}
    return {"workload": f"causal self-attention fwd+bwd, {np.dtype(dtype).name}, B={B} H={H} T={T} D={D}",
            "launches_timed": launches, "us": us, "tflops": tf,
            "frac_mfma_peak": {n: v / peak for n, v in tf.items()}, "peak_tflops": peak,
            "flops_per_step": fwd_f + bwd_f}


EXTRA_CONFIGS = {
    "c1": dict(dtype=np.float32, B=4, H=6, T=256, D=32),                    # BASELINE configs[0]
    "c3": dict(dtype=np.float16, B=1, H=16, T=8192, D=128, sigma=0.5),      # BASELINE configs[2]
    "c2_d128": dict(dtype=np.float16, B=8, H=12, T=1024, D=128),            # configs[1] at head width 128
    "c5_attn": dict(dtype=np.float32, B=8, H=12, T=1024, D=64),             # one layer's attention of configs[4]
}


def bench_decode(steps: int, warmup: int, rotate: int = 4):
    """Decode over `rotate` distinct KV caches in turn so the 256 MB last-level cache
    cannot serve a 403 MB working set from one call to the next."""
    B, H, L, D = C4["B"], C4["H"], C4["L"], C4["D"]
    x = synth.attention_inputs("c4", B, H, 1, D, np.float16, base_seed=0, kv_len=L,
                               names=("q", "k", "v"))
    qb = rocm.DeviceBuffer.from_numpy(x["q"][:, :, 0])
    caches = []
    for r in range(rotate):
        kk = np.roll(x["k"], r, axis=0)
        vv = np.roll(x["v"], r, axis=0)
        caches.append((rocm.DeviceBuffer.from_numpy(kk), rocm.DeviceBuffer.from_numpy(vv)))
    ob = rocm.DeviceBuffer((B, H, D), np.float16)
    scale = rocm.default_scale(D)

    def call(i):
        kb, vb = caches[i % rotate]
        rocm.attn_decode_raw(np.float16, qb.ptr, kb.ptr, vb.ptr, ob.ptr, B, H, L, D, scale)

    for i in range(warmup):
        call(i)
    rocm.sync()
    # one event pair around all the calls, as for the attention kernels: a pair per launch adds
    # about 5 us of command-processor work to each
    timer = rocm.Timer()
    timer.start()
    for i in range(steps):
        call(i)
    timer.stop()
    rocm.sync()
    nbytes = 2.0 * B * H * L * D * 2 + 2 * B * H * D * 2
    total_us = 1e3 * timer.elapsed_ms() / steps  # the whole call: main kernel (+ merge when a head is split)
    return dict(bytes=nbytes, kernel_us=total_us, call_us=total_us,
                gbs_kernel=nbytes / (total_us * 1e-6) / 1e9,
                gbs_call=nbytes / (total_us * 1e-6) / 1e9)


def bench_copy(steps: int, warmup: int):
    """Plain device copy of known size through the library's copy kernel: 256 MiB read
    and 256 MiB written per launch.  It exists to calibrate hardware byte counters
    (what FETCH_SIZE / WRITE_SIZE report for a kernel whose traffic is known)."""
    n = 128 * 1024 * 1024  # f16 elements
    src = rocm.DeviceBuffer((n,), np.float16, zeros=True)
    dst = rocm.DeviceBuffer((n,), np.float16)
    for _ in range(warmup):
        rocm.copy_compact_raw(np.float16, src.ptr, (n,), (1,), dst.ptr)
    rocm.sync()
    timer = rocm.Timer()
    timer.start()
    for _ in range(steps):
        rocm.copy_compact_raw(np.float16, src.ptr, (n,), (1,), dst.ptr)
    timer.stop()
    rocm.sync()
    us = 1e3 * timer.elapsed_ms() / steps
    return dict(bytes_read=2 * n, bytes_written=2 * n, kernel_us=us,
                gbs=4.0 * n / (us * 1e-6) / 1e9)


def bench_rope(steps: int, warmup: int):
    """RoPE + head split (forward) and inverse RoPE + head merge (backward) at the C2
    geometry; HBM-bound: each launch reads one [B,T,H,D] tensor and writes one."""
    B, H, T, D = C2["B"], C2["H"], C2["T"], C2["D"]
    cos, sin = synth.rotary_tables(T, D, dtype=np.float16)
    x = synth.normal((B, T, H, D), synth.tensor_seed(0, "rope", "x"), 1.0).astype(np.float16)
    dx, dc, ds = (rocm.DeviceBuffer.from_numpy(a) for a in (x, cos, sin))
    y = rocm.DeviceBuffer((B, H, T, D), np.float16)
    g = rocm.DeviceBuffer((B, T, H, D), np.float16)

    def step():
        rocm.rope_fwd_raw(np.float16, dx.ptr, dc.ptr, ds.ptr, y.ptr, B, T, H, D)
        rocm.rope_bwd_raw(np.float16, y.ptr, dc.ptr, ds.ptr, g.ptr, B, T, H, D)

    for _ in range(warmup):
        step()
    rocm.sync()
    rocm.profile_enable(True)
    for _ in range(steps):
        step()
    prof = rocm.profile_collect()
    rocm.profile_enable(False)
    nbytes = 2.0 * B * T * H * D * 2
    out = {"bytes_per_launch": nbytes}
    for name, (calls, ms) in prof.items():
        us = 1e3 * ms / calls
        out[name] = {"avg_us": us, "GB/s": nbytes / (us * 1e-6) / 1e9}
    return out


def bench_log_softmax(steps: int, warmup: int):
    """Row-wise log-softmax forward and backward at config 5's logits, [8192, 50257] f32
    (1.65 GB).  HBM-bound: the forward must read x and write y (2 x 1.65 GB), the
    backward read grad and y and write dx (3 x 1.65 GB); the second sweep over each
    201 KB row is served by L2."""
    outer, inner = 8192, 50257
    rows = synth.normal((256, inner), synth.tensor_seed(0, "lsm", "x"), 2.0).astype(np.float32)
    x = rocm.DeviceBuffer((outer, inner), np.float32)
    for r in range(0, outer, 256):  # the same 256 rows tiled: content does not change the work
        rocm._check(rocm.load().deers_rocm_htod(
            ctypes.c_void_p(x.ptr.value + r * inner * 4),
            rows.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(rows.nbytes)))
    y = rocm.DeviceBuffer((outer, inner), np.float32)
    g = rocm.DeviceBuffer((outer, inner), np.float32, zeros=True)
    d = rocm.DeviceBuffer((outer, inner), np.float32)

    def step():
        rocm.log_softmax_fwd_raw(np.float32, x.ptr, y.ptr, outer, inner)
        rocm.log_softmax_bwd_raw(np.float32, g.ptr, y.ptr, d.ptr, outer, inner)

    for _ in range(warmup):
        step()
    rocm.sync()
    rocm.profile_enable(True)
    for _ in range(steps):
        step()
    prof = rocm.profile_collect()
    rocm.profile_enable(False)
    one = float(outer) * inner * 4
    alg = {"log_softmax_fwd": 2 * one, "log_softmax_bwd": 3 * one}
    out = {"shape": [outer, inner], "dtype": "f32"}
    for name, (calls, ms) in prof.items():
        us = 1e3 * ms / calls
        out[name] = {"avg_us": us, "bytes_per_launch": alg[name],
                     "GB/s": alg[name] / (us * 1e-6) / 1e9,
                     "frac_hbm_peak": alg[name] / (us * 1e-6) / 1e9 / PEAK_HBM_GBS}
    return out


def bench_composed_chain(steps: int, warmup: int):
    """C2's forward as the reference's own op chain on the device (seven storage kernels and
    two [8,12,1024,1024] f16 intermediates, rocm.attn_fwd_composed_raw) beside the fused kernel
    on the same inputs: what fusing buys on this GPU, not a headline number."""
    B, H, T, D = C2["B"], C2["H"], C2["T"], C2["D"]
    dt = np.float16
    q, k, v = (rocm.DeviceBuffer.from_numpy(
        synth.normal((B, H, T, D), synth.tensor_seed(0, "c2", n), 1.0).astype(dt)) for n in "qkv")
    mask = rocm.DeviceBuffer.from_numpy(rocm.causal_mask_host(B, T, dt))
    o = rocm.DeviceBuffer((B, H, T, D), dt)
    lse16 = rocm.DeviceBuffer((B, H, T), dt)
    lse32 = rocm.DeviceBuffer((B, H, T), np.float32)
    s, p = rocm.DeviceBuffer((B, H, T, T), dt), rocm.DeviceBuffer((B, H, T, T), dt)
    scale = rocm.default_scale(D)
    reps = max(5, steps // 10)
    times = {}
    for name, fn in (("composed", lambda: rocm.attn_fwd_composed_raw(dt, q.ptr, k.ptr, v.ptr, mask.ptr, o.ptr,
                                                                     lse16.ptr, s.ptr, p.ptr, B, H, T, D, scale)),
                     ("fused", lambda: rocm.attn_fwd_raw(dt, q.ptr, k.ptr, v.ptr, o.ptr, lse32.ptr, B, H, T, D, scale))):
        for _ in range(3):
            fn()
        rocm.sync()
        t = rocm.Timer()
        t.start()
        for _ in range(reps):
            fn()
        t.stop()
        times[name] = 1e3 * t.elapsed_ms() / reps
    return {"composed_chain_us": times["composed"], "fused_kernel_us": times["fused"],
            "ratio": times["composed"] / times["fused"],
            "intermediate_bytes": 2.0 * B * H * T * T * 2}


def bench_storage(steps: int, warmup: int):
    """The generic storage kernels at the shapes the reference's unfused attention chain gives
    them at C2's geometry in f32 (src/models/gpt.rs:139-144: scores [8,12,1024,1024] = 403 MB):
    scalar_mul, add of the head-broadcast mask, log_sum_exp over the rows, sub of the
    row-broadcast lse, exp; plus row sum / max, a transposed (strided) unary pass, and the
    loss's gather / scatter_add at [8192, 50257].  All HBM-bound; bytes are the algorithmic
    minimum (every operand once)."""
    B, H, T = C2["B"], C2["H"], C2["T"]
    n = B * H * T * T
    one = 4.0 * n
    x = rocm.DeviceBuffer((B, H, T, T), np.float32)
    rocm.fill_raw(np.float32, x.ptr, n, 0.25)
    y = rocm.DeviceBuffer((B, H, T, T), np.float32)
    z = rocm.DeviceBuffer((B, H, T, T), np.float32)
    mask = rocm.DeviceBuffer((B, 1, T, T), np.float32, zeros=True)
    rows = rocm.DeviceBuffer((B * H * T,), np.float32)
    nv, vv = 8192, 50257
    logp = rocm.DeviceBuffer((nv, vv), np.float32)  # 1.65 GB
    rocm.fill_raw(np.float32, logp.ptr, nv * vv, -10.0)
    tgt = rocm.DeviceBuffer.from_numpy(
        (np.arange(nv, dtype=np.int64) * 7919 % vv).reshape(nv, 1))
    pick = rocm.DeviceBuffer((nv, 1), np.float32)
    shape = (B, H, T, T)
    plan = [
        ("unary_scalar_mul", 2 * one, lambda: rocm.unary_raw(np.float32, "scalar_mul", x.ptr, shape, None, 0.125, y.ptr)),
        ("binary_add", 2 * one + 4.0 * B * T * T,
         lambda: rocm.binary_raw(np.float32, "add", y.ptr, None, mask.ptr, [T * T, 0, T, 1], shape, z.ptr)),
        ("log_sum_exp", one, lambda: rocm.log_sum_exp_raw(np.float32, z.ptr, rows.ptr, B * H * T, T)),
        ("binary_sub", 2 * one + 4.0 * B * H * T,
         lambda: rocm.binary_raw(np.float32, "sub", z.ptr, None, rows.ptr, [H * T, T, 1, 0], shape, y.ptr)),
        ("unary_exp", 2 * one, lambda: rocm.unary_raw(np.float32, "exp", y.ptr, shape, None, 0.0, z.ptr)),
        ("binary_mul", 3 * one, lambda: rocm.binary_raw(np.float32, "mul", x.ptr, None, z.ptr, None, shape, y.ptr)),
        ("reduce_sum", one, lambda: rocm.reduce_raw(np.float32, "sum", z.ptr, rows.ptr, B * H * T, T)),
        ("reduce_max", one, lambda: rocm.reduce_raw(np.float32, "max", z.ptr, rows.ptr, B * H * T, T)),
        ("unary_neg", 2 * one,  # last two axes swapped: the strided path
         lambda: rocm.unary_raw(np.float32, "neg", x.ptr, shape, [H * T * T, T * T, 1, T], 0.0, y.ptr)),
        ("gather", 16.0 * nv, lambda: rocm.gather_raw(np.float32, logp.ptr, tgt.ptr, pick.ptr, nv, vv, 1, 1)),
        ("scatter_add", 20.0 * nv, lambda: rocm.scatter_add_raw(np.float32, pick.ptr, tgt.ptr, logp.ptr, nv, vv, 1, 1)),
    ]
    strided_name = "unary_neg"
    out = {"shape": list(shape), "dtype": "f32"}
    out["attention_forward_composed_f16_c2"] = bench_composed_chain(steps, warmup)
    for name, nbytes, fn in plan:
        for _ in range(max(1, warmup // 4)):
            fn()
        rocm.sync()
        rocm.profile_enable(True)
        for _ in range(max(3, steps // 10)):
            fn()
        prof = rocm.profile_collect()
        rocm.profile_enable(False)
        calls, ms = prof[name]
        us = 1e3 * ms / calls
        key = name + ("_transposed_view" if name == strided_name else "")
        out[key] = {"avg_us": us, "bytes_per_launch": nbytes, "GB/s": nbytes / (us * 1e-6) / 1e9,
                    "frac_hbm_peak": nbytes / (us * 1e-6) / 1e9 / PEAK_HBM_GBS}
    return out


def bench_adamw(steps: int, warmup: int):
    """Fused AdamW step over 124,439,808 f32 parameters (GPT-2 small, as one tensor), and
    the sum of squares of as many gradients.  HBM-bound: the step reads w, g, m, v and
    writes w, m, v (28 B per parameter); the reduction reads g (4 B)."""
    n = 124_439_808
    w = rocm.DeviceBuffer((n,), np.float32)
    rocm.fill_raw(np.float32, w.ptr, n, 0.02)
    g = rocm.DeviceBuffer((n,), np.float32)
    rocm.fill_raw(np.float32, g.ptr, n, 1e-3)
    m = rocm.DeviceBuffer((n,), np.float32, zeros=True)
    v = rocm.DeviceBuffer((n,), np.float32, zeros=True)
    total = rocm.DeviceBuffer((1,), np.float32)
    t = [0]

    def step():
        t[0] += 1
        rocm.sum_squares_raw(np.float32, g.ptr, n, total.ptr)
        rocm.adamw_step_raw(np.float32, w.ptr, g.ptr, m.ptr, v.ptr, n, 3e-4, 0.9, 0.95, 1e-8, 0.1,
                            t[0], 0.5)

    for _ in range(warmup):
        step()
    rocm.sync()
    rocm.profile_enable(True)
    for _ in range(steps):
        step()
    prof = rocm.profile_collect()
    rocm.profile_enable(False)
    alg = {"adamw_step": 28.0 * n, "sumsq": 4.0 * n}
    out = {"parameters": n, "dtype": "f32"}
    for name, (calls, ms) in prof.items():
        us = 1e3 * ms / calls
        out[name] = {"avg_us": us, "bytes_per_launch": alg[name],
                     "GB/s": alg[name] / (us * 1e-6) / 1e9,
                     "frac_hbm_peak": alg[name] / (us * 1e-6) / 1e9 / PEAK_HBM_GBS}
    return out


def bench_gpt(steps: int, warmup: int):
    """End-to-end GPT training step (BASELINE configs[4]): f32 parameters, 12 layers,
    12 heads, n_embd 768, MLP 3072, vocabulary 50257, sequence 1024, batch 8; forward,
    cross-entropy, backward, gradient-norm clipping, AdamW, all on the device through the
    C++ host (deers_amd/host/gpt_step), with the library's GEMM kernel picked per problem by
    timing during the untimed warm-up steps.  Reports the step time and tokens per second
    and the time per kernel family from a profiled pass."""
    import subprocess
    exe = os.path.join(ROOT, "deers_amd", "host", "gpt_step")
    if not os.path.exists(exe):
        raise RuntimeError("deers_amd/host/gpt_step is not built (run __graft_entry__.build())")
    cfg = {"vocab_size": 50257, "seq_len": 1024, "n_layer": 12, "n_head": 12, "n_embd": 768,
           "mlp_hidden": 3072, "batch": 8}
    r = subprocess.run([exe] + [str(cfg[k]) for k in ("vocab_size", "seq_len", "n_layer", "n_head",
                                                      "n_embd", "mlp_hidden", "batch")]
                       + [str(steps), str(warmup), "tune"], capture_output=True, text=True, timeout=600)
    if r.returncode != 0:
        raise RuntimeError("gpt_step failed: " + r.stderr.strip())
    out = json.loads(r.stdout.strip().splitlines()[-1])
    tokens = cfg["batch"] * cfg["seq_len"]
    # matrix-product work: every Linear (blocks + LM head) forward and both backward products
    linear_params = cfg["n_layer"] * (4 * cfg["n_embd"] ** 2 + 2 * cfg["n_embd"] * cfg["mlp_hidden"]) \
        + cfg["n_embd"] * cfg["vocab_size"]
    gemm_flops = 6.0 * linear_params * tokens
    fwd_f, bwd_f = attn_flops(cfg["batch"], cfg["n_head"], cfg["seq_len"], cfg["n_embd"] // cfg["n_head"])
    attn = cfg["n_layer"] * (fwd_f + bwd_f)
    out["workload"] = ("GPT training step, f32, 12 layers x 12 heads x 768, MLP 3072, vocab 50257, "
                       "seq 1024, batch 8 (BASELINE configs[4]); synthetic token ids, random-init weights")
    out["flops_per_step"] = {"matmul": gemm_flops, "attention": attn}
    out["model_tflops"] = (gemm_flops + attn) / (out["ms_per_step"] * 1e-3) / 1e12
    # greedy generation with KV caches on the same architecture in f16 (32 sequences, 512 cached
    # tokens, 256 new ones): one decode step = one pass over the weights and the caches
    rg = subprocess.run([exe, "generate"] + [str(cfg[k]) for k in ("vocab_size", "seq_len", "n_layer",
                                                                     "n_head", "n_embd", "mlp_hidden")]
                        + ["32", "512", "256"], capture_output=True, text=True, timeout=600)
    if rg.returncode == 0:
        out["generation_f16"] = json.loads(rg.stdout.strip().splitlines()[-1])
    else:
        out["generation_f16"] = {"error": rg.stderr.strip()}
    mm = out["kernels"].get("matmul")
    if mm:
        mm["tflops"] = gemm_flops / (mm["ms_per_step"] * 1e-3) / 1e12
        mm["frac_f32_matrix_peak"] = mm["tflops"] / 157.3
    return out


def cpu_baseline_gpt():
    """The composed CPU oracle (numpy GEMMs on all host threads + the C attention oracle) on
    a bounded sample of the GPT step: one of the 8 sequences (batch 1, T = 1024) through the
    full 12-layer model, forward + loss + backward + AdamW, timed once after no warm-up.
    kind "port": the Rust reference cannot be built here."""
    import oracle  # the checker; only ever the thing measured in this baseline leg
    from oracle import gpt as ogpt
    cfg = dict(vocab_size=50257, sequence_len=1024, n_layer=12, n_head=12, n_embd=768,
               mlp_hidden_dim=3072, rms_norm_eps=1e-5, rope_base=10000.0)
    rng = np.random.default_rng(0)
    C, Hd, V = cfg["n_embd"], cfg["mlp_hidden_dim"], cfg["vocab_size"]
    uni = lambda r, c: rng.uniform(-1 / np.sqrt(r), 1 / np.sqrt(r), (r, c)).astype(np.float32)
    w = [rng.standard_normal((V, C)).astype(np.float32)]
    for _ in range(cfg["n_layer"]):
        w += [uni(C, C), uni(C, C), uni(C, C), uni(C, C), uni(C, Hd), uni(Hd, C)]
    w.append(uni(C, V))
    ids = rng.integers(0, V, (1, 1024))
    targets = rng.integers(0, V, 1024)
    mom = [(np.zeros_like(a), np.zeros_like(a)) for a in w]
    t0 = time.perf_counter()
    ogpt.train_step(cfg, w, mom, 1, ids, targets, 3e-4, (0.9, 0.95), 1e-8, 0.1, max_norm=1.0)
    sec = time.perf_counter() - t0
    return {"value": 1024 / sec, "unit": "tokens/s", "cores": oracle.max_threads(), "kind": "port",
            "seconds_per_step": sec,
            "sample": "1 of the 8 sequences (batch 1, T=1024), whole 12-layer model, one training step"}


def cpu_baseline():
    """The CPU oracle (kind "port": a restatement of the reference's materialised CPU
    attention; the Rust reference itself cannot be built here) on the full B=8 H=12
    T=1024 D=64 problem, 1 warm-up + 2 timed fwd+bwd passes, median.  GEMMs use all
    host threads, element-wise passes one thread, mirroring the reference."""
    import oracle  # the checker; only ever the thing measured in this baseline leg
    B, H, T, D = C2["B"], C2["H"], C2["T"], C2["D"]
    x = synth.attention_inputs("c2", B, H, T, D, np.float16, base_seed=0)
    q, k, v, do = (x[n].astype(np.float32) for n in ("q", "k", "v", "do"))
    threads = oracle.max_threads()
    times = []
    for it in range(3):
        t0 = time.perf_counter()
        oracle.attn_fwd(q, k, v, nthreads=threads)
        oracle.attn_bwd(q, k, v, do, nthreads=threads)
        if it > 0:
            times.append(time.perf_counter() - t0)
    sec = statistics.median(times)
    fwd, bwd = attn_flops(B, H, T, D)
    return {"value": (fwd + bwd) / sec / 1e12, "unit": "TFLOP/s", "cores": threads,
            "kind": "port", "seconds_per_step": sec,
            "sample": "full workload (B=8 H=12 T=1024 D=64, f32 on the f16-rounded inputs), "
                      "1 warm-up + 2 timed fwd+bwd passes, median"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gpt", action="store_true",
                    help="skip the end-to-end GPT training step reported beside the headline")
    ap.add_argument("--only", choices=["all", "fwd", "bwd", "c1", "c3", "c2_d128", "c5_attn", "decode", "copy", "rope", "log_softmax", "adamw", "gpt", "storage"], default="all",
                    help="profiling aid: launch only this part and print its kernel times "
                         "(the headline JSON line needs the default, all)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the attention path has no cross-GPU exchange "
                 "(it shards over batch x heads with no communication); run with --gpus 1")
    if not rocm.available():
        sys.exit("no gfx950 device visible: the attention path has no CPU fallback")
    rocm.init(0)

    if args.only != "all":
        if args.only == "decode":
            print(json.dumps({"only": "decode", **bench_decode(args.steps, args.warmup)}))
        elif args.only == "rope":
            print(json.dumps({"only": "rope", **bench_rope(args.steps, args.warmup)}))
        elif args.only == "log_softmax":
            print(json.dumps({"only": "log_softmax",
                              **bench_log_softmax(min(args.steps, 20), min(args.warmup, 5))}))
        elif args.only == "adamw":
            print(json.dumps({"only": "adamw",
                              **bench_adamw(min(args.steps, 20), min(args.warmup, 5))}))
        elif args.only == "storage":
            print(json.dumps({"only": "storage", **bench_storage(args.steps, args.warmup)}))
        elif args.only == "gpt":
            print(json.dumps({"only": "gpt", **bench_gpt(min(args.steps, 10), min(args.warmup, 3))}))
        elif args.only == "copy":
            print(json.dumps({"only": "copy", **bench_copy(args.steps, args.warmup)}))
        elif args.only in EXTRA_CONFIGS:
            print(json.dumps({"only": args.only,
                              **bench_attention_config(launches=max(50, min(args.steps, 200)), **EXTRA_CONFIGS[args.only])}))
        else:
            tr = bench_train(args.steps, args.warmup, args.only)
            print(json.dumps({"only": args.only, "kernels": tr["kernels"]}))
        return

    B, H, T, D = C2["B"], C2["H"], C2["T"], C2["D"]
    fwd_f, bwd_f = attn_flops(B, H, T, D)
    tr = bench_train(args.steps, args.warmup)
    ms_per_step = tr["dev_ms"] / args.steps
    tflops = (fwd_f + bwd_f) / (ms_per_step * 1e-3) / 1e12

    # dominant kernel of the step and its roofline
    kern = tr["kernels"]
    dom = max(kern, key=lambda n: kern[n]["avg_us"] * kern[n]["calls"])
    # Algorithmic FLOPs per launch (FlashAttention convention, causal-halved): forward = 2 tile
    # GEMMs = 4*B*H*T^2*D/2, backward = 2.5 x forward (5 tile GEMMs).  The backward kernel
    # really executes 7 (its two halves each recompute S and dP): that figure is reported
    # beside the algorithmic one, never used for `frac`.
    gemm = 2.0 * B * H * T * T * D / 2.0
    algorithmic_flops = {"attn_fwd_f16": fwd_f, "attn_bwd_f16": bwd_f}
    executed_flops = {"attn_fwd_f16": 2 * gemm, "attn_bwd_f16": 7 * gemm}
    for n, st in kern.items():
        if n in algorithmic_flops:
            st["tflops"] = algorithmic_flops[n] / (st["avg_us"] * 1e-6) / 1e12
            st["frac_mfma_peak"] = st["tflops"] / PEAK_F16_TFLOPS
            st["executed_tflops"] = executed_flops[n] / (st["avg_us"] * 1e-6) / 1e12
    achieved = kern[dom].get("tflops")
    # HBM bytes per launch at this shape: rocprofv3 FETCH_SIZE / WRITE_SIZE passes, scaled by
    # what the same counters read for a copy of known size.  A profiler measurement kept in
    # the named file, not taken in this run.
    measured_traffic = {"attn_bwd_f16": 161.4e6, "attn_fwd_f16": 51.0e6}
    roofline = {"kernel": dom, "bound": "mfma", "achieved": achieved, "peak": PEAK_F16_TFLOPS,
                "unit": "TFLOP/s", "frac": (achieved / PEAK_F16_TFLOPS) if achieved else None,
                "traffic": measured_traffic.get(dom),
                "traffic_source": "profiles/c2_c4_hbm_traffic_fetch_write.txt (rocprofv3 --pmc, not this run)",
                "avg_launch_us": kern[dom]["avg_us"], "launches_timed": kern[dom]["calls"],
                "flops_per_launch": algorithmic_flops.get(dom),
                "executed_flops_per_launch": executed_flops.get(dom)}

    dec_calls = max(args.steps, 50)
    dec = bench_decode(dec_calls, max(args.warmup, 10))

    out = {
        "metric": "causal attn fwd+bwd TFLOP/s & %MFMA peak (T=1024,D=64,f16); decode HBM GB/s",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "warmup_effective": tr["warmup_effective"], "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "causal self-attention fwd+bwd, f16 in / f32 accumulate, "
                               "B=8 H=12 T=1024 D=64 (BASELINE configs[1])",
                   "flops_per_step": fwd_f + bwd_f, "flop_convention": "7*B*H*T^2*D"},
        "frac_mfma_peak": tflops / PEAK_F16_TFLOPS,
        "peak_tflops_f16_dense": PEAK_F16_TFLOPS,
        "timed_region": "`warmup` untimed + exactly `steps` timed fwd+bwd steps, run after the settling pass "
                        "(%d steps) and the per-kernel pass (%d launches of each kernel between one event pair), "
                        "so that short runs see settled clocks: `warmup_effective` counts all of them"
                        % (max(args.steps, KERNEL_PASS_MIN_STEPS), max(args.steps, KERNEL_PASS_MIN_STEPS)),
        "wall_ms_per_step": tr["wall_ms"] / args.steps,
        "step_us_event_pairs": tr["step_us"],
        "kernels": kern,
        "roofline": roofline,
        "decode": {"workload": "decode f16 B=32 H=12 L=4096 D=64 (BASELINE configs[3]), "
                               "4 KV caches in rotation",
                   "timing": "one event pair around %d back-to-back calls" % dec_calls,
                   "bytes_per_call": dec["bytes"], "kernel_us": dec["kernel_us"],
                   "call_us": dec["call_us"], "GB/s": dec["gbs_kernel"],
                   "GB/s_whole_call": dec["gbs_call"], "peak_GB/s": PEAK_HBM_GBS,
                   "frac_hbm_peak": dec["gbs_kernel"] / PEAK_HBM_GBS},
    }
    # BASELINE configs[0] and configs[2] (and configs[1]'s shape at head width 128), reported
    # beside the headline, never part of `value`
    for name, cfg in EXTRA_CONFIGS.items():
        try:
            out[name] = bench_attention_config(**cfg)
        except Exception as e:  # the headline line must not depend on them
            out[name] = {"error": str(e)}
    if not args.no_gpt:
        # BASELINE configs[4], reported beside the headline (never part of `value`)
        try:
            g = bench_gpt(5, 2)
            out["gpt_train_step"] = {k: g[k] for k in ("workload", "ms_per_step", "tokens_per_s",
                                                       "parameters", "model_tflops", "kernels",
                                                       "generation_f16")}
        except Exception as e:  # the headline line must not depend on it
            out["gpt_train_step"] = {"error": str(e)}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        if "gpt_train_step" in out and "error" not in out["gpt_train_step"]:
            try:
                out["gpt_train_step"]["cpu_baseline"] = cpu_baseline_gpt()
            except Exception as e:
                out["gpt_train_step"]["cpu_baseline"] = {"error": str(e)}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
