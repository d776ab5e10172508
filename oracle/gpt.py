"""CPU restatement of the reference's GPT training step (TEST INFRASTRUCTURE, not product
code): GPT::forward (src/models/gpt.rs:328-355), loss::cross_entropy (src/loss.rs:21-24),
the reverse sweep through the ops it is built from, and AdamW (src/optim.rs:214-251),
composed from the functions of this package.  Weights are a list in parameters() order
(src/models/gpt.rs:357-365): wte [V,C]; per block q, k, v, out [C,C], up [C,H], down
[H,C]; lm_head [C,V]; every Linear is y = x @ W (src/nn.rs:183-190)."""
from __future__ import annotations

import numpy as np

import oracle


def _block_weights(weights, layer):
    return weights[1 + 6 * layer: 7 + 6 * layer]


def gpt_forward(cfg: dict, weights, ids, dtype=np.float32, keep=False):
    """Logits [B,T,V]; with keep=True also the activations the backward needs."""
    B, T = ids.shape
    C, H = cfg["n_embd"], cfg["n_head"]
    D = C // H
    eps = cfg["rms_norm_eps"]
    w = [np.asarray(a, dtype=dtype) for a in weights]
    cos, sin = oracle.rope_tables(T, D, base=cfg["rope_base"], dtype=np.float32)
    cos, sin = cos.astype(dtype), sin.astype(dtype)
    x = oracle.index_select(w[0], ids.reshape(-1)).reshape(B, T, C)
    saved = []
    for layer in range(cfg["n_layer"]):
        wq, wk, wv, wo, up, down = _block_weights(w, layer)
        n1 = oracle.rms_norm_fwd(x, eps, dtype=dtype)
        flat = n1.reshape(B * T, C)
        q = (flat @ wq).reshape(B, T, H, D)
        k = (flat @ wk).reshape(B, T, H, D)
        v = (flat @ wv).reshape(B, T, H, D)
        qh = oracle.rope_apply(q, cos, sin, dtype=dtype).transpose(0, 2, 1, 3)
        kh = oracle.rope_apply(k, cos, sin, dtype=dtype).transpose(0, 2, 1, 3)
        vh = v.transpose(0, 2, 1, 3)
        y = oracle.attn_fwd(qh, kh, vh, dtype=dtype)                    # [B,H,T,D]
        merged = np.ascontiguousarray(y.transpose(0, 2, 1, 3)).reshape(B * T, C)
        h = x + (merged @ wo).reshape(B, T, C)
        n2 = oracle.rms_norm_fwd(h, eps, dtype=dtype)
        pre = n2.reshape(B * T, C) @ up                                  # [B*T, Hd]
        act = oracle.relu_sq_fwd(pre)
        out = h + (act @ down).reshape(B, T, C)
        saved.append((x, n1, qh, kh, vh, merged, h, n2, pre, act))
        x = out
    nf = oracle.rms_norm_fwd(x, eps, dtype=dtype)
    logits = (nf.reshape(B * T, C) @ w[-1]).reshape(B, T, cfg["vocab_size"])
    if keep:
        return logits, (w, cos, sin, saved, x, nf)
    return logits


def gpt_loss_and_grads(cfg: dict, weights, ids, targets, dtype=np.float32):
    """(loss, [gradient per weight]) of cross_entropy(GPT(ids).reshape(B*T, V), targets)."""
    B, T = ids.shape
    C, H, V = cfg["n_embd"], cfg["n_head"], cfg["vocab_size"]
    D = C // H
    eps = cfg["rms_norm_eps"]
    logits, (w, cos, sin, saved, x_last, nf) = gpt_forward(cfg, weights, ids, dtype=dtype, keep=True)
    flat_logits = logits.reshape(B * T, V)
    loss = oracle.cross_entropy_fwd(flat_logits, targets, dtype=dtype)
    grads = [None] * len(w)
    dlogits = oracle.cross_entropy_bwd(flat_logits, targets, dtype=dtype)          # [B*T, V]
    grads[-1] = nf.reshape(B * T, C).T @ dlogits
    dnf = (dlogits @ w[-1].T).reshape(B, T, C)
    dx = oracle.rms_norm_bwd(x_last, dnf, eps, dtype=dtype)
    for layer in reversed(range(cfg["n_layer"])):
        wq, wk, wv, wo, up, down = _block_weights(w, layer)
        x, n1, qh, kh, vh, merged, h, n2, pre, act = saved[layer]
        # out = h + down(relu_sq(up(norm2(h))))
        dflat = dx.reshape(B * T, C)
        grads[1 + 6 * layer + 5] = act.T @ dflat
        dact = dflat @ down.T
        dpre = oracle.relu_sq_bwd(pre, dact.astype(pre.dtype))
        grads[1 + 6 * layer + 4] = n2.reshape(B * T, C).T @ dpre
        dn2 = (dpre @ up.T).reshape(B, T, C)
        dh = dx + oracle.rms_norm_bwd(h, dn2, eps, dtype=dtype)
        # h = x + out_proj(merge(attn(rope(q), rope(k), v)))
        dhf = dh.reshape(B * T, C)
        grads[1 + 6 * layer + 3] = merged.T @ dhf
        dmerged = (dhf @ wo.T).reshape(B, T, H, D).transpose(0, 2, 1, 3)        # [B,H,T,D]
        dqh, dkh, dvh = oracle.attn_bwd(qh, kh, vh, dmerged, dtype=dtype)
        dq = oracle.rope_apply_bwd(dqh.transpose(0, 2, 1, 3), cos, sin, dtype=dtype).reshape(B * T, C)
        dk = oracle.rope_apply_bwd(dkh.transpose(0, 2, 1, 3), cos, sin, dtype=dtype).reshape(B * T, C)
        dv = np.ascontiguousarray(dvh.transpose(0, 2, 1, 3)).reshape(B * T, C)
        flat = n1.reshape(B * T, C)
        grads[1 + 6 * layer + 0] = flat.T @ dq
        grads[1 + 6 * layer + 1] = flat.T @ dk
        grads[1 + 6 * layer + 2] = flat.T @ dv
        dn1 = (dq @ wq.T + dk @ wk.T + dv @ wv.T).reshape(B, T, C)
        dx = dh + oracle.rms_norm_bwd(x, dn1, eps, dtype=dtype)
    grads[0] = oracle.index_add(V, dx.reshape(B * T, C), ids.reshape(-1))
    return loss, [g.astype(dtype) for g in grads]


def train_step(cfg: dict, weights, moments, step: int, ids, targets, lr: float, betas=(0.9, 0.999),
               eps: float = 1e-8, weight_decay: float = 0.0, max_norm: float | None = None,
               dtype=np.float32):
    """One step of the reference's training loop (examples/tinystories_train.rs): loss,
    backward, optional clip_grad_norm, AdamW.  `moments` is a list of (m, v) per weight.
    Returns (loss, norm or None, new weights, new moments)."""
    loss, grads = gpt_loss_and_grads(cfg, weights, ids, targets, dtype=dtype)
    norm = None
    if max_norm is not None:
        norm, grads = oracle.clip_grad_norm(grads, max_norm, dtype=dtype)
    new_w, new_m = [], []
    for w, g, (m, v) in zip(weights, grads, moments):
        w2, m2, v2 = oracle.adamw_step(w, g, m, v, step, lr, betas, eps, weight_decay, dtype=dtype)
        new_w.append(w2)
        new_m.append((m2, v2))
    return loss, norm, new_w, new_m
