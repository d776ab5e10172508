"""Pins of the composed GPT oracle (oracle/gpt.py): an independent torch model in float64
with autograd (a library, as the reference's tests/gpt.rs uses candle), and central
differences of the oracle's own forward."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import gpt as ogpt

# the reference's test configuration (tests/gpt.rs:39-50), and one with a head width the
# device kernels support
REF_CFG = dict(vocab_size=8, sequence_len=4, n_layer=1, n_head=2, n_embd=4, mlp_hidden_dim=8,
               rms_norm_eps=1e-5, rope_base=10000.0)
CFG32 = dict(vocab_size=37, sequence_len=16, n_layer=2, n_head=2, n_embd=64, mlp_hidden_dim=96,
             rms_norm_eps=1e-5, rope_base=10000.0)
REF_IDS = np.int64([[1, 2, 3], [4, 3, 2]])      # tests/gpt.rs:52-58
REF_TARGETS = np.int64([2, 3, 4, 3, 2, 1])      # tests/gpt.rs:60-66


def make_weights(cfg, seed, dtype=np.float64):
    rng = np.random.default_rng(seed)
    C, Hd, V = cfg["n_embd"], cfg["mlp_hidden_dim"], cfg["vocab_size"]
    uni = lambda r, c: rng.uniform(-1 / math.sqrt(r), 1 / math.sqrt(r), (r, c))
    w = [rng.standard_normal((V, C))]
    for _ in range(cfg["n_layer"]):
        w += [uni(C, C), uni(C, C), uni(C, C), uni(C, C), uni(C, Hd), uni(Hd, C)]
    w.append(uni(C, V))
    return [a.astype(dtype) for a in w]


def torch_gpt_loss(cfg, weights, ids, targets):
    """The same model from torch's own building blocks, float64."""
    F = torch.nn.functional
    B, T = ids.shape
    C, H = cfg["n_embd"], cfg["n_head"]
    D = C // H
    w = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in weights]
    half = D // 2
    inv_freq = 1.0 / (cfg["rope_base"] ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    ang = torch.arange(T, dtype=torch.float64)[:, None] * inv_freq[None, :]
    cos, sin = ang.cos()[None, :, None, :], ang.sin()[None, :, None, :]

    def rope(x):  # [B,T,H,D]
        x1, x2 = x[..., :half], x[..., half:]
        return torch.cat([x1 * cos + x2 * sin, -x1 * sin + x2 * cos], dim=-1)

    norm = lambda x: F.rms_norm(x, (C,), eps=cfg["rms_norm_eps"])
    x = F.embedding(torch.tensor(ids), w[0])
    for layer in range(cfg["n_layer"]):
        wq, wk, wv, wo, up, down = w[1 + 6 * layer: 7 + 6 * layer]
        n1 = norm(x)
        q = rope((n1 @ wq).view(B, T, H, D)).transpose(1, 2)
        k = rope((n1 @ wk).view(B, T, H, D)).transpose(1, 2)
        v = (n1 @ wv).view(B, T, H, D).transpose(1, 2)
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + y.transpose(1, 2).reshape(B, T, C) @ wo
        x = x + (norm(x) @ up).relu().square() @ down
    logits = norm(x) @ w[-1]
    loss = F.cross_entropy(logits.view(B * T, -1), torch.tensor(targets))
    loss.backward()
    return logits.detach().numpy(), float(loss.detach()), [a.grad.numpy() for a in w]


@pytest.mark.parametrize("cfg,ids,targets", [
    (REF_CFG, REF_IDS, REF_TARGETS),
    (CFG32, None, None),
])
def test_gpt_oracle_matches_torch_autograd(cfg, ids, targets):
    rng = np.random.default_rng(3)
    if ids is None:
        ids = rng.integers(0, cfg["vocab_size"], (3, 11))
        ids[1, 4:8] = ids[0, 0]  # repeated tokens exercise the embedding scatter
        targets = rng.integers(0, cfg["vocab_size"], ids.size)
    w = make_weights(cfg, 5)
    # float32 inputs of the rope tables limit agreement to ~1e-7 relative
    logits, loss_t, grads_t = torch_gpt_loss(cfg, w, ids, targets)
    got_logits = ogpt.gpt_forward(cfg, w, ids, dtype=np.float64)
    assert np.abs(got_logits - logits).max() < 1e-6
    loss, grads = ogpt.gpt_loss_and_grads(cfg, w, ids, targets, dtype=np.float64)
    assert abs(float(loss) - loss_t) < 1e-7
    assert len(grads) == len(grads_t) == 2 + 6 * cfg["n_layer"]
    for i, (g, gt) in enumerate(zip(grads, grads_t)):
        assert g.shape == gt.shape
        assert np.abs(g - gt).max() < 1e-7, i
    # the f32 evaluation, which the device is compared with, stays within 1e-5 of it
    loss32, grads32 = ogpt.gpt_loss_and_grads(cfg, [a.astype(np.float32) for a in w], ids, targets)
    assert abs(float(loss32) - loss_t) < 1e-5
    for g, gt in zip(grads32, grads_t):
        assert np.abs(g - gt).max() < 2e-5


def test_gpt_oracle_gradients_by_central_differences():
    cfg, ids, targets = REF_CFG, REF_IDS, REF_TARGETS
    w = make_weights(cfg, 7)
    _, grads = ogpt.gpt_loss_and_grads(cfg, w, ids, targets, dtype=np.float64)
    loss_of = lambda ws: float(oracle.cross_entropy_fwd(
        ogpt.gpt_forward(cfg, ws, ids, dtype=np.float64).reshape(ids.size, -1), targets, dtype=np.float64))
    h = 1e-6
    for wi, pos in [(0, (1, 2)), (0, (3, 0)), (1, (0, 1)), (2, (3, 3)), (3, (2, 0)), (4, (1, 1)),
                    (5, (0, 7)), (6, (5, 2)), (7, (3, 4))]:
        wp = [a.copy() for a in w]
        wm = [a.copy() for a in w]
        wp[wi][pos] += h
        wm[wi][pos] -= h
        fd = (loss_of(wp) - loss_of(wm)) / (2 * h)
        assert abs(fd - grads[wi][pos]) < 1e-7, (wi, pos)
    # an embedding row no token selects gets no gradient; row 3 is selected twice
    assert (grads[0][0] == 0).all() and (grads[0][5:] == 0).all() and np.abs(grads[0][3]).max() > 0


def test_gpt_oracle_train_step_moves_the_loss_down():
    cfg = CFG32
    rng = np.random.default_rng(9)
    ids = rng.integers(0, cfg["vocab_size"], (2, 9))
    targets = rng.integers(0, cfg["vocab_size"], ids.size)
    w = make_weights(cfg, 11, dtype=np.float32)
    mom = [(np.zeros_like(a), np.zeros_like(a)) for a in w]
    losses = []
    for t in range(1, 6):
        loss, norm, w, mom = ogpt.train_step(cfg, w, mom, t, ids, targets, 1e-2, weight_decay=0.01,
                                             max_norm=1.0)
        losses.append(float(loss))
        assert norm is not None and np.isfinite(norm)
    assert losses[-1] < losses[0]
    assert abs(losses[0] - math.log(cfg["vocab_size"])) < 1.5  # near-uniform predictions at init
