"""Pins the CPU oracle (oracle/attention_ref.cc) before anything trusts it.

Each check is chosen so a plausible slip (dropped term, wrong sign or index,
transposed operand, off-by-one in the mask) fails at least one of them:
literal vectors the reference's own tests hold, closed forms, brute force in
float64, finite differences, structural invariants, and a library routine.
"""
import glob
import math
import os

import numpy as np
import pytest

import oracle
from deers_amd import synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
NINF = -np.inf


# ---- literal vectors from the reference's tests ---------------------------------------------

def test_causal_mask_literal():
    # tests/nn.rs:193-219
    m = oracle.causal_mask(2, 3, 0)
    assert m.shape == (2, 1, 3, 3)
    row = [0, NINF, NINF, 0, 0, NINF, 0, 0, 0]
    assert m.ravel().tolist() == row + row


def test_causal_mask_with_offset_literal():
    # tests/nn.rs:221-232
    m = oracle.causal_mask(1, 2, 3)
    assert m.shape == (1, 1, 2, 5)
    assert m.ravel().tolist() == [0, 0, 0, 0, NINF, 0, 0, 0, 0, 0]


def test_decode_mask_row_is_all_zero():
    assert not np.isinf(oracle.causal_mask(2, 1, 40)).any()


def test_matmul_integer_products():
    # tests/tensor.rs:83-110 inputs; the product of small integers is exact in f32.
    a = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)
    b = np.array([[7, 8], [9, 10], [11, 12]], dtype=np.float32)
    assert oracle.matmul(a, b).tolist() == [[58, 64], [139, 154]]


def test_matmul_transposed_views_and_batches():
    rng = np.random.default_rng(0)
    a = rng.integers(-4, 5, size=(2, 3, 5, 7)).astype(np.float32)
    b = rng.integers(-4, 5, size=(2, 3, 6, 7)).astype(np.float32)
    got = oracle.matmul(a, b.transpose(0, 1, 3, 2), nthreads=3)      # rhs passed as a view
    assert np.array_equal(got, np.einsum("bhik,bhjk->bhij", a, b))
    got = oracle.matmul(a.transpose(0, 1, 3, 2), a)                   # lhs passed as a view
    assert np.array_equal(got, np.einsum("bhki,bhkj->bhij", a, a))


def test_scalar_mul_narrows_scalar_first():
    # `v * self.0 as f32` (src/storage.rs:105-123): the f64 scale is rounded to f32 first.
    x = np.array([3.0, -7.5, 1e-3], dtype=np.float32)
    s = 1.0 / math.sqrt(32.0)
    assert np.array_equal(oracle.scalar_mul(x, s), x * np.float32(s))


def test_log_sum_exp_closed_form():
    # input of tests/tensor.rs:1887
    x = np.array([[1.0, 2.0, 3.0], [1.5, 0.5, -1.0]], dtype=np.float32)
    want = [3 + math.log(1 + math.exp(-1) + math.exp(-2)),
            1.5 + math.log(1 + math.exp(-1) + math.exp(-2.5))]
    np.testing.assert_allclose(oracle.log_sum_exp(x), want, rtol=0, atol=2e-7)


def test_softmax_closed_form_and_masked_row():
    x = np.array([[1.0, 2.0, 3.0], [1.5, 0.5, -1.0], [0.25, NINF, NINF]], dtype=np.float32)
    e = np.exp(x.astype(np.float64) - x.astype(np.float64).max(1, keepdims=True))
    np.testing.assert_allclose(oracle.softmax(x), e / e.sum(1, keepdims=True), atol=1e-7)
    assert oracle.softmax(x)[2].tolist() == [1.0, 0.0, 0.0]


# ---- forward: brute force, invariants -----------------------------------------------------------

def brute_force_fwd(q, k, v, scale):
    """The definition, element by element in float64 (small shapes only)."""
    B, H, tq, D = q.shape
    tk = k.shape[2]
    off = tk - tq
    y = np.zeros((B, H, tq, D))
    for b in range(B):
        for h in range(H):
            for i in range(tq):
                w = [math.exp(scale * sum(float(q[b, h, i, d]) * float(k[b, h, j, d])
                                          for d in range(D)))
                     for j in range(i + off + 1)]
                z = sum(w)
                for d in range(D):
                    y[b, h, i, d] = sum(w[j] * float(v[b, h, j, d]) for j in range(len(w))) / z
    return y


def rand(shape, seed):
    return synth.normal(shape, seed)


@pytest.mark.parametrize("tq,tk", [(7, 7), (3, 9), (1, 6)])
def test_fwd_matches_brute_force(tq, tk):
    q, k, v = rand((2, 2, tq, 4), 1), rand((2, 2, tk, 4), 2), rand((2, 2, tk, 4), 3)
    want = brute_force_fwd(q, k, v, 0.5)
    np.testing.assert_allclose(oracle.attn_fwd(q, k, v, dtype=np.float64), want, atol=1e-12)
    np.testing.assert_allclose(oracle.attn_fwd(q, k, v), want, atol=2e-6)


def test_fwd_invariants():
    B, H, T, D = 2, 3, 19, 8
    q, k, v = rand((B, H, T, D), 4), rand((B, H, T, D), 5), rand((B, H, T, D), 6)
    y, lse, p = oracle.attn_fwd(q, k, v, return_lse=True, return_attn=True)
    np.testing.assert_allclose(p.sum(-1), 1.0, atol=1e-6)            # rows are distributions
    assert np.all(np.triu(p, 1) == 0)                                 # strictly-future weights are 0
    np.testing.assert_array_equal(y[:, :, 0], v[:, :, 0])             # first token sees only itself
    # causality: perturbing K/V after position t leaves y[..t] unchanged
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 10:] += 3.0
    v2[:, :, 10:] -= 2.0
    np.testing.assert_array_equal(oracle.attn_fwd(q, k2, v2)[:, :, :10], y[:, :, :10])
    # q = 0 -> uniform weights -> running mean of v
    ym = oracle.attn_fwd(np.zeros_like(q), k, v, dtype=np.float64)
    want = np.cumsum(v.astype(np.float64), 2) / np.arange(1, T + 1)[None, None, :, None]
    np.testing.assert_allclose(ym, want, atol=1e-12)
    # lse really is the log of the softmax denominator
    s = np.einsum("bhid,bhjd->bhij", q, k).astype(np.float64) / math.sqrt(D)
    s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    np.testing.assert_allclose(lse, np.log(np.exp(s).sum(-1)), atol=2e-6)


def test_default_scale_is_inverse_sqrt_d():
    q, k, v = rand((1, 1, 5, 16), 7), rand((1, 1, 5, 16), 8), rand((1, 1, 5, 16), 9)
    np.testing.assert_array_equal(oracle.attn_fwd(q, k, v), oracle.attn_fwd(q, k, v, scale=0.25))


# ---- backward: finite differences, invariants ----------------------------------------------------

@pytest.mark.parametrize("tq,tk", [(6, 6), (2, 5)])
def test_bwd_matches_central_differences(tq, tk):
    q, k, v = (rand((1, 2, t, 4), s).astype(np.float64) for t, s in ((tq, 11), (tk, 12), (tk, 13)))
    do = rand((1, 2, tq, 4), 14).astype(np.float64)
    dq, dk, dv = oracle.attn_bwd(q, k, v, do, dtype=np.float64)

    def loss(q_, k_, v_):
        return float((oracle.attn_fwd(q_, k_, v_, dtype=np.float64) * do).sum())

    eps = 1e-6
    for name, x, g in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        num = np.zeros_like(x)
        for idx in np.ndindex(*x.shape):
            xp, xm = x.copy(), x.copy()
            xp[idx] += eps
            xm[idx] -= eps
            args_p = {"q": q, "k": k, "v": v, name: xp}
            args_m = {"q": q, "k": k, "v": v, name: xm}
            num[idx] = (loss(args_p["q"], args_p["k"], args_p["v"])
                        - loss(args_m["q"], args_m["k"], args_m["v"])) / (2 * eps)
        np.testing.assert_allclose(g, num, atol=1e-8, err_msg=name)


def test_bwd_invariants():
    B, H, T, D = 1, 2, 17, 8
    q, k, v, do = (rand((B, H, T, D), s) for s in (21, 22, 23, 24))
    dq, dk, dv = oracle.attn_bwd(q, k, v, do)
    p = oracle.attn_fwd(q, k, v, return_attn=True)[1].astype(np.float64)
    np.testing.assert_allclose(dv, np.einsum("bhij,bhid->bhjd", p, do), atol=2e-6)   # dV = P^T dO
    # the last key/value is seen only by the last query
    do2 = do.copy()
    do2[:, :, :-1] = 0
    dq2, dk2, dv2 = oracle.attn_bwd(q, k, v, do2)
    np.testing.assert_allclose(dk2[:, :, -1], dk[:, :, -1], atol=1e-7)
    np.testing.assert_allclose(dv2[:, :, -1], dv[:, :, -1], atol=1e-7)
    assert np.all(dq2[:, :, :-1] == 0)
    # the backward map is linear in dO
    dq3, dk3, dv3 = oracle.attn_bwd(q, k, v, 2 * do)
    np.testing.assert_allclose(dq3, 2 * dq, atol=1e-6)
    np.testing.assert_allclose(dk3, 2 * dk, atol=1e-6)
    # first query attends only to key 0: its softmax is constant 1, so dq[0] = 0
    np.testing.assert_allclose(dq[:, :, 0], 0, atol=1e-7)
    assert np.isfinite(dq).all() and np.isfinite(dk).all() and np.isfinite(dv).all()


# ---- a library routine: torch SDPA + autograd, and the fixtures made from it -----------------

def test_against_torch_sdpa_live():
    torch = pytest.importorskip("torch")
    B, H, T, D = 2, 3, 40, 16
    q, k, v, do = (rand((B, H, T, D), s) for s in (31, 32, 33, 34))
    qt, kt, vt = (torch.tensor(a, requires_grad=True) for a in (q, k, v))
    y = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, is_causal=True)
    y.backward(torch.tensor(do))
    np.testing.assert_allclose(oracle.attn_fwd(q, k, v), y.detach().numpy(), atol=2e-6)
    for got, want in zip(oracle.attn_bwd(q, k, v, do), (qt.grad, kt.grad, vt.grad)):
        np.testing.assert_allclose(got, want.numpy(), atol=1e-5)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "*.npz"))),
                         ids=lambda p: os.path.basename(p)[:-4])
def test_against_golden_fixtures(path):
    f = np.load(path)
    q, k, v, do = f["q"], f["k"], f["v"], f["do"]
    y, lse = oracle.attn_fwd(q, k, v, return_lse=True)
    np.testing.assert_allclose(y, f["y"], atol=5e-6)
    np.testing.assert_allclose(lse, f["lse"], atol=5e-6)
    for got, name in zip(oracle.attn_bwd(q, k, v, do), ("dq", "dk", "dv")):
        np.testing.assert_allclose(got, f[name], atol=2e-5, err_msg=name)


def test_fixture_inputs_regenerate_from_seed():
    f = np.load(os.path.join(GOLDEN, "f16_b2h3t33d64.npz"))
    B, H, T, D, L, seed, ver = f["header"].tolist()
    assert ver == synth.GENERATOR_VERSION
    x = synth.attention_inputs("f16_b2h3t33d64", B, H, T, D, np.float16, base_seed=seed)
    for name in ("q", "k", "v", "do"):
        np.testing.assert_array_equal(x[name], f[name])


# ---- rotary embedding oracle: pinned by closed forms and invariants, not by retyping ----

def test_rope_tables_closed_forms():
    cos, sin = oracle.rope_tables(5, 8, base=10000.0)
    assert cos.shape == (5, 4) and sin.shape == (5, 4)
    # t = 0 is the identity rotation
    assert np.array_equal(cos[0], np.ones(4, np.float32)) and np.array_equal(sin[0], np.zeros(4, np.float32))
    # channel 0 has inv_freq 1: the angle is t itself
    assert np.allclose(cos[:, 0], np.cos(np.arange(5.0)), atol=1e-6)
    assert np.allclose(sin[:, 0], np.sin(np.arange(5.0)), atol=1e-6)
    # channel i has inv_freq base^(-2i/D): last channel of D=8 is 10000^(-6/8) = 10^-3
    assert np.allclose(sin[3, 3], np.sin(3.0 * 1e-3), atol=1e-7)
    # half tables in f16 are the rounded f32 ones
    ch, sh = oracle.rope_tables(5, 8, dtype=np.float16)
    assert np.array_equal(ch, cos.astype(np.float16)) and np.array_equal(sh, sin.astype(np.float16))


def test_rope_apply_known_rotation_and_sign():
    # D = 2, one channel, angle = t: a plain 2-D rotation by -t of (x1, x2)
    cos, sin = oracle.rope_tables(3, 2)
    x = np.zeros((1, 3, 1, 2), np.float32)
    x[0, :, 0] = [1.0, 0.0]
    y = oracle.rope_apply(x, cos, sin)
    # (1,0) -> (cos t, -sin t): a dropped sign or swapped halves fails here
    assert np.allclose(y[0, :, 0, 0], np.cos(np.arange(3.0)), atol=1e-6)
    assert np.allclose(y[0, :, 0, 1], -np.sin(np.arange(3.0)), atol=1e-6)
    x[0, :, 0] = [0.0, 1.0]
    y = oracle.rope_apply(x, cos, sin)
    assert np.allclose(y[0, :, 0, 0], np.sin(np.arange(3.0)), atol=1e-6)
    assert np.allclose(y[0, :, 0, 1], np.cos(np.arange(3.0)), atol=1e-6)


def test_rope_apply_invariants():
    rng = np.random.default_rng(11)
    B, T, H, D = 2, 7, 3, 8
    cos, sin = oracle.rope_tables(T, D)
    q = rng.standard_normal((B, T, H, D))
    k = rng.standard_normal((B, T, H, D))
    c64, s64 = cos.astype(np.float64), sin.astype(np.float64)
    yq = oracle.rope_apply(q, c64, s64, dtype=np.float64)
    yk = oracle.rope_apply(k, c64, s64, dtype=np.float64)
    half = D // 2
    # each (x1_i, x2_i) pair is rotated: its norm is preserved
    n_in = q[..., :half] ** 2 + q[..., half:] ** 2
    n_out = yq[..., :half] ** 2 + yq[..., half:] ** 2
    assert np.allclose(n_in, n_out, atol=1e-6)
    # relative-position property: <rope(q,t1), rope(k,t2)> depends on t1 - t2 only.
    # Use the same q, k vector at every position and compare (t1,t2) = (5,3) with (4,2), (2,0).
    qs = np.broadcast_to(q[:, :1], q.shape).copy()
    ks = np.broadcast_to(k[:, :1], k.shape).copy()
    yqs = oracle.rope_apply(qs, c64, s64, dtype=np.float64)
    yks = oracle.rope_apply(ks, c64, s64, dtype=np.float64)
    dot = lambda t1, t2: np.einsum("bhd,bhd->bh", yqs[:, t1], yks[:, t2])
    # the f32 tables make angles exact only to ~1e-7 relative
    assert np.allclose(dot(5, 3), dot(4, 2), atol=1e-5) and np.allclose(dot(5, 3), dot(2, 0), atol=1e-5)
    # position 0 is the identity
    assert np.array_equal(yq[:, 0], q[:, 0])


def test_rope_backward_is_the_transpose():
    rng = np.random.default_rng(12)
    B, T, H, D = 1, 5, 2, 8
    cos, sin = oracle.rope_tables(T, D)
    c64, s64 = cos.astype(np.float64), sin.astype(np.float64)
    x = rng.standard_normal((B, T, H, D))
    dy = rng.standard_normal((B, T, H, D))
    # the op is linear: <rope(x), dy> = <x, rope_bwd(dy)>, and central differences agree
    lhs = np.sum(oracle.rope_apply(x, c64, s64, dtype=np.float64) * dy)
    dx = oracle.rope_apply_bwd(dy, c64, s64, dtype=np.float64)
    assert np.isclose(lhs, np.sum(x * dx), rtol=1e-12)
    eps = 1e-6
    for idx in [(0, 1, 0, 2), (0, 4, 1, 6), (0, 3, 1, 0)]:
        xp, xm = x.copy(), x.copy()
        xp[idx] += eps
        xm[idx] -= eps
        fd = (np.sum(oracle.rope_apply(xp, c64, s64, dtype=np.float64) * dy)
              - np.sum(oracle.rope_apply(xm, c64, s64, dtype=np.float64) * dy)) / (2 * eps)
        assert np.isclose(fd, dx[idx], atol=1e-8)
    # a rotation's transpose is its inverse
    back = oracle.rope_apply_bwd(oracle.rope_apply(x, c64, s64, dtype=np.float64), c64, s64,
                                 dtype=np.float64)
    assert np.allclose(back, x, atol=1e-6)


# ---- row-wise log-softmax (src/storage/cpu.rs:793-888) ----

REF_LSM_INPUT = np.array([[1.0, 2.0, 3.0], [1.5, 0.5, -1.0]], dtype=np.float32)  # tests/tensor.rs:296


def test_log_softmax_reference_literal_against_library_and_definition():
    from scipy.special import log_softmax as scipy_lsm
    y = oracle.log_softmax_fwd(REF_LSM_INPUT)
    # the reference's own test compares with a library log-softmax on this input
    assert np.abs(y - scipy_lsm(REF_LSM_INPUT.astype(np.float64), axis=1)).max() < 1e-6
    # textbook definition, no max subtraction: x - ln(sum e^x)
    naive = [[v - math.log(sum(math.exp(u) for u in row)) for v in row] for row in REF_LSM_INPUT.tolist()]
    assert np.abs(y - np.array(naive)).max() < 1e-6
    # row [1,2,3]: last entry is -ln(1 + e^-1 + e^-2)
    assert abs(y[0, 2] + math.log(1 + math.exp(-1) + math.exp(-2))) < 1e-6


def test_log_softmax_invariants():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((7, 333)) * 4).astype(np.float32)
    y = oracle.log_softmax_fwd(x)
    assert np.abs(np.exp(y.astype(np.float64)).sum(axis=1) - 1).max() < 1e-5
    # shift invariance per row, and stability where the naive form overflows
    assert np.abs(oracle.log_softmax_fwd(x + np.float32(3.0)) - y).max() < 1e-5
    big = np.array([[1000.0, 1000.0, 999.0]], dtype=np.float32)
    yb = oracle.log_softmax_fwd(big)
    # lse = 1000.86 carries an f32 ulp of 6e-5
    assert np.isfinite(yb).all() and abs(yb[0, 0] + math.log(2 + math.exp(-1))) < 1e-4
    # a constant row is -ln(n); a single column is 0
    assert np.abs(oracle.log_softmax_fwd(np.full((2, 10), 3.5, np.float32)) + math.log(10)).max() < 1e-6
    assert (oracle.log_softmax_fwd(rng.standard_normal((4, 1)).astype(np.float32)) == 0).all()
    # f16 rows: computed in f32, rounded once
    xh = x.astype(np.float16)
    yh = oracle.log_softmax_fwd(xh, dtype=np.float16)
    assert yh.dtype == np.float16
    assert (yh == oracle.log_softmax_fwd(xh.astype(np.float32)).astype(np.float16)).all()


def test_log_softmax_backward_finite_differences_and_closed_form():
    from scipy.special import log_softmax as scipy_lsm
    rng = np.random.default_rng(6)
    x = rng.standard_normal((3, 9))
    g = rng.standard_normal((3, 9))
    y = oracle.log_softmax_fwd(x, dtype=np.float64)
    dx = oracle.log_softmax_bwd(g, y, dtype=np.float64)
    # central differences of the library routine, not of the oracle
    h = 1e-6
    for (i, j) in [(0, 0), (1, 4), (2, 8), (0, 5)]:
        xp, xm = x.copy(), x.copy()
        xp[i, j] += h
        xm[i, j] -= h
        fd = (np.sum(scipy_lsm(xp, axis=1) * g) - np.sum(scipy_lsm(xm, axis=1) * g)) / (2 * h)
        assert abs(fd - dx[i, j]) < 1e-6
    # rows of dx sum to zero (softmax sums to one)
    assert np.abs(dx.sum(axis=1)).max() < 1e-12
    # the reference's backward test: loss = sum(log_softmax(x)) so g = 1 and
    # dx = 1 - n * softmax(x)  (tests/tensor.rs:323-351)
    yr = oracle.log_softmax_fwd(REF_LSM_INPUT)
    dr = oracle.log_softmax_bwd(np.ones_like(yr), yr)
    e = np.exp(REF_LSM_INPUT.astype(np.float64))
    assert np.abs(dr - (1 - 3 * e / e.sum(axis=1, keepdims=True))).max() < 1e-6


# ---- AdamW step and clip_grad_norm (src/optim.rs:214-296) ----

def _adam_textbook(w, grads, lr, b1=0.9, b2=0.999, eps=1e-8, wd=0.0):
    """Loshchilov & Hutter's AdamW in float64, written from the paper's update rule
    (division by the bias corrections, decay folded into the update), not from the oracle."""
    w = np.asarray(w, dtype=np.float64).copy()
    m = np.zeros_like(w)
    v = np.zeros_like(w)
    for t, g in enumerate(grads, start=1):
        g = np.asarray(g, dtype=np.float64)
        m = b1 * m + (1 - b1) * g
        v = b2 * v + (1 - b2) * g * g
        w = w - lr * ((m / (1 - b1 ** t)) / (np.sqrt(v / (1 - b2 ** t)) + eps) + wd * w)
    return w


def test_adamw_reference_unit_tests():
    z = np.zeros(1, np.float32)
    # test_adamw_step (src/optim.rs:417-432): x = 0, loss (x-3)^2, lr 0.1 -> the first
    # Adam step moves by lr * sign(-g) = +0.1
    w, m, v = oracle.adamw_step(np.float32([0.0]), np.float32([-6.0]), z, z, 1, 0.1)
    assert abs(w[0] - 0.1) < 1e-6 and abs(m[0] + 0.6) < 1e-6 and abs(v[0] - 0.036) < 1e-6
    # test_adamw_weight_decay (459-471): zero gradient, only the decay acts: 5 * (1 - 0.1*0.1)
    w, m, v = oracle.adamw_step(np.float32([5.0]), z, z, z, 1, 0.1, weight_decay=0.1)
    assert abs(w[0] - 4.95) < 1e-6 and m[0] == 0 and v[0] == 0
    # test_adamw_loss_decreases (435-456): 20 steps on (x-3)^2
    x, m, v, losses = np.float32([0.0]), z, z, []
    for t in range(1, 21):
        losses.append(float((x[0] - 3) ** 2))
        x, m, v = oracle.adamw_step(x, 2 * (x - np.float32(3.0)), m, v, t, 0.1)
    assert losses[-1] < 0.2 * losses[0]
    # test_adamw_converges_quadratic (536-553): 100 steps on x^2 + y^2 from (5, -3)
    p, m, v = np.float32([5.0, -3.0]), np.zeros(2, np.float32), np.zeros(2, np.float32)
    for t in range(1, 101):
        p, m, v = oracle.adamw_step(p, 2 * p, m, v, t, 0.1)
    assert np.abs(p).max() < 0.1


def test_adamw_matches_textbook_rule_over_many_steps():
    rng = np.random.default_rng(11)
    w0 = rng.standard_normal(64).astype(np.float32)
    grads = [rng.standard_normal(64).astype(np.float32) * 0.3 for _ in range(25)]
    w, m, v = w0, np.zeros(64, np.float32), np.zeros(64, np.float32)
    for t, g in enumerate(grads, start=1):
        w, m, v = oracle.adamw_step(w, g, m, v, t, 3e-3, betas=(0.9, 0.95), weight_decay=0.1)
    want = _adam_textbook(w0, grads, 3e-3, 0.9, 0.95, 1e-8, 0.1)
    assert np.abs(w - want).max() < 2e-6
    # first step in closed form: w(1 - lr*wd) - lr * g / (|g| + eps)
    w1, _, _ = oracle.adamw_step(w0, grads[0], np.zeros(64, np.float32), np.zeros(64, np.float32), 1,
                                 0.01, weight_decay=0.5)
    g0 = grads[0].astype(np.float64)
    assert np.abs(w1 - (w0 * (1 - 0.005) - 0.01 * g0 / (np.abs(g0) + 1e-8))).max() < 1e-6


def test_adamw_f16_rounds_every_op_and_every_scalar():
    # f16 tensors: eps = 1e-8 is below half the smallest f16 subnormal and becomes 0, so a
    # zero gradient gives 0/0 = NaN in the reference's chain; a non-zero one is finite
    h = np.float16
    z = np.zeros(2, h)
    w, m, v = oracle.adamw_step(h([1.0, 1.0]), h([0.0, 0.5]), z, z, 1, 0.1, dtype=h)
    assert w.dtype == h and np.isnan(w[0]) and abs(float(w[1]) - 0.9) < 1e-3
    assert oracle._scalar(1e-8, h) == 0 and oracle._scalar(0.999, h) == h(0.999)
    assert abs(oracle._powi(0.999, 1000) - 0.999 ** 1000) < 1e-14
    assert oracle._powi(2.0, 10) == 1024.0 and oracle._powi(2.0, -2) == 0.25 and oracle._powi(3.0, 0) == 1.0


def test_clip_grad_norm_reference_cases():
    # test_clip_grad_norm_scales_large_gradients (src/optim.rs:556-570)
    norm, (g,) = oracle.clip_grad_norm([np.float32([3.0, 4.0])], 1.0)
    assert abs(norm - 5.0) < 1e-5 and abs(g[0] - 0.6) < 1e-4 and abs(g[1] - 0.8) < 1e-4
    # below the threshold nothing changes; several tensors share one norm
    a, b = np.float32([1.0, 2.0]), np.float32([2.0])
    norm, (ga, gb) = oracle.clip_grad_norm([a, b], 10.0)
    assert abs(norm - 3.0) < 1e-6 and (ga == a).all() and (gb == b).all()
    norm, (ga, gb) = oracle.clip_grad_norm([a, b], 1.5)
    assert abs(np.sqrt((ga ** 2).sum() + (gb ** 2).sum()) - 1.5) < 1e-5
    # a non-finite norm is returned and nothing is rescaled
    norm, (gi,) = oracle.clip_grad_norm([np.float32([np.inf, 1.0])], 1.0)
    assert np.isinf(norm) and gi[1] == 1.0
    assert oracle.clip_grad_norm([], 1.0)[0] == 0.0


# ---- embedding, RMSNorm, relu^2, cross-entropy (src/nn.rs, src/models/gpt.rs, src/loss.rs) ----

def test_index_select_and_add_reference_literals():
    # tests/tensor.rs:2290-2320 and 2359-2385
    data = np.float32([10, 11, 12, 20, 21, 22, 30, 31, 32, 40, 41, 42]).reshape(4, 3)
    assert (oracle.index_select(data, [2, 0, 3]) == data[[2, 0, 3]]).all()
    assert (oracle.index_select(data, [2, 0, 3])[0] == [30, 31, 32]).all()
    grad = oracle.index_add(4, np.ones((3, 3), np.float32), [2, 0, 2])
    assert (grad.ravel() == np.float32([1, 1, 1, 0, 0, 0, 2, 2, 2, 0, 0, 0])).all()
    with pytest.raises(IndexError):
        oracle.index_select(data, [4])
    with pytest.raises(IndexError):
        oracle.index_add(4, np.ones((1, 3), np.float32), [-1])
    # accumulation order is ascending position: visible in f16, where addition is not associative
    src = np.float16([[2048.0], [1.0], [1.0]])
    assert oracle.index_add(1, src, [0, 0, 0])[0, 0] == np.float16(2048.0)      # (2048+1)+1 = 2048
    assert oracle.index_add(1, src[::-1].copy(), [0, 0, 0])[0, 0] == np.float16(2050.0)  # (1+1)+2048


def test_rms_norm_reference_case_library_and_differences():
    import torch
    # tests/nn.rs:171-185: [1,2,3] / sqrt(14/3)
    y = oracle.rms_norm_fwd(np.float32([[1, 2, 3]]), 1e-5)
    assert np.abs(y - np.float32([1, 2, 3]) / np.sqrt(14.0 / 3.0)).max() < 1e-4
    rng = np.random.default_rng(21)
    x = rng.standard_normal((5, 48)).astype(np.float32)
    dy = rng.standard_normal((5, 48)).astype(np.float32)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ty = torch.nn.functional.rms_norm(tx, (48,), eps=1e-5)
    ty.backward(torch.tensor(dy, dtype=torch.float64))
    assert np.abs(oracle.rms_norm_fwd(x, 1e-5) - ty.detach().numpy()).max() < 1e-6
    assert np.abs(oracle.rms_norm_bwd(x, dy, 1e-5) - tx.grad.numpy()).max() < 1e-5
    # every output row has mean square 1 (up to eps); the gradient is orthogonal to x
    assert np.abs((oracle.rms_norm_fwd(x, 0.0).astype(np.float64) ** 2).mean(axis=1) - 1).max() < 1e-6
    d64 = oracle.rms_norm_bwd(x.astype(np.float64), dy.astype(np.float64), 0.0, dtype=np.float64)
    assert np.abs((d64 * x).sum(axis=1)).max() < 1e-12
    # central differences of the forward
    x64, h = x.astype(np.float64), 1e-6
    d = oracle.rms_norm_bwd(x64, dy.astype(np.float64), 1e-5, dtype=np.float64)
    for (i, j) in [(0, 0), (3, 17), (4, 47)]:
        xp, xm = x64.copy(), x64.copy()
        xp[i, j] += h
        xm[i, j] -= h
        fd = ((oracle.rms_norm_fwd(xp, 1e-5, dtype=np.float64) - oracle.rms_norm_fwd(xm, 1e-5, dtype=np.float64)) * dy).sum() / (2 * h)
        assert abs(fd - d[i, j]) < 1e-6


def test_relu_sq_closed_forms():
    x = np.float32([-2.0, -0.0, 0.0, 0.5, 3.0])
    dy = np.float32([1.0, 1.0, 1.0, 2.0, -1.0])
    assert (oracle.relu_sq_fwd(x) == np.float32([0, 0, 0, 0.25, 9.0])).all()
    assert (oracle.relu_sq_bwd(x, dy) == np.float32([0, 0, 0, 2.0, -6.0])).all()
    xh = np.float16([0.1, 1.7, -3.0])
    assert oracle.relu_sq_fwd(xh).dtype == np.float16
    assert (oracle.relu_sq_fwd(xh) == (np.maximum(xh, 0) * np.maximum(xh, 0))).all()


def test_cross_entropy_reference_cases_and_library():
    import torch
    # log_softmax([1,2,3]) = [-2.4076, -1.4076, -0.4076] (the literals of src/loss.rs:34-36):
    # targets 2 and 0 on two such rows give (0.4076 + 2.4076) / 2
    row = np.float32([[1, 2, 3], [1, 2, 3]])
    assert abs(float(oracle.cross_entropy_fwd(row, [2, 0])) - 1.4076) < 1e-4
    assert abs(float(oracle.cross_entropy_fwd(np.zeros((3, 10), np.float32), [1, 5, 9])) - math.log(10)) < 1e-6
    # src/loss.rs:66-86: gradient rows sum to zero
    logits = np.float32([[1, 2, 3], [1, -1, 0]])
    g = oracle.cross_entropy_bwd(logits, [2, 0])
    assert np.abs(g.sum(axis=1)).max() < 1e-6
    # library: torch's cross_entropy and autograd in f64
    rng = np.random.default_rng(22)
    x = (rng.standard_normal((7, 33)) * 3).astype(np.float32)
    t = rng.integers(0, 33, 7)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    tl = torch.nn.functional.cross_entropy(tx, torch.tensor(t))
    (tl * 0.7).backward()
    assert abs(float(oracle.cross_entropy_fwd(x, t)) - float(tl)) < 1e-6
    assert np.abs(oracle.cross_entropy_bwd(x, t, upstream=0.7) - tx.grad.numpy()).max() < 1e-7
    # closed form: (softmax - onehot) / N
    p = np.exp(x.astype(np.float64))
    p /= p.sum(axis=1, keepdims=True)
    p[np.arange(7), t] -= 1
    assert np.abs(oracle.cross_entropy_bwd(x, t) - p / 7).max() < 1e-7


def test_synthetic_rotary_tables_equal_the_oracle_tables():
    """deers_amd.synth.rotary_tables feeds the benchmark; it must be the table the oracle
    (src/models/gpt.rs:12-47) pins, bit for bit, in both storage types."""
    from deers_amd import synth
    for T, D in ((1, 2), (7, 32), (1024, 64), (300, 128)):
        for dt in (np.float32, np.float16):
            c, s = synth.rotary_tables(T, D, dtype=dt)
            oc, os_ = oracle.rope_tables(T, D, dtype=dt)
            assert c.dtype == dt and np.array_equal(c, oc) and np.array_equal(s, os_)
