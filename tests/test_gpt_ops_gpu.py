"""Embedding lookup / scatter, RMSNorm, relu^2 and cross-entropy kernels against the numpy
restatements of src/storage/cpu.rs:555-660, src/nn.rs:244-251, src/models/gpt.rs:196-197
and src/loss.rs:11-24."""
import ctypes

import numpy as np
import pytest

import oracle
from deers_amd import rocm, synth

TOL = {np.dtype(np.float16): 5e-3, np.dtype(np.float32): 1e-4}


@pytest.fixture(scope="module", autouse=True)
def _init():
    if not rocm.available():
        pytest.skip("no gfx950 device")
    rocm.init(0)


def _dev(a):
    return rocm.DeviceBuffer.from_numpy(a)


def _tokens(n, vocab, seed, repeats=True):
    rng = np.random.default_rng(seed)
    t = rng.integers(0, vocab, n).astype(np.int64)
    if repeats and n > 8:  # text repeats tokens: make some ids very frequent
        t[rng.integers(0, n, n // 3)] = t[0]
        t[rng.integers(0, n, n // 5)] = (t[1] + 1) % vocab
    return t


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("vocab,width,n", [(4, 3, 3), (10, 4, 6), (101, 64, 70), (1000, 192, 1025),
                                           (50257, 768, 4096), (257, 130, 333)])
def test_index_select_and_index_add(dtype, vocab, width, n):
    table = synth.normal((vocab, width), synth.tensor_seed(71, "emb", "w"), 1.0).astype(dtype)
    idx = _tokens(n, vocab, 71)
    dt, di = _dev(table), _dev(idx)
    out = rocm.DeviceBuffer((n, width), dtype)
    rocm.index_select_raw(dtype, dt.ptr, di.ptr, out.ptr, vocab, n, width)
    assert np.array_equal(out.numpy(), oracle.index_select(table, idx))
    # backward: scatter-add of an upstream gradient, bit for bit in the reference's order
    g = synth.normal((n, width), synth.tensor_seed(71, "emb", "g"), 1.0).astype(dtype)
    dg = _dev(g)
    dst = rocm.DeviceBuffer((vocab, width), dtype, zeros=True)
    rocm.index_add_raw(dtype, dg.ptr, di.ptr, dst.ptr, vocab, n, width)
    want = oracle.index_add(vocab, g, idx)
    assert np.array_equal(dst.numpy(), want)
    again = rocm.DeviceBuffer((vocab, width), dtype, zeros=True)
    rocm.index_add_raw(dtype, dg.ptr, di.ptr, again.ptr, vocab, n, width)
    assert np.array_equal(again.numpy(), dst.numpy())


@pytest.mark.gpu
def test_index_literals_of_the_reference_and_out_of_range():
    # tests/tensor.rs:2290-2385
    data = np.float32([10, 11, 12, 20, 21, 22, 30, 31, 32, 40, 41, 42]).reshape(4, 3)
    dt = _dev(data)
    out = rocm.DeviceBuffer((3, 3), np.float32)
    i203, i202, ones = _dev(np.int64([2, 0, 3])), _dev(np.int64([2, 0, 2])), _dev(np.ones((3, 3), np.float32))
    rocm.index_select_raw(np.float32, dt.ptr, i203.ptr, out.ptr, 4, 3, 3)
    assert (out.numpy() == data[[2, 0, 3]]).all()
    grad = rocm.DeviceBuffer((4, 3), np.float32, zeros=True)
    rocm.index_add_raw(np.float32, ones.ptr, i202.ptr, grad.ptr, 4, 3, 3)
    assert (grad.numpy().ravel() == np.float32([1, 1, 1, 0, 0, 0, 2, 2, 2, 0, 0, 0])).all()
    # an index out of range is skipped by the kernel and reported by the next sync, once
    rocm.sync()
    bad = _dev(np.int64([1, 4, -1]))
    rocm.index_select_raw(np.float32, dt.ptr, bad.ptr, out.ptr, 4, 3, 3)
    with pytest.raises(rocm.RocmError, match="out of bounds"):
        rocm.sync()
    rocm.sync()  # the flag was cleared
    got = out.numpy()
    assert (got[0] == data[1]).all() and (got[1:] == 0).all()
    rocm.index_add_raw(np.float32, ones.ptr, bad.ptr, grad.ptr, 4, 3, 3)
    with pytest.raises(rocm.RocmError, match="out of bounds"):
        grad.numpy()
    assert (grad.numpy()[1] == 1).all()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("outer,inner", [(1, 3), (2, 4), (5, 48), (7, 191), (64, 192), (33, 768),
                                         (3, 4100), (8192, 768)])
def test_rms_norm_fwd_bwd(dtype, outer, inner):
    x = synth.normal((outer, inner), synth.tensor_seed(72, "rms", "x"), 2.0).astype(dtype)
    dy = synth.normal((outer, inner), synth.tensor_seed(72, "rms", "dy"), 1.0).astype(dtype)
    if (outer, inner) == (1, 3):
        x = np.array([[1.0, 2.0, 3.0]], dtype=dtype)  # tests/nn.rs:171-185
    dx_, dd = _dev(x), _dev(dy)
    y = rocm.DeviceBuffer((outer, inner), dtype)
    rocm.rms_norm_fwd_raw(dtype, dx_.ptr, y.ptr, outer, inner, 1e-5)
    want = oracle.rms_norm_fwd(x.astype(np.float32), 1e-5)
    assert np.abs(y.numpy().astype(np.float32) - want).max() <= TOL[np.dtype(dtype)]
    g = rocm.DeviceBuffer((outer, inner), dtype)
    rocm.rms_norm_bwd_raw(dtype, dx_.ptr, dd.ptr, g.ptr, outer, inner, 1e-5)
    want_g = oracle.rms_norm_bwd(x.astype(np.float32), dy.astype(np.float32), 1e-5)
    assert np.abs(g.numpy().astype(np.float32) - want_g).max() <= TOL[np.dtype(dtype)]
    if dtype == np.float32:
        assert np.abs((y.numpy().astype(np.float64) ** 2).mean(axis=1) - 1).max() < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("outer,inner", [(1, 3), (5, 48), (7, 191), (33, 768), (3, 4100), (8192, 768)])
def test_rms_norm_bwd_add_is_the_backward_followed_by_an_add(dtype, outer, inner):
    """deers_rocm_rms_norm_bwd_add: RMSNorm's backward and the accumulation onto the gradient its
    input already holds (src/backprop.rs:101-112) in one pass, bit for bit what
    deers_rocm_rms_norm_bwd followed by the oracle's add gives; the addend stays as it is unless
    it is the output."""
    x = synth.normal((outer, inner), synth.tensor_seed(73, "rms", "x"), 2.0).astype(dtype)
    dy = synth.normal((outer, inner), synth.tensor_seed(73, "rms", "dy"), 1.0).astype(dtype)
    acc = synth.normal((outer, inner), synth.tensor_seed(73, "rms", "acc"), 1.0).astype(dtype)
    dx_, dd, da = _dev(x), _dev(dy), _dev(acc)
    g = rocm.DeviceBuffer((outer, inner), dtype)
    rocm.rms_norm_bwd_raw(dtype, dx_.ptr, dd.ptr, g.ptr, outer, inner, 1e-5)
    want = (acc.astype(np.float32) + g.numpy().astype(np.float32)).astype(dtype)
    out = rocm.DeviceBuffer((outer, inner), dtype)
    rocm.rms_norm_bwd_add_raw(dtype, dx_.ptr, dd.ptr, da.ptr, out.ptr, outer, inner, 1e-5)
    assert np.array_equal(out.numpy(), want)
    assert np.array_equal(da.numpy(), acc)
    rocm.rms_norm_bwd_add_raw(dtype, dx_.ptr, dd.ptr, da.ptr, da.ptr, outer, inner, 1e-5)
    assert np.array_equal(da.numpy(), want)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n,skew", [(1, 0), (5, 0), (4099, 0), (1 << 20, 0), (1000, 1), (1000, 3)])
def test_relu_sq_is_bit_exact(dtype, n, skew):
    item = np.dtype(dtype).itemsize
    x = synth.normal((n + 8,), synth.tensor_seed(73, "relu", "x"), 2.0).astype(dtype)
    dy = synth.normal((n + 8,), synth.tensor_seed(73, "relu", "dy"), 1.0).astype(dtype)
    bx, bd = _dev(x), _dev(dy)
    out = _dev(np.full(n + 8, 7.0, dtype=dtype))
    at = lambda b: ctypes.c_void_p(b.ptr.value + skew * item)
    rocm.relu_sq_fwd_raw(dtype, at(bx), at(out), n)
    got = out.numpy()
    assert np.array_equal(got[skew:skew + n], oracle.relu_sq_fwd(x[skew:skew + n]))
    assert (got[:skew] == 7).all() and (got[skew + n:] == 7).all()
    rocm.relu_sq_bwd_raw(dtype, at(bx), at(bd), at(out), n)
    got = out.numpy()
    assert np.array_equal(got[skew:skew + n], oracle.relu_sq_bwd(x[skew:skew + n], dy[skew:skew + n]))
    assert (got[:skew] == 7).all() and (got[skew + n:] == 7).all()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n,v", [(2, 3), (6, 8), (7, 33), (5, 2049), (64, 256), (3, 8200), (16, 50257),
                                 (2, 70001)])  # the last one is longer than a workgroup's registers hold
def test_cross_entropy_fwd_bwd(dtype, n, v):
    x = synth.normal((n, v), synth.tensor_seed(74, "ce", "x"), 3.0).astype(dtype)
    t = _tokens(n, v, 74, repeats=False)
    if (n, v) == (2, 3):  # src/loss.rs:66-86
        x = np.array([[1, 2, 3], [1, -1, 0]], dtype=dtype)
        t = np.int64([2, 0])
    bx, bt = _dev(x), _dev(t)
    lse = rocm.DeviceBuffer((n,), np.float32)
    loss = rocm.DeviceBuffer((1,), np.float32)
    rocm.cross_entropy_fwd_raw(dtype, bx.ptr, bt.ptr, lse.ptr, loss.ptr, n, v)
    x32 = x.astype(np.float32)
    want = float(oracle.cross_entropy_fwd(x32, t))
    assert abs(float(loss.numpy()[0]) - want) <= 1e-5 * max(1.0, abs(want))
    want_lse = np.log(np.exp(x32.astype(np.float64)).sum(axis=1))
    assert np.abs(lse.numpy() - want_lse).max() <= 1e-5 * np.abs(want_lse).max()
    up = _dev(np.float32([0.7]))
    d = _dev(np.full((n, v), 9.0, dtype=dtype))
    rocm.cross_entropy_bwd_raw(dtype, bx.ptr, bt.ptr, lse.ptr, up.ptr, d.ptr, n, v)
    want_d = oracle.cross_entropy_bwd(x32, t, upstream=0.7)
    tol = 1e-6 if dtype == np.float32 else 5e-4
    assert np.abs(d.numpy().astype(np.float32) - want_d).max() <= tol
    # NULL upstream means 1
    rocm.cross_entropy_bwd_raw(dtype, bx.ptr, bt.ptr, lse.ptr, ctypes.c_void_p(), d.ptr, n, v)
    assert np.abs(d.numpy().astype(np.float32) - oracle.cross_entropy_bwd(x32, t)).max() <= tol
    if dtype == np.float32:
        assert np.abs(d.numpy().astype(np.float64).sum(axis=1)).max() < 1e-6
    # the forward that also writes the gradient for an upstream gradient of one: the forward's
    # loss and row statistics, the backward's bits
    lse2, loss2 = rocm.DeviceBuffer((n,), np.float32), rocm.DeviceBuffer((1,), np.float32)
    d2 = _dev(np.full((n, v), 9.0, dtype=dtype))
    rocm.cross_entropy_fwd_grad_raw(dtype, bx.ptr, bt.ptr, lse2.ptr, loss2.ptr, d2.ptr, n, v)
    assert np.array_equal(lse2.numpy(), lse.numpy()) and np.array_equal(loss2.numpy(), loss.numpy())
    assert np.array_equal(d2.numpy(), d.numpy())
    # the upstream factor afterwards: one leaves the bits, another multiplies and rounds once
    one, f07 = _dev(np.float32([1.0])), _dev(np.float32([0.7]))
    rocm.scale_by_scalar_raw(dtype, d2.ptr, n * v, one.ptr)
    assert np.array_equal(d2.numpy(), d.numpy())
    rocm.scale_by_scalar_raw(dtype, d2.ptr, n * v, f07.ptr)
    # (the f16 product may be rounded from the exact value or from its f32 rounding: the two differ
    # only on ties)
    got = d2.numpy()
    once = (d.numpy().astype(np.float64) * np.float64(np.float32(0.7))).astype(dtype)
    twice = (d.numpy().astype(np.float32) * np.float32(0.7)).astype(dtype)
    assert np.all((got == once) | (got == twice))


@pytest.mark.gpu
def test_cross_entropy_views_and_bad_target():
    # logits that start off a 16-byte boundary, gradient written at the same and at another phase
    n, v = 5, 1001
    x = synth.normal((n * v + 16,), synth.tensor_seed(75, "ce", "x"), 2.0).astype(np.float32)
    t = _tokens(n, v, 75, repeats=False)
    bx, bt = _dev(x), _dev(t)
    lse = rocm.DeviceBuffer((n,), np.float32)
    loss = rocm.DeviceBuffer((1,), np.float32)
    at = lambda b, k: ctypes.c_void_p(b.ptr.value + 4 * k)
    rocm.cross_entropy_fwd_raw(np.float32, at(bx, 3), bt.ptr, lse.ptr, loss.ptr, n, v)
    view = x[3:3 + n * v].reshape(n, v)
    assert abs(float(loss.numpy()[0]) - float(oracle.cross_entropy_fwd(view, t))) < 1e-5
    want = oracle.cross_entropy_bwd(view, t)
    for skew_out in (3, 2):
        d = _dev(np.full(n * v + 16, 9.0, dtype=np.float32))
        rocm.cross_entropy_bwd_raw(np.float32, at(bx, 3), bt.ptr, lse.ptr, ctypes.c_void_p(),
                                   at(d, skew_out), n, v)
        got = d.numpy()
        assert np.abs(got[skew_out:skew_out + n * v].reshape(n, v) - want).max() < 1e-6
        assert (got[:skew_out] == 9).all() and (got[skew_out + n * v:] == 9).all()
        # the gradient-writing forward on the same views: same bits, nothing outside them
        d2 = _dev(np.full(n * v + 16, 9.0, dtype=np.float32))
        lse2, loss2 = rocm.DeviceBuffer((n,), np.float32), rocm.DeviceBuffer((1,), np.float32)
        rocm.cross_entropy_fwd_grad_raw(np.float32, at(bx, 3), bt.ptr, lse2.ptr, loss2.ptr, at(d2, skew_out), n, v)
        assert np.array_equal(d2.numpy(), got) and np.array_equal(lse2.numpy(), lse.numpy())
    # a target out of range is reported at the next sync and contributes zero loss
    rocm.sync()
    t_bad = t.copy()
    t_bad[2] = v
    bt_bad = _dev(t_bad)
    rocm.cross_entropy_fwd_raw(np.float32, at(bx, 3), bt_bad.ptr, lse.ptr, loss.ptr, n, v)
    with pytest.raises(rocm.RocmError, match="out of bounds"):
        rocm.sync()


@pytest.mark.gpu
def test_gpt_ops_argument_errors():
    buf = rocm.DeviceBuffer((16,), np.float32, zeros=True)
    idx = _dev(np.int64([0]))
    null = ctypes.c_void_p()
    with pytest.raises(rocm.RocmError):
        rocm.index_select_raw(np.float32, null, idx.ptr, buf.ptr, 4, 1, 4)
    with pytest.raises(rocm.RocmError):
        rocm.rms_norm_fwd_raw(np.float32, buf.ptr, buf.ptr, 4, 0, 1e-5)
    with pytest.raises(rocm.RocmError):
        rocm.relu_sq_bwd_raw(np.float32, buf.ptr, null, buf.ptr, 16)
    with pytest.raises(rocm.RocmError):
        rocm.cross_entropy_fwd_raw(np.float32, buf.ptr, idx.ptr, buf.ptr, buf.ptr, 0, 4)
    rocm.index_select_raw(np.float32, null, null, null, 4, 0, 4)  # empty: no-op
    rocm.sync()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("outer,inner", [(1, 1), (3, 7), (32, 300), (5, 50257)])
def test_argmax_rows(dtype, outer, inner):
    x = synth.normal((outer, inner), synth.tensor_seed(76, "argmax", "x"), 2.0).astype(dtype)
    if inner > 4:
        x[0, 3] = x[0].max()          # a tie: the lowest index wins
        x[0, inner - 1] = x[0].max()
        x[outer - 1, :] = -np.inf      # nothing to pick: index 0
    bx = _dev(x)
    out = _dev(np.full(outer, -1, np.int64))
    rocm.argmax_rows_raw(dtype, bx.ptr, out.ptr, outer, inner)
    assert np.array_equal(out.numpy(), np.argmax(x, axis=1))


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1 << 14, (1 << 14) + 1, (1 << 18) + 37])
def test_index_add_over_several_index_slices(n):
    # a launch covers 2^14 positions; longer index vectors take one launch per slice, in
    # order, with the same sequence of additions (heavily repeated rows cross the seams)
    vocab, width = 997, 4
    idx = _tokens(n, vocab, 77, repeats=False)
    g = synth.normal((n, width), synth.tensor_seed(77, "emb", "g"), 1.0).astype(np.float32)
    dg, di = _dev(g), _dev(idx)
    dst = rocm.DeviceBuffer((vocab, width), np.float32, zeros=True)
    rocm.index_add_raw(np.float32, dg.ptr, di.ptr, dst.ptr, vocab, n, width)
    want = np.zeros((vocab, width), np.float32)
    np.add.at(want, idx, g)  # unbuffered, in position order: the same sequence of f32 additions
    assert np.array_equal(dst.numpy(), want)
