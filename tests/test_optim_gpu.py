"""Fused AdamW step, sum of squares and scaling (deers_rocm_adamw_step / _sum_squares /
_scale) against the numpy restatement of src/optim.rs:214-296.  The step keeps the
reference's op order and per-op rounding, so it is compared bit for bit."""
import ctypes

import numpy as np
import pytest

import oracle
from deers_amd import rocm, synth


@pytest.fixture(scope="module", autouse=True)
def _init():
    if not rocm.available():
        pytest.skip("no gfx950 device")
    rocm.init(0)


def _state(n, dtype, seed):
    w = synth.normal((n,), synth.tensor_seed(seed, "opt", "w"), 1.0).astype(dtype)
    g = synth.normal((n,), synth.tensor_seed(seed, "opt", "g"), 0.5).astype(dtype)
    m = (synth.normal((n,), synth.tensor_seed(seed, "opt", "m"), 0.1)).astype(dtype)
    v = np.abs(synth.normal((n,), synth.tensor_seed(seed, "opt", "v"), 0.05)).astype(dtype)
    return w, g, m, v


def _same_bits(a, b):
    return np.array_equal(a.view(np.uint16 if a.dtype == np.float16 else np.uint32),
                          b.view(np.uint16 if b.dtype == np.float16 else np.uint32)) or \
        np.array_equal(a, b, equal_nan=True)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("n", [1, 3, 4, 7, 8, 255, 1024, 1027, 65536 + 5, 3 * 1000 * 1000 + 1])
@pytest.mark.parametrize("wd,step", [(0.0, 1), (0.1, 7)])
def test_adamw_step_is_bit_exact(dtype, n, wd, step):
    w, g, m, v = _state(n, dtype, 51)
    if step == 1:
        m[:] = 0
        v[:] = 0
    eps = 1e-8 if dtype == np.float32 else 1e-3  # f16: an eps that survives the cast
    bw, bg, bm, bv = (rocm.DeviceBuffer.from_numpy(a) for a in (w, g, m, v))
    rocm.adamw_step_raw(dtype, bw.ptr, bg.ptr, bm.ptr, bv.ptr, n, 3e-3, 0.9, 0.95, eps, wd, step)
    ww, wm, wv = oracle.adamw_step(w, g, m, v, step, 3e-3, (0.9, 0.95), eps, wd, dtype=dtype)
    assert _same_bits(bm.numpy(), wm)
    assert _same_bits(bv.numpy(), wv)
    assert _same_bits(bw.numpy(), ww)
    assert np.array_equal(bg.numpy(), g)  # the gradient is only read


@pytest.mark.gpu
def test_adamw_reference_unit_tests_on_device():
    # src/optim.rs:417-471 and 536-553 through the kernel
    def run(w, g, steps, lr, wd=0.0, grad_fn=None):
        n = len(w)
        bw = rocm.DeviceBuffer.from_numpy(np.float32(w))
        bm = rocm.DeviceBuffer((n,), np.float32, zeros=True)
        bv = rocm.DeviceBuffer((n,), np.float32, zeros=True)
        for t in range(1, steps + 1):
            cur = bw.numpy()
            bg = rocm.DeviceBuffer.from_numpy(np.float32(grad_fn(cur) if grad_fn else g))
            rocm.adamw_step_raw(np.float32, bw.ptr, bg.ptr, bm.ptr, bv.ptr, n, lr, 0.9, 0.999, 1e-8,
                                wd, t)
        return bw.numpy()
    assert abs(run([0.0], [-6.0], 1, 0.1)[0] - 0.1) < 1e-6
    assert abs(run([5.0], [0.0], 1, 0.1, wd=0.1)[0] - 4.95) < 1e-6
    assert np.abs(run([5.0, -3.0], None, 100, 0.1, grad_fn=lambda p: 2 * p)).max() < 0.1


@pytest.mark.gpu
def test_adamw_many_steps_track_the_oracle_bit_for_bit():
    n = 4099
    w, _, _, _ = _state(n, np.float32, 52)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    bw, bm, bv = (rocm.DeviceBuffer.from_numpy(a) for a in (w, m, v))
    for t in range(1, 13):
        g = synth.normal((n,), synth.tensor_seed(52, "opt", f"g{t}"), 0.3).astype(np.float32)
        bg = rocm.DeviceBuffer.from_numpy(g)
        rocm.adamw_step_raw(np.float32, bw.ptr, bg.ptr, bm.ptr, bv.ptr, n, 1e-2, 0.9, 0.999, 1e-8, 0.01, t)
        w, m, v = oracle.adamw_step(w, g, m, v, t, 1e-2, (0.9, 0.999), 1e-8, 0.01)
    assert _same_bits(bw.numpy(), w) and _same_bits(bm.numpy(), m) and _same_bits(bv.numpy(), v)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_adamw_f16_quirks_and_unaligned_views(dtype):
    n, item = 1000, np.dtype(dtype).itemsize
    w, g, m, v = _state(n + 8, dtype, 53)
    g[5] = 0
    m[5] = 0
    v[5] = 0  # with the default eps an f16 tensor divides 0 by 0 here, an f32 one does not
    bufs = [rocm.DeviceBuffer.from_numpy(a) for a in (w, g, m, v)]
    skew = 3  # elements: the views start off any 16-byte boundary
    ptrs = [ctypes.c_void_p(b.ptr.value + skew * item) for b in bufs]
    rocm.adamw_step_raw(dtype, *ptrs, n, 1e-2, 0.9, 0.999, 1e-8, 0.0, 3)
    ww, wm, wv = oracle.adamw_step(w[skew:skew + n], g[skew:skew + n], m[skew:skew + n],
                                   v[skew:skew + n], 3, 1e-2, dtype=dtype)
    got_w = bufs[0].numpy()
    assert _same_bits(got_w[skew:skew + n], ww)
    assert np.isnan(ww[5 - skew]) == (dtype == np.float16)
    # neighbours of the view are untouched
    assert np.array_equal(got_w[:skew], w[:skew]) and np.array_equal(got_w[skew + n:], w[skew + n:])
    assert _same_bits(bufs[2].numpy()[skew:skew + n], wm) and _same_bits(bufs[3].numpy()[skew:skew + n], wv)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_clip_grad_norm_pieces(dtype):
    sizes = [1, 5, 1000, 256 * 1024 + 3, 2 * 1000 * 1000]
    grads = [synth.normal((n,), synth.tensor_seed(54, "opt", f"g{i}"), 0.7).astype(dtype)
             for i, n in enumerate(sizes)]
    bufs = [rocm.DeviceBuffer.from_numpy(g) for g in grads]
    total = rocm.DeviceBuffer((1,), np.float32)
    for i, (b, g) in enumerate(zip(bufs, grads)):
        rocm.sum_squares_raw(dtype, b.ptr, g.size, total.ptr, accumulate=i > 0)
    want = sum(float((g.astype(np.float64) ** 2).sum()) for g in grads)
    got = float(total.numpy()[0])
    assert abs(got - want) <= 1e-6 * want
    # same inputs, same bits
    again = rocm.DeviceBuffer((1,), np.float32)
    for i, (b, g) in enumerate(zip(bufs, grads)):
        rocm.sum_squares_raw(dtype, b.ptr, g.size, again.ptr, accumulate=i > 0)
    assert again.numpy()[0] == total.numpy()[0]
    # the reference's own case: [3, 4] clipped to norm 1 (src/optim.rs:556-570)
    b = rocm.DeviceBuffer.from_numpy(np.array([3.0, 4.0], dtype=dtype))
    rocm.sum_squares_raw(dtype, b.ptr, 2, total.ptr)
    norm = np.float32(np.sqrt(total.numpy()[0]))
    assert abs(norm - 5.0) < 1e-5
    scale = 1.0 / (float(norm) + 1e-6)
    rocm.scale_raw(dtype, b.ptr, 2, scale)
    _, (want_g,) = oracle.clip_grad_norm([np.array([3.0, 4.0], dtype=dtype)], 1.0, dtype=dtype)
    assert _same_bits(b.numpy(), want_g)
    # scaling a big gradient in place matches the oracle's rounding, bit for bit
    rocm.scale_raw(dtype, bufs[3].ptr, sizes[3], 0.37)
    assert _same_bits(bufs[3].numpy(), (grads[3] * oracle._scalar(0.37, dtype)).astype(dtype))
    # an empty tensor contributes nothing
    rocm.sum_squares_raw(dtype, ctypes.c_void_p(), 0, total.ptr)
    assert total.numpy()[0] == 0.0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_folded_grad_scale_equals_scale_then_step(dtype):
    n = 5003
    w, g, m, v = _state(n, dtype, 55)
    eps = 1e-8 if dtype == np.float32 else 1e-3
    a = [rocm.DeviceBuffer.from_numpy(x) for x in (w, g, m, v)]
    b = [rocm.DeviceBuffer.from_numpy(x) for x in (w, g, m, v)]
    rocm.adamw_step_raw(dtype, *(x.ptr for x in a), n, 1e-2, 0.9, 0.999, eps, 0.1, 4, grad_scale=0.25)
    rocm.scale_raw(dtype, b[1].ptr, n, 0.25)
    rocm.adamw_step_raw(dtype, *(x.ptr for x in b), n, 1e-2, 0.9, 0.999, eps, 0.1, 4)
    for i in (0, 2, 3):
        assert _same_bits(a[i].numpy(), b[i].numpy())
    assert np.array_equal(a[1].numpy(), g)  # folded: the gradient itself is not rewritten
    gs = (g * oracle._scalar(0.25, dtype)).astype(dtype)
    ww, _, _ = oracle.adamw_step(w, gs, m, v, 4, 1e-2, (0.9, 0.999), eps, 0.1, dtype=dtype)
    assert _same_bits(a[0].numpy(), ww)


@pytest.mark.gpu
def test_optimizer_argument_errors():
    buf = rocm.DeviceBuffer((16,), np.float32, zeros=True)
    with pytest.raises(rocm.RocmError):
        rocm.adamw_step_raw(np.float32, buf.ptr, buf.ptr, buf.ptr, buf.ptr, 16, 1e-3, 0.9, 0.999, 1e-8, 0.0, 0)
    with pytest.raises(rocm.RocmError):
        rocm.adamw_step_raw(np.float32, buf.ptr, ctypes.c_void_p(), buf.ptr, buf.ptr, 16, 1e-3, 0.9, 0.999,
                            1e-8, 0.0, 1)
    with pytest.raises(rocm.RocmError):
        rocm.sum_squares_raw(np.float32, buf.ptr, 16, ctypes.c_void_p())
    with pytest.raises(rocm.RocmError):
        rocm.scale_raw(np.float32, buf.ptr, -1, 2.0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_multi_tensor_step_and_norm_equal_the_single_tensor_calls(dtype):
    # 110 tensors (more than one launch's worth) of ragged sizes, one of them a view that is
    # not 16-byte aligned: every tensor gets exactly the bits of its own single-tensor call
    rng = np.random.default_rng(57)
    sizes = [1, 3, 4, 5, 768, 4096 + 1, 3 * 4096, 100_000] + [int(s) for s in rng.integers(1, 30_000, 102)]
    eps = 1e-8 if dtype == np.float32 else 1e-3
    item = np.dtype(dtype).itemsize
    states = [_state(n + 8, dtype, 100 + i) for i, n in enumerate(sizes)]
    skew = [0] * len(sizes)
    skew[6] = 1  # an unaligned view
    a = [[rocm.DeviceBuffer.from_numpy(x) for x in st] for st in states]
    b = [[rocm.DeviceBuffer.from_numpy(x) for x in st] for st in states]
    at = lambda buf, k: ctypes.c_void_p(buf.ptr.value + k * item)
    rocm.adamw_step_multi_raw(dtype, *[[at(t[j], skew[i]) for i, t in enumerate(a)] for j in range(4)], sizes,
                              1e-2, 0.9, 0.95, eps, 0.1, 5, grad_scale=0.5)
    for i, (t, n) in enumerate(zip(b, sizes)):
        rocm.adamw_step_raw(dtype, *(at(x, skew[i]) for x in t), n, 1e-2, 0.9, 0.95, eps, 0.1, 5, grad_scale=0.5)
    for i, (ta, tb) in enumerate(zip(a, b)):
        for j in range(4):
            assert _same_bits(ta[j].numpy(), tb[j].numpy()), (i, j)
    # and against the oracle for a few of them
    for i in (0, 4, 6, 7, 50):
        w, g, m, v = (x[skew[i]:skew[i] + sizes[i]] for x in states[i])
        gs = (g * oracle._scalar(0.5, dtype)).astype(dtype)
        ww, wm, wv = oracle.adamw_step(w, gs, m, v, 5, 1e-2, (0.9, 0.95), eps, 0.1, dtype=dtype)
        assert _same_bits(a[i][0].numpy()[skew[i]:skew[i] + sizes[i]], ww)
        assert _same_bits(a[i][2].numpy()[skew[i]:skew[i] + sizes[i]], wm)
    # the norm: all aligned gradients in one reduction
    ptrs = [t[1].ptr for i, t in enumerate(a) if skew[i] == 0]
    ns = [n + 8 for i, n in enumerate(sizes) if skew[i] == 0]
    total = rocm.DeviceBuffer((1,), np.float32)
    rocm.sum_squares_multi_raw(dtype, ptrs, ns, total.ptr)
    want = sum(float((st[1].astype(np.float64) ** 2).sum()) for i, st in enumerate(states) if skew[i] == 0)
    got = float(total.numpy()[0])
    assert abs(got - want) <= 1e-6 * want
    again = rocm.DeviceBuffer((1,), np.float32)
    rocm.sum_squares_multi_raw(dtype, ptrs, ns, again.ptr)
    assert again.numpy()[0] == total.numpy()[0]
    rocm.sum_squares_multi_raw(dtype, ptrs, ns, again.ptr, accumulate=True)
    assert abs(float(again.numpy()[0]) - 2 * got) <= 1e-6 * got
    with pytest.raises(rocm.RocmError):
        rocm.sum_squares_multi_raw(dtype, [at(a[0][1], 1)], [4], total.ptr)
    rocm.sum_squares_multi_raw(dtype, [], [], total.ptr)
    assert total.numpy()[0] == 0.0
