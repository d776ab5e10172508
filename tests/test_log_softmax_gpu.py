"""Row-wise log-softmax (deers_rocm_log_softmax_fwd / _bwd) against the numpy restatement
of src/storage/cpu.rs:793-888, on the shapes of the reference's tests and of the GPT loss."""
import ctypes

import numpy as np
import pytest

import oracle
from deers_amd import rocm, synth

TOL = {np.dtype(np.float16): 5e-3, np.dtype(np.float32): 1e-4}

# (outer, inner): the reference's 2x3 literal, a single column, the tiny-GPT vocabulary
# and the GPT-2 one (odd width), row counts that leave a workgroup of four wavefront-rows
# partly empty, and widths on both sides of every boundary between the kernels' tiers
# (a row is cut into 16-byte chunks; a tier holds 64, 256, 1024, 4096, 8192, 13312 or
# 16384 chunks; wider rows take the two-sweep kernel), for 4 and for 8 elements per chunk.
_EDGES_F32 = [250, 251, 1018, 1019, 4090, 4091, 16378, 16379, 32762, 32763, 53242, 53243, 65530,
              65531]
_EDGES_F16 = [498, 499, 2034, 2035, 8178, 8179, 32754, 32755, 65522, 65523]
SHAPES = ([(2, 3), (5, 1), (64, 256), (9, 257), (3, 511), (6, 1024), (2, 1025), (4, 4096),
           (3, 4097), (7, 12289), (3, 20000), (16, 50257), (2, 65537), (3, 70001), (2, 131100)]
          + [(3, w) for w in _EDGES_F32 + _EDGES_F16])


@pytest.fixture(scope="module", autouse=True)
def _init():
    if not rocm.available():
        pytest.skip("no gfx950 device")
    rocm.init(0)


def _run_fwd(x):
    dx = rocm.DeviceBuffer.from_numpy(x)
    y = rocm.DeviceBuffer(x.shape, x.dtype)
    rocm.log_softmax_fwd_raw(x.dtype, dx.ptr, y.ptr, x.shape[0], x.shape[1])
    return y.numpy()


def _run_bwd(g, lsm):
    dg, dl = rocm.DeviceBuffer.from_numpy(g), rocm.DeviceBuffer.from_numpy(lsm)
    out = rocm.DeviceBuffer(g.shape, g.dtype)
    rocm.log_softmax_bwd_raw(g.dtype, dg.ptr, dl.ptr, out.ptr, g.shape[0], g.shape[1])
    return out.numpy()


@pytest.mark.gpu
def test_reference_literal():
    # tests/tensor.rs:294-351: input [[1,2,3],[1.5,0.5,-1]], loss = sum(log_softmax)
    x = np.array([[1.0, 2.0, 3.0], [1.5, 0.5, -1.0]], dtype=np.float32)
    y = _run_fwd(x)
    e = np.exp(x.astype(np.float64))
    assert np.abs(y - np.log(e / e.sum(axis=1, keepdims=True))).max() < 1e-6
    dx = _run_bwd(np.ones_like(x), y)
    assert np.abs(dx - (1 - 3 * e / e.sum(axis=1, keepdims=True))).max() < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("outer,inner", SHAPES)
def test_fwd_bwd_match_oracle(dtype, outer, inner):
    x = synth.normal((outer, inner), synth.tensor_seed(31, "lsm", "x"), 3.0).astype(dtype)
    g = synth.normal((outer, inner), synth.tensor_seed(31, "lsm", "g"), 1.0).astype(dtype)
    y = _run_fwd(x)
    want = oracle.log_softmax_fwd(x.astype(np.float32))
    # f16 outputs of magnitude up to ~20 carry an ulp of 1.6e-2: compare in ulps of the
    # rounded result there, in absolute terms for f32
    if dtype == np.float16:
        assert np.abs(y.astype(np.float32) - want).max() <= 5e-3 + np.abs(want).max() * 2 ** -11
    else:
        assert np.abs(y - want).max() <= TOL[np.dtype(dtype)]
    dx = _run_bwd(g, y)
    want_dx = oracle.log_softmax_bwd(g.astype(np.float32), y.astype(np.float32))
    if dtype == np.float16:
        # the row sum of g (up to ~sqrt(inner)) multiplies probabilities <= 1
        bound = 5e-3 + np.abs(want_dx).max() * 2 ** -11
    else:
        bound = TOL[np.dtype(dtype)]
    assert np.abs(dx.astype(np.float32) - want_dx).max() <= bound


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("skew_in,skew_out", [(1, 1), (3, 3), (0, 1), (2, 5)])
def test_views_at_any_element_offset(dtype, skew_in, skew_out):
    # operands that start `skew` elements into an allocation: equal offsets within 16
    # bytes take the chunked kernels with a partial first chunk in row 0, unequal ones
    # the two-sweep kernel; neighbours of the view must stay untouched
    outer, inner = 5, 1000
    item = np.dtype(dtype).itemsize
    x = synth.normal((outer, inner), synth.tensor_seed(34, "lsm", "x"), 3.0).astype(dtype)
    g = synth.normal((outer, inner), synth.tensor_seed(34, "lsm", "g"), 1.0).astype(dtype)
    pad = 16
    def padded(a, skew):
        flat = np.full(a.size + 2 * pad, 7.0, dtype=dtype)
        flat[skew:skew + a.size] = a.ravel()
        return flat
    def at(buf, skew):
        return ctypes.c_void_p(buf.ptr.value + skew * item)
    dx = rocm.DeviceBuffer.from_numpy(padded(x, skew_in))
    dy = rocm.DeviceBuffer.from_numpy(np.full(x.size + 2 * pad, 7.0, dtype=dtype))
    rocm.log_softmax_fwd_raw(dtype, at(dx, skew_in), at(dy, skew_out), outer, inner)
    got = dy.numpy()
    y = got[skew_out:skew_out + x.size].reshape(outer, inner)
    assert (got[:skew_out] == 7.0).all() and (got[skew_out + x.size:] == 7.0).all()
    want = oracle.log_softmax_fwd(x.astype(np.float32))
    tol = 5e-3 + np.abs(want).max() * 2 ** -11 if dtype == np.float16 else 1e-4
    assert np.abs(y.astype(np.float32) - want).max() <= tol
    dg = rocm.DeviceBuffer.from_numpy(padded(g, skew_in))
    dl = rocm.DeviceBuffer.from_numpy(padded(y, skew_in))
    dd = rocm.DeviceBuffer.from_numpy(np.full(x.size + 2 * pad, 7.0, dtype=dtype))
    rocm.log_softmax_bwd_raw(dtype, at(dg, skew_in), at(dl, skew_in), at(dd, skew_out), outer, inner)
    got = dd.numpy()
    d = got[skew_out:skew_out + x.size].reshape(outer, inner)
    assert (got[:skew_out] == 7.0).all() and (got[skew_out + x.size:] == 7.0).all()
    want_d = oracle.log_softmax_bwd(g.astype(np.float32), y.astype(np.float32))
    tol = 5e-3 + np.abs(want_d).max() * 2 ** -11 if dtype == np.float16 else 1e-4
    assert np.abs(d.astype(np.float32) - want_d).max() <= tol


@pytest.mark.gpu
def test_extreme_rows_stay_finite():
    x = np.zeros((4, 1000), dtype=np.float32)
    x[0] = 1e4                 # naive exp overflows
    x[1, ::2] = -1e4           # half the row underflows to probability 0
    x[2] = -3e4
    x[3, 7] = 88.0
    y = _run_fwd(x)
    want = oracle.log_softmax_fwd(x)
    assert np.isfinite(y).all()
    assert np.abs(y - want).max() <= 1e-3  # values near 1e4 carry an f32 ulp of 1e-3
    assert np.abs(y[0] + np.log(1000.0)).max() < 1e-3
    xh = x.astype(np.float16)  # 1e4 is finite in f16, -3e4 too
    yh = _run_fwd(xh)
    assert np.isfinite(yh).all()


@pytest.mark.gpu
def test_in_place_is_allowed():
    x = synth.normal((9, 777), synth.tensor_seed(32, "lsm", "x"), 2.0).astype(np.float32)
    g = synth.normal((9, 777), synth.tensor_seed(32, "lsm", "g"), 1.0).astype(np.float32)
    y = _run_fwd(x)
    buf = rocm.DeviceBuffer.from_numpy(x)
    rocm.log_softmax_fwd_raw(np.float32, buf.ptr, buf.ptr, 9, 777)
    assert np.array_equal(buf.numpy(), y)
    dg, dl = rocm.DeviceBuffer.from_numpy(g), rocm.DeviceBuffer.from_numpy(y)
    want = _run_bwd(g, y)
    rocm.log_softmax_bwd_raw(np.float32, dg.ptr, dl.ptr, dg.ptr, 9, 777)
    assert np.array_equal(dg.numpy(), want)


@pytest.mark.gpu
def test_properties_at_the_loss_shape():
    # GPT-2 vocabulary width, 1024 of config 5's 8192 rows (rows are independent):
    # probabilities sum to one, gradients of a one-hot-weighted loss sum to zero per row
    outer, inner = 1024, 50257
    x = synth.normal((outer, inner), synth.tensor_seed(33, "lsm", "x"), 2.0).astype(np.float32)
    dx_ = rocm.DeviceBuffer.from_numpy(x)
    y = rocm.DeviceBuffer(x.shape, np.float32)
    rocm.log_softmax_fwd_raw(np.float32, dx_.ptr, y.ptr, outer, inner)
    yh = y.numpy()
    assert np.abs(np.exp(yh.astype(np.float64)).sum(axis=1) - 1).max() < 1e-5
    assert np.abs((x - yh) - (x - yh)[:, :1]).max() < 1e-4  # x - y is the row's lse
    g = np.zeros_like(x)
    g[np.arange(outer), np.arange(outer) % inner] = -1.0 / outer  # nll_loss's upstream gradient
    dg = rocm.DeviceBuffer.from_numpy(g)
    out = rocm.DeviceBuffer(x.shape, np.float32)
    rocm.log_softmax_bwd_raw(np.float32, dg.ptr, y.ptr, out.ptr, outer, inner)
    d = out.numpy().astype(np.float64)
    assert np.abs(d.sum(axis=1)).max() < 1e-7
    # cross-entropy gradient: (softmax - onehot) / outer
    assert np.abs(d - (np.exp(yh.astype(np.float64)) / outer + g)).max() < 1e-7


@pytest.mark.gpu
def test_argument_errors():
    buf = rocm.DeviceBuffer((4, 4), np.float32)
    with pytest.raises(rocm.RocmError):
        rocm.log_softmax_fwd_raw(np.float32, buf.ptr, buf.ptr, 4, 0)
    with pytest.raises(rocm.RocmError):
        rocm.log_softmax_fwd_raw(np.float32, ctypes.c_void_p(), buf.ptr, 4, 4)
    with pytest.raises(rocm.RocmError):
        rocm.log_softmax_bwd_raw(np.float32, buf.ptr, ctypes.c_void_p(), buf.ptr, 4, 4)
    rocm.log_softmax_fwd_raw(np.float32, ctypes.c_void_p(), ctypes.c_void_p(), 0, 4)  # empty: no-op
