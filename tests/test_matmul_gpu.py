"""deers_rocm_matmul (library GEMM behind BackendStorage::matmul) against the CPU oracle's
gemm_strided restatement and the reference's own integer-valued conformance cases
(tests/tensor.rs:83-110)."""
import ctypes

import numpy as np
import pytest

import oracle
from deers_amd import rocm


@pytest.fixture(scope="module", autouse=True)
def _init():
    if not rocm.available():
        pytest.skip("no gfx950 device")
    rocm.init(0)


def _close(got, want, dtype, tol):
    """f32: max abs error <= tol (1e-4, scaled by the largest value where the caller says so).
    f16: the product is an f32-accumulated sum rounded once to f16, so each element is held to
    half an f16 unit of its exact value (2^-11 relative) plus 1e-3 for the order of the f32
    accumulation: 3e-3 for values up to 4, inside the path's 5e-3."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    if np.dtype(dtype) == np.float16:
        return bool(np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -11 + 1e-3))
    return bool(np.max(np.abs(got - want), initial=0.0) <= tol)


def _run(a, b, dtype, a_view=None, b_view=None):
    """a [batch,m,k], b [batch,k,n] numpy; *_view = (buffer array, (rs, cs, bs))."""
    batch, m, k = a.shape
    n = b.shape[2]
    abuf, astr = a_view if a_view else (np.ascontiguousarray(a), (k, 1, m * k))
    bbuf, bstr = b_view if b_view else (np.ascontiguousarray(b), (n, 1, k * n))
    da, db = rocm.DeviceBuffer.from_numpy(abuf.astype(dtype)), rocm.DeviceBuffer.from_numpy(bbuf.astype(dtype))
    dc = rocm.DeviceBuffer((batch, m, n), dtype)
    rocm.matmul_raw(dtype, da.ptr, astr, db.ptr, bstr, dc.ptr, batch, m, n, k)
    return dc.numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_matmul_reference_integer_cases(dtype):
    a = np.array([[[1, 2, 3], [4, 5, 6]]], np.float32)
    b = np.array([[[7, 8], [9, 10], [11, 12]]], np.float32)
    assert np.array_equal(_run(a, b, dtype)[0], np.array([[58, 64], [139, 154]], dtype))
    # batched 2x2x3 @ 2x3x2
    a2 = np.arange(12, dtype=np.float32).reshape(2, 2, 3)
    b2 = np.arange(12, dtype=np.float32).reshape(2, 3, 2)
    assert np.array_equal(_run(a2, b2, dtype), np.einsum("bmk,bkn->bmn", a2, b2).astype(dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float16, None), (np.float32, 1e-4)])
@pytest.mark.parametrize("batch,m,n,k", [(1, 1, 1, 1), (3, 5, 7, 9), (2, 130, 33, 64), (1, 1024, 768, 768)])
def test_matmul_matches_oracle(dtype, tol, batch, m, n, k):
    rng = np.random.default_rng(31)
    a = rng.standard_normal((batch, m, k)).astype(dtype)
    b = (rng.standard_normal((batch, k, n)) / np.sqrt(k)).astype(dtype)
    want = oracle.matmul(a.astype(np.float32), b.astype(np.float32))
    assert _close(_run(a, b, dtype), want, dtype, tol)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float16, None), (np.float32, 1e-4)])
def test_matmul_transposed_views_and_broadcast_weights(dtype, tol):
    rng = np.random.default_rng(32)
    batch, m, n, k = 4, 17, 24, 40
    a = rng.standard_normal((batch, m, k)).astype(dtype)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(dtype)
    want = np.einsum("bmk,kn->bmn", a.astype(np.float32), w.astype(np.float32))
    # b is one [k,n] weight for every batch entry: batch stride 0
    got = _run(a, np.broadcast_to(w, (batch, k, n)), dtype, b_view=(w, (n, 1, 0)))
    assert _close(got, want, dtype, tol)
    # a given as the transposed view of an [batch,k,m] buffer (dB = A^T @ dC in MatMul::backward)
    at = np.ascontiguousarray(a.transpose(0, 2, 1))
    got_t = _run(a, np.broadcast_to(w, (batch, k, n)), dtype, a_view=(at, (1, m, k * m)),
                 b_view=(w, (n, 1, 0)))
    assert np.array_equal(got_t, got)
    # b given as the transposed view of an [n,k] buffer (dA = dC @ B^T)
    wt = np.ascontiguousarray(w.T)
    got_bt = _run(a, np.broadcast_to(w, (batch, k, n)), dtype, b_view=(wt, (1, k, 0)))
    assert _close(got_bt, want, dtype, tol)


@pytest.mark.gpu
def test_matmul_edge_cases_and_errors():
    buf = rocm.DeviceBuffer((64,), np.float32, zeros=True)
    out = rocm.DeviceBuffer.from_numpy(np.ones((2, 3), np.float32))
    rocm.matmul_raw(np.float32, buf.ptr, (0, 1, 0), buf.ptr, (3, 1, 0), out.ptr, 1, 2, 3, 0)  # k = 0
    assert np.array_equal(out.numpy(), np.zeros((2, 3), np.float32))
    rocm.matmul_raw(np.float32, buf.ptr, (4, 1, 0), buf.ptr, (3, 1, 0), out.ptr, 1, 0, 3, 4)  # m = 0: no-op
    with pytest.raises(rocm.RocmError):  # neither stride of a is 1
        rocm.matmul_raw(np.float32, buf.ptr, (8, 2, 0), buf.ptr, (3, 1, 0), out.ptr, 1, 2, 3, 4)
    with pytest.raises(rocm.RocmError):
        rocm.matmul_raw(np.float32, None, (4, 1, 0), buf.ptr, (3, 1, 0), out.ptr, 1, 2, 3, 4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float16, None), (np.float32, 1e-4)])
def test_matmul_with_kernel_tuning_gives_the_same_product(dtype, tol):
    # with tuning on, the first call of a problem times every kernel the BLAS lists for it;
    # whatever it settles on, the product is the same within the type's tolerance, on plain,
    # transposed and broadcast operands, on the first (tuning) call and on later ones
    rng = np.random.default_rng(35)
    rocm.matmul_tune(True)
    try:
        for batch, m, n, k in [(1, 512, 96, 768), (2, 130, 33, 64), (1, 64, 1000, 192)]:
            a = rng.standard_normal((batch, m, k)).astype(dtype)
            b = (rng.standard_normal((batch, k, n)) / np.sqrt(k)).astype(dtype)
            want = oracle.matmul(a.astype(np.float32), b.astype(np.float32))
            for _ in range(2):
                assert _close(_run(a, b, dtype), want, dtype, tol)
            # A^T stored: logical a[b,i,j] = buf[b,j,i]
            at = np.ascontiguousarray(a.transpose(0, 2, 1))
            for _ in range(2):
                got = _run(a, b, dtype, a_view=(at, (1, m, m * k)))
                assert _close(got, want, dtype, tol)
    finally:
        rocm.matmul_tune(False)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float16, None), (np.float32, 1e-4)])
@pytest.mark.parametrize("batch,m,n,k", [(1, 32, 768, 768), (2, 7, 33, 64), (1, 5, 3, 1)])
def test_matmul_acc_adds_the_product_into_c(dtype, tol, batch, m, n, k):
    """deers_rocm_matmul_acc: c += a @ b (the residual add of src/models/gpt.rs:237-239 riding on
    the projection), against the oracle's product plus the addend."""
    rng = np.random.default_rng(batch * 1000 + m)
    a = rng.standard_normal((batch, m, k)).astype(dtype)
    b = rng.standard_normal((batch, k, n)).astype(dtype)
    c0 = rng.standard_normal((batch, m, n)).astype(dtype)
    da, db, dc = (rocm.DeviceBuffer.from_numpy(x) for x in (a, b, c0))
    rocm.matmul_acc_raw(dtype, da.ptr, (k, 1, m * k), db.ptr, (n, 1, k * n), dc.ptr, batch, m, n, k)
    want = oracle.matmul(a.astype(np.float32), b.astype(np.float32)) + c0.astype(np.float32)
    # b is not scaled by 1/sqrt(k) here: values reach ~100, so the f32 bound scales with them
    ftol = None if tol is None else tol * max(1.0, float(np.abs(want).max()))
    got1 = dc.numpy()
    assert _close(got1, want, dtype, ftol)
    # twice more: the accumulator keeps growing by the same product (the second call adds to the
    # first call's ROUNDED result, so the expectation starts from what the device holds)
    rocm.matmul_acc_raw(dtype, da.ptr, (k, 1, m * k), db.ptr, (n, 1, k * n), dc.ptr, batch, m, n, k)
    want2 = got1.astype(np.float32) + oracle.matmul(a.astype(np.float32), b.astype(np.float32))
    ftol2 = None if tol is None else tol * max(1.0, float(np.abs(want2).max()))
    assert _close(dc.numpy(), want2, dtype, ftol2)
    # k = 0 leaves c alone
    before = dc.numpy()
    rocm.matmul_acc_raw(dtype, da.ptr, (1, 1, 1), db.ptr, (n, 1, 1), dc.ptr, batch, m, n, 0)
    assert np.array_equal(dc.numpy(), before)


@pytest.mark.gpu
@pytest.mark.parametrize("tune", [False, True])
@pytest.mark.parametrize("dtype,tol", [(np.float16, None), (np.float32, 1e-4)])
@pytest.mark.parametrize("batch,m,n,k", [(1, 256, 768, 768), (1, 32, 768, 768), (2, 7, 33, 64), (1, 5, 3, 1)])
def test_matmul_add_writes_product_plus_addend_elsewhere(dtype, tol, batch, m, n, k, tune):
    """deers_rocm_matmul_add: c = a @ b + addend with the addend left as it is (the residual
    stream of src/models/gpt.rs:237-239 inside an autograd graph, or a gradient that another
    entry of the store shares, src/backprop.rs:101-112), what deers_rocm_matmul_acc gives on a
    copy of the addend; with the kernel picked by timing as well, whose trial runs must
    touch neither the addend nor the output's final value; k = 0 copies the addend."""
    rng = np.random.default_rng(batch * 1000 + m + n)
    a = rng.standard_normal((batch, m, k)).astype(dtype)
    b = (rng.standard_normal((batch, k, n)) / np.sqrt(k)).astype(dtype)
    c0 = rng.standard_normal((batch, m, n)).astype(dtype)
    da, db, dadd, dacc = (rocm.DeviceBuffer.from_numpy(x) for x in (a, b, c0, c0))
    dc = rocm.DeviceBuffer((batch, m, n), dtype)
    rocm.matmul_tune(tune)
    try:
        for _ in range(2):  # the second call of a tuned problem takes the remembered kernel
            rocm.matmul_add_raw(dtype, da.ptr, (k, 1, m * k), db.ptr, (n, 1, k * n), dadd.ptr, dc.ptr, batch, m, n, k)
            assert np.array_equal(dadd.numpy(), c0)
            want = oracle.matmul(a.astype(np.float32), b.astype(np.float32)) + c0.astype(np.float32)
            ftol = None if tol is None else tol * max(1.0, float(np.abs(want).max()))
            assert _close(dc.numpy(), want, dtype, ftol)
        rocm.matmul_acc_raw(dtype, da.ptr, (k, 1, m * k), db.ptr, (n, 1, k * n), dacc.ptr, batch, m, n, k)
        # (a few f16 rows against a weight matrix accumulate in place on the library's own kernel,
        # out of place on the BLAS: one rounding either way, not always the same bits)
        assert _close(dc.numpy(), dacc.numpy().astype(np.float32), dtype, ftol)
        # the addend may be the output
        rocm.matmul_add_raw(dtype, da.ptr, (k, 1, m * k), db.ptr, (n, 1, k * n), dadd.ptr, dadd.ptr, batch, m, n, k)
        assert np.array_equal(dadd.numpy(), dacc.numpy())
        rocm.matmul_add_raw(dtype, da.ptr, (1, 1, 1), db.ptr, (n, 1, 1), dacc.ptr, dc.ptr, batch, m, n, 0)
        assert np.array_equal(dc.numpy(), dacc.numpy())
    finally:
        rocm.matmul_tune(False)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float16, None), (np.float32, 1e-4)])
def test_matmul_add_takes_transposed_and_broadcast_operands(dtype, tol):
    """The gradient products that carry an addend read views: out_grad @ w^T with w^T the
    transposed view of a weight (MatMul::backward, src/ops.rs:1089-1101), x^T @ out_grad with x^T
    a transposed view, and a batch of left operands against one broadcast right operand
    (batch stride 0).  Same operand rules as deers_rocm_matmul."""
    rng = np.random.default_rng(99)
    m, n, k, batch = 96, 40, 64, 3
    # b^T: the weight is stored [n, k]; the product reads it as [k, n] through strides (1, k)
    a = rng.standard_normal((1, m, k)).astype(dtype)
    w = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(dtype)
    c0 = rng.standard_normal((1, m, n)).astype(dtype)
    da, dw, dadd = (rocm.DeviceBuffer.from_numpy(x) for x in (a, w, c0))
    dc = rocm.DeviceBuffer((1, m, n), dtype)
    rocm.matmul_add_raw(dtype, da.ptr, (k, 1, 0), dw.ptr, (1, k, 0), dadd.ptr, dc.ptr, 1, m, n, k)
    want = oracle.matmul(a.astype(np.float32), w.T[None].astype(np.float32)) + c0.astype(np.float32)
    assert _close(dc.numpy(), want, dtype, None if tol is None else tol * max(1.0, float(np.abs(want).max())))
    # a^T: x stored [m, k] read as [k, m]; x^T @ g + addend, a weight gradient onto a held one
    g = (rng.standard_normal((1, m, n)) / np.sqrt(m)).astype(dtype)
    acc = rng.standard_normal((1, k, n)).astype(dtype)
    dg, dacc = rocm.DeviceBuffer.from_numpy(g), rocm.DeviceBuffer.from_numpy(acc)
    dout = rocm.DeviceBuffer((1, k, n), dtype)
    rocm.matmul_add_raw(dtype, da.ptr, (1, k, 0), dg.ptr, (n, 1, 0), dacc.ptr, dout.ptr, 1, k, n, m)
    want = oracle.matmul(a[0].T[None].astype(np.float32), g.astype(np.float32)) + acc.astype(np.float32)
    assert _close(dout.numpy(), want, dtype, None if tol is None else tol * max(1.0, float(np.abs(want).max())))
    assert np.array_equal(dacc.numpy(), acc)
    # a batch of left operands against one right operand (batch stride 0)
    ab = rng.standard_normal((batch, m, k)).astype(dtype)
    b1 = (rng.standard_normal((1, k, n)) / np.sqrt(k)).astype(dtype)
    cb = rng.standard_normal((batch, m, n)).astype(dtype)
    dab, db1, dcb = (rocm.DeviceBuffer.from_numpy(x) for x in (ab, b1, cb))
    dob = rocm.DeviceBuffer((batch, m, n), dtype)
    rocm.matmul_add_raw(dtype, dab.ptr, (k, 1, m * k), db1.ptr, (n, 1, 0), dcb.ptr, dob.ptr, batch, m, n, k)
    want = oracle.matmul(ab.astype(np.float32), np.broadcast_to(b1, (batch, k, n)).astype(np.float32)) + cb.astype(np.float32)
    assert _close(dob.numpy(), want, dtype, None if tol is None else tol * max(1.0, float(np.abs(want).max())))


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(32, 768, 768), (32, 3072, 768), (32, 768, 3072), (7, 2304, 768),
                                   (1, 768, 256), (32, 776, 512), (5, 8, 256), (31, 40, 1024)])
def test_few_rows_against_a_weight_matrix_take_the_streaming_kernel(m, n, k):
    """f16 products with at most 32 rows, K a multiple of 256 and N a multiple of 8 (a generation
    step's projections) run on the library's own one-pass kernel instead of the BLAS: same
    contract (f32 accumulation, one rounding), checked against the oracle, with and without the
    addend, through a strided x (rows of a wider buffer) as well."""
    rng = np.random.default_rng(m * 7 + n + k)
    a = rng.standard_normal((1, m, k)).astype(np.float16)
    b = (rng.standard_normal((1, k, n)) / np.sqrt(k)).astype(np.float16)
    want = oracle.matmul(a.astype(np.float32), b.astype(np.float32))
    got = _run(a, b, np.float16)
    assert np.abs(got.astype(np.float32) - want).max() <= 4e-3 * max(1.0, float(np.abs(want).max()))
    # y += x @ W, the addend added in f32 before the single rounding
    c0 = rng.standard_normal((1, m, n)).astype(np.float16)
    da, db, dc = (rocm.DeviceBuffer.from_numpy(x) for x in (a, b, c0))
    rocm.matmul_acc_raw(np.float16, da.ptr, (k, 1, m * k), db.ptr, (n, 1, k * n), dc.ptr, 1, m, n, k)
    want_acc = want + c0.astype(np.float32)
    assert np.abs(dc.numpy().astype(np.float32) - want_acc).max() <= 4e-3 * max(1.0, float(np.abs(want_acc).max()))
    assert np.array_equal(dc.numpy(), (want_acc.astype(np.float16))) or \
        np.abs(dc.numpy().astype(np.float32) - want_acc.astype(np.float16).astype(np.float32)).max() <= 2e-3 * max(1.0, float(np.abs(want_acc).max()))
    # x as the middle third of a [m, 3k] buffer (row stride 3k)
    wide = rng.standard_normal((m, 3 * k)).astype(np.float16)
    dw = rocm.DeviceBuffer.from_numpy(wide)
    import ctypes
    dc2 = rocm.DeviceBuffer((1, m, n), np.float16)
    rocm.matmul_raw(np.float16, ctypes.c_void_p(dw.ptr.value + k * 2), (3 * k, 1, 0), db.ptr, (n, 1, k * n),
                    dc2.ptr, 1, m, n, k)
    want2 = oracle.matmul(wide[None, :, k:2 * k].astype(np.float32), b.astype(np.float32))
    assert np.abs(dc2.numpy().astype(np.float32) - want2).max() <= 4e-3 * max(1.0, float(np.abs(want2).max()))
    # bit-reproducible
    got2 = _run(a, b, np.float16)
    assert np.array_equal(got, got2)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(32, 2304, 768), (32, 3072, 768), (32, 768, 3072), (3, 16, 256),
                                   (17, 776, 1024)])
def test_decode_linear_prologues(m, n, k):
    """deers_rocm_decode_linear: the weightless RMSNorm of src/nn.rs:244-251 and the MLP's
    relu(x)^2 (src/models/gpt.rs:196-203) folded into the few-rows product.  relu_sq gives the
    bits of relu_sq_fwd followed by matmul; rms_norm skips the f16 rounding of the normalised
    row, so it is compared with the f64 evaluation at the f16 tolerance; both with and without
    the addend."""
    rng = np.random.default_rng(m + 3 * n + 5 * k)
    x = (rng.standard_normal((m, k)) * 1.7).astype(np.float16)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float16)
    y0 = rng.standard_normal((m, n)).astype(np.float16)
    eps = 1e-5
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    dx, dw = rocm.DeviceBuffer.from_numpy(x), rocm.DeviceBuffer.from_numpy(w)

    def run(prologue, accumulate):
        dy = rocm.DeviceBuffer.from_numpy(y0.copy())
        rocm.decode_linear_raw(np.float16, prologue, eps, dx.ptr, k, dw.ptr, n, dy.ptr, accumulate, m, n, k)
        return dy.numpy()

    # rms_norm: row factor from the definition
    inv = 1.0 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps)
    want = (x64 * inv) @ w64
    for acc in (False, True):
        ref = want + (y0.astype(np.float64) if acc else 0.0)
        got = run("rms_norm", acc).astype(np.float64)
        assert np.abs(got - ref).max() <= 4e-3 * max(1.0, np.abs(ref).max()), acc
    # relu_sq: same bits as the two separate entry points
    r = rocm.DeviceBuffer((m, k), np.float16)
    rocm.relu_sq_fwd_raw(np.float16, dx.ptr, r.ptr, m * k)
    sep = rocm.DeviceBuffer((m, n), np.float16)
    rocm.matmul_raw(np.float16, r.ptr, (k, 1, m * k), dw.ptr, (n, 1, k * n), sep.ptr, 1, m, n, k)
    assert np.array_equal(run("relu_sq", False), sep.numpy())
    want_r = (np.maximum(x.astype(np.float32), 0) ** 2).astype(np.float16).astype(np.float64) @ w64
    got = run("relu_sq", True).astype(np.float64)
    ref = want_r + y0.astype(np.float64)
    assert np.abs(got - ref).max() <= 4e-3 * max(1.0, np.abs(ref).max())
    # the packed weight layout [n/32][k][32] gives the same bits as the row-major one
    if n % 32 == 0:
        tiles = np.ascontiguousarray(w.reshape(k, n // 32, 32).transpose(1, 0, 2))
        dt_ = rocm.DeviceBuffer.from_numpy(tiles)
        for prologue in ("plain", "rms_norm", "relu_sq"):
            dy = rocm.DeviceBuffer.from_numpy(y0.copy())
            rocm.decode_linear_raw(np.float16, prologue, eps, dx.ptr, k, dt_.ptr, rocm.LINEAR_W_PACKED, dy.ptr,
                                   True, m, n, k)
            assert np.array_equal(dy.numpy(), run(prologue, True)), prologue
        # and copy_view with the documented strides is the packing
        packed = rocm.DeviceBuffer((n // 32, k, 32), np.float16)
        rocm.copy_view_raw(np.float16, dw.ptr, (32, n, 1), packed.ptr, (32 * k, 32, 1), (n // 32, k, 32))
        assert np.array_equal(packed.numpy(), tiles)
    # plain = deers_rocm_matmul on the same operands
    plain = rocm.DeviceBuffer((m, n), np.float16)
    rocm.matmul_raw(np.float16, dx.ptr, (k, 1, m * k), dw.ptr, (n, 1, k * n), plain.ptr, 1, m, n, k)
    assert np.array_equal(run("plain", False), plain.numpy())


@pytest.mark.gpu
def test_decode_linear_rejects_what_the_kernel_does_not_take():
    x = rocm.DeviceBuffer((40, 512), np.float16)
    w = rocm.DeviceBuffer((512, 64), np.float16)
    y = rocm.DeviceBuffer((40, 64), np.float16)
    for m, n, k in ((40, 64, 512), (8, 60, 512), (8, 64, 384)):
        with pytest.raises(rocm.RocmError):
            rocm.decode_linear_raw(np.float16, "plain", 0.0, x.ptr, 512, w.ptr, 64, y.ptr, False, m, n, k)
    with pytest.raises(rocm.RocmError):
        rocm.decode_linear_raw(np.float32, "plain", 0.0, x.ptr, 512, w.ptr, 64, y.ptr, False, 8, 64, 512)


@pytest.mark.gpu
@pytest.mark.parametrize("n,k,n2,k2", [(2304, 768, 768, 768), (768, 3072, 2304, 768), (768, 768, 768, 3072),
                                       (64, 256, 3072, 768)])
def test_decode_linear_prefetch_hint_changes_nothing_but_time(n, k, n2, k2):
    """deers_rocm_decode_linear_hint names the packed weight of the following product; the launch
    it rides on (split or not) gives the same bits with and without it, the hinted weight is
    only read, and a hint is used once."""
    m = 32
    rng = np.random.default_rng(n + k + n2)
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float16)
    nxt = rng.standard_normal((n2 // 32, k2, 32)).astype(np.float16)
    dx, dw, dn = (rocm.DeviceBuffer.from_numpy(a) for a in (x, w, nxt))
    y0 = rng.standard_normal((m, n)).astype(np.float16)

    def run(hint):
        dy = rocm.DeviceBuffer.from_numpy(y0.copy())
        if hint:
            rocm.decode_linear_hint_raw(dn.ptr, n2, k2)
        rocm.decode_linear_raw(np.float16, "relu_sq", 0.0, dx.ptr, k, dw.ptr, n, dy.ptr, True, m, n, k)
        return dy.numpy()

    plain = run(False)
    assert np.array_equal(run(True), plain)
    assert np.array_equal(run(False), plain)      # the hint did not linger
    assert np.array_equal(dn.numpy(), nxt)        # and its target is untouched
    rocm.decode_linear_hint_raw(dn.ptr, n2, k2)
    rocm.decode_linear_hint_raw(None, 0, 0)       # cleared again
    assert np.array_equal(run(False), plain)
    with pytest.raises(rocm.RocmError):
        rocm.decode_linear_hint_raw(ctypes.c_void_p(dn.ptr.value + 2), n2, k2)   # unaligned
