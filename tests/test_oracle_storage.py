"""Pins oracle/storage_ops.py (the generic storage kernels of src/storage/cpu.rs) before the GPU
tests trust it: literal inputs of the reference's own tests evaluated with library routines
(numpy's half arithmetic, scipy, torch on the CPU), closed forms, and brute-force loops in the
reference's element order."""
import math

import numpy as np
import pytest
import scipy.special
import torch

from oracle import storage_ops as so


def _rand(shape, seed, dtype=np.float32, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(dtype)


# ---- unary ------------------------------------------------------------------------------------

def test_unary_closed_forms():
    x = np.array([0.0, 1.0, -2.0, 0.5], np.float32)
    assert so.unary("neg", x).tolist() == [-0.0, -1.0, 2.0, -0.5]
    assert np.signbit(so.unary("neg", x)[0])
    assert so.unary("relu", x).tolist() == [0.0, 1.0, 0.0, 0.5]
    assert so.unary("relu_backward", x).tolist() == [0.0, 1.0, 0.0, 1.0]
    np.testing.assert_allclose(so.unary("exp", x), [1.0, math.e, math.exp(-2), math.exp(0.5)], rtol=1e-6)
    np.testing.assert_allclose(so.unary("log", np.array([1.0, math.e, 8.0], np.float32)),
                               [0.0, 1.0, math.log(8)], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(so.unary("sin", np.array([0.0, math.pi / 2], np.float32)), [0.0, 1.0], atol=1e-7)
    np.testing.assert_allclose(so.unary("cos", np.array([0.0, math.pi], np.float32)), [1.0, -1.0], atol=1e-7)
    np.testing.assert_allclose(so.unary("tanh", np.array([0.0, 20.0, -20.0], np.float32)), [0.0, 1.0, -1.0])
    assert so.unary("scalar_add", x, 1.5).tolist() == [1.5, 2.5, -0.5, 2.0]
    assert so.unary("scalar_mul", x, -2.0).tolist() == [-0.0, -2.0, 4.0, -1.0]
    assert so.unary("scalar_div", x, 4.0).tolist() == [0.0, 0.25, -0.5, 0.125]
    assert so.unary("powf", np.array([2.0, 3.0, 9.0], np.float32), 2.0).tolist() == [4.0, 9.0, 81.0]
    assert so.unary("powf", np.array([4.0, 9.0], np.float32), 0.5).tolist() == [2.0, 3.0]


def test_unary_special_values():
    x = np.array([np.nan, -np.inf, np.inf, -0.0], np.float32)
    assert so.unary("relu", x).tolist() == [0.0, 0.0, np.inf, 0.0]          # f32::max drops the NaN
    assert so.unary("relu_backward", x).tolist() == [0.0, 0.0, 1.0, 0.0]    # NaN > 0 is false
    assert np.isnan(so.unary("exp", x)[0]) and so.unary("exp", x)[1] == 0.0
    assert np.isnan(so.unary("log", np.array([-1.0], np.float32))[0])
    assert so.unary("log", np.array([0.0], np.float32))[0] == -np.inf


@pytest.mark.parametrize("op", ["exp", "log", "sin", "cos", "tanh"])
@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_unary_against_torch(op, dtype):
    x = _rand((7, 33), 3, dtype, 2.0)
    if op == "log":
        x = np.abs(x) + dtype(0.01)
    want = getattr(torch, op)(torch.from_numpy(x)).numpy()
    got = so.unary(op, x)
    if dtype == np.float16:  # both compute in f32 and round once: at most one f16 ulp apart
        assert np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32)).max() <= 1
    else:
        np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-7)


def test_unary_f16_scalar_is_rounded_to_f16_first():
    # scalar_op! macro: v op f16::from_f32(s as f32); numpy's own half arithmetic is the check
    x = _rand(4096, 5, np.float16, 30.0)
    for p in (0.1, 1.0 / 3.0, 1.0009765625 + 2.0 ** -13, 7.3):
        ph = np.float16(np.float32(p))
        assert np.array_equal(so.unary("scalar_mul", x, p), x * ph)
        assert np.array_equal(so.unary("scalar_add", x, p), x + ph)
        assert np.array_equal(so.unary("scalar_div", x, p), x / ph)
    # and the distinction matters: multiplying by the f32 scalar gives other bits somewhere
    f32_route = (x.astype(np.float32) * np.float32(0.1)).astype(np.float16)
    assert not np.array_equal(so.unary("scalar_mul", x, 0.1), f32_route)


def test_powf_exponent_is_not_rounded_to_f16():
    x = (np.abs(_rand(2048, 6, np.float16)) + np.float16(0.5)).astype(np.float16)
    e = 2.0 + 2.0 ** -12  # not representable in f16
    want = np.power(x.astype(np.float32), np.float32(e)).astype(np.float16)
    assert np.array_equal(so.unary("powf", x, e), want)
    rounded = np.power(x.astype(np.float32), np.float32(np.float16(e))).astype(np.float16)
    assert np.array_equal(rounded, np.power(x.astype(np.float32), np.float32(2.0)).astype(np.float16))


# ---- binary -----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_binary_against_library_arithmetic(dtype):
    a, b = _rand((5, 17), 8, dtype, 3.0), _rand((5, 17), 9, dtype, 3.0)
    b[0, 0] = a[0, 0]
    with np.errstate(all="ignore"):
        assert np.array_equal(so.binary("add", a, b), a + b)
        assert np.array_equal(so.binary("sub", a, b), a - b)
        assert np.array_equal(so.binary("mul", a, b), a * b)
        assert np.array_equal(so.binary("div", a, b), a / b)
    eq = so.binary("eq", a, b)
    assert eq[0, 0] == 1 and eq.sum() == (a == b).sum() and eq.dtype == dtype
    ap = np.abs(a) + dtype(0.1)
    with np.errstate(over="ignore"):
        want = torch.pow(torch.from_numpy(ap).float(), torch.from_numpy(b).float()).numpy().astype(dtype)
    got = so.binary("pow", ap, b)
    if dtype == np.float16:
        assert np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32)).max() <= 1
    else:
        np.testing.assert_allclose(got, want, rtol=2e-6)


def test_binary_broadcast_view_and_nan_equality():
    a = _rand((4, 6), 1)
    row = _rand((1, 6), 2)
    b = np.broadcast_to(row, (4, 6))  # stride-0 view, as the Broadcast op hands over
    assert np.array_equal(so.binary("add", a, b), a + row)
    n = np.array([np.nan, 1.0], np.float32)
    assert so.binary("eq", n, n).tolist() == [0.0, 1.0]
    assert so.binary("add", np.array([-np.inf], np.float32), np.array([3.0], np.float32))[0] == -np.inf


# ---- reduce -----------------------------------------------------------------------------------

def test_reduce_reference_literals():
    # tests/tensor.rs:515-538 (sum over axis 1 of [[1,2,3],[4,5,6]]) and 625-648 (max of [[1,3],[2,4]])
    assert so.reduce("sum", np.array([[1, 2, 3], [4, 5, 6]], np.float32)).tolist() == [6.0, 15.0]
    assert so.reduce("max", np.array([[1, 3], [2, 4]], np.float32)).tolist() == [3.0, 4.0]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_reduce_is_left_to_right_in_the_storage_type(dtype):
    x = _rand((9, 41), 11, dtype, 10.0)
    want = []
    for row in x:  # brute force with numpy scalars of the storage type
        acc = row[0]
        for v in row[1:]:
            acc = dtype(acc + v)
        want.append(acc)
    assert np.array_equal(so.reduce("sum", x), np.array(want, dtype))
    assert np.array_equal(so.reduce("max", x), x.max(axis=1))
    if dtype == np.float32:
        np.testing.assert_allclose(so.reduce("sum", x), [math.fsum(r.tolist()) for r in x], rtol=1e-5)
    else:  # the f16 accumulator is visibly worse than an exact sum: that is what the reference does
        exact = np.array([math.fsum(r.astype(np.float64).tolist()) for r in x])
        assert np.abs(so.reduce("sum", x).astype(np.float64) - exact).max() > 0


def test_reduce_max_nan_handling():
    x = np.array([[np.nan, 1.0, 2.0], [3.0, np.nan, -1.0], [np.nan, np.nan, np.nan]], np.float32)
    r = so.reduce("max", x)
    assert r[0] == 2.0 and r[1] == 3.0 and np.isnan(r[2])


# ---- log-sum-exp ------------------------------------------------------------------------------

def test_log_sum_exp_reference_literal():
    # tests/tensor.rs:1885-1909
    x = np.array([[1.0, 2.0, 3.0], [1.5, 0.5, -1.0]], np.float32)
    got = so.log_sum_exp(x)
    np.testing.assert_allclose(got, scipy.special.logsumexp(x.astype(np.float64), axis=1), rtol=1e-6)
    np.testing.assert_allclose(got[0], 3 + math.log(1 + math.exp(-1) + math.exp(-2)), rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_log_sum_exp_against_scipy(dtype):
    x = _rand((13, 257), 21, dtype, 4.0)
    want = scipy.special.logsumexp(x.astype(np.float64), axis=1)
    got = so.log_sum_exp(x)
    assert got.dtype == dtype
    np.testing.assert_allclose(got.astype(np.float64), want, rtol=1e-3 if dtype == np.float16 else 1e-5)
    big = (x.astype(np.float32) + 1000).astype(np.float32)  # overflow-safe
    np.testing.assert_allclose(so.log_sum_exp(big), scipy.special.logsumexp(big.astype(np.float64), axis=1),
                               rtol=1e-6)


def test_log_sum_exp_special_rows():
    inf = np.inf
    x = np.array([[-inf, 1.0, -inf], [-inf, -inf, -inf], [inf, 0.0, 1.0], [np.nan, 0.0, 1.0]], np.float32)
    r = so.log_sum_exp(x)
    assert r[0] == 1.0           # -inf entries contribute exp(-inf) = 0
    assert np.isnan(r[1])        # max = -inf: (-inf) - (-inf) is NaN, as in the reference
    assert np.isnan(r[2])        # max = +inf: inf - inf
    assert np.isnan(r[3])        # the NaN is skipped by the max but not by the sum


# ---- gather / scatter_add / cat ---------------------------------------------------------------

def test_gather_reference_literal():
    # tests/tensor.rs:2226-2257
    data = np.array([[10, 20, 30], [40, 50, 60]], np.float32)
    idx = np.array([[1], [2]], np.int64)
    assert so.gather(data, 1, idx).tolist() == [[20.0], [60.0]]


@pytest.mark.parametrize("dim", [0, 1, 2])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int64])
def test_gather_against_libraries(dim, dtype):
    rng = np.random.default_rng(31 + dim)
    shape = [5, 7, 4]
    src = (rng.standard_normal(shape) * 100).astype(dtype)
    ishape = list(shape)
    ishape[dim] = 9
    idx = rng.integers(0, shape[dim], ishape).astype(np.int64)
    want = np.take_along_axis(src, idx, axis=dim)
    assert np.array_equal(so.gather(src, dim, idx), want)
    assert np.array_equal(torch.gather(torch.from_numpy(src), dim, torch.from_numpy(idx)).numpy(), want)


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_scatter_add_against_torch_and_brute_force(dim):
    rng = np.random.default_rng(41 + dim)
    ishape = [4, 6, 3]
    dshape = list(ishape)
    dshape[dim] = 5  # fewer slots than sources: collisions
    idx = rng.integers(0, dshape[dim], ishape).astype(np.int64)
    src = rng.integers(-8, 9, ishape).astype(np.float32)  # integers: any order gives the same sum
    want = torch.zeros(dshape).scatter_add_(dim, torch.from_numpy(idx), torch.from_numpy(src)).numpy()
    assert np.array_equal(so.scatter_add(src, dim, idx, dshape), want)
    # gather is its adjoint: <scatter_add(src), w> == <src, gather(w)>
    w = rng.standard_normal(dshape).astype(np.float32)
    lhs = float((so.scatter_add(src, dim, idx, dshape).astype(np.float64) * w).sum())
    rhs = float((src.astype(np.float64) * so.gather(w, dim, idx)).sum())
    assert abs(lhs - rhs) < 1e-3


def test_scatter_add_f16_order_and_rounding():
    # one column, many collisions: the f16 running sum depends on the order; brute force in the
    # reference's order (src/storage/cpu.rs:914-934) with numpy half scalars
    rng = np.random.default_rng(5)
    n = 300
    src = (rng.standard_normal((n, 1)) * 50).astype(np.float16)
    idx = rng.integers(0, 3, (n, 1)).astype(np.int64)
    want = np.zeros((3, 1), np.float16)
    for i in range(n):
        want[idx[i, 0], 0] = np.float16(want[idx[i, 0], 0] + src[i, 0])
    assert np.array_equal(so.scatter_add(src, 0, idx, (3, 1)), want)


def test_cat():
    a, b = _rand((2, 3), 1), _rand((4,), 2)
    assert np.array_equal(so.cat([a, b]), np.concatenate([a.ravel(), b]))


def test_cat_reference_literal():
    # tests/tensor.rs:1942-1972: two [2, 2] tensors along dim 0
    lhs, rhs = np.array([1, 2, 3, 4], np.float32).reshape(2, 2), np.array([5, 6, 7, 8], np.float32).reshape(2, 2)
    assert so.cat([lhs, rhs]).tolist() == [1, 2, 3, 4, 5, 6, 7, 8]


# ---- index_select / index_add along any dimension -------------------------------------------

def test_index_select_dim_reference_literals():
    # tests/tensor.rs:2289-2321 (dim 0) and 2323-2357 (dim 2 of [2, 2, 3])
    x = np.array([10, 11, 12, 20, 21, 22, 30, 31, 32, 40, 41, 42], np.float32).reshape(4, 3)
    assert so.index_select_dim(x, 0, [2, 0, 3]).ravel().tolist() == [30, 31, 32, 10, 11, 12, 40, 41, 42]
    y = np.arange(1, 13, dtype=np.float32).reshape(2, 2, 3)
    assert so.index_select_dim(y, 2, [2, 0]).ravel().tolist() == [3, 1, 6, 4, 9, 7, 12, 10]


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_index_select_dim_against_libraries(dim):
    x = _rand((3, 5, 4), 31)
    idx = np.random.default_rng(32).integers(0, x.shape[dim], 7)
    got = so.index_select_dim(x, dim, idx)
    assert np.array_equal(got, np.take(x, idx, axis=dim))
    assert np.array_equal(got, torch.index_select(torch.from_numpy(x), dim, torch.from_numpy(idx)).numpy())
    with pytest.raises(IndexError):
        so.index_select_dim(x, dim, [x.shape[dim]])


def test_index_add_dim_reference_literal():
    # tests/tensor.rs:2359-2385: the gradient of a sum through index_select(0, [2, 0, 2]) of [4, 3]
    got = so.index_add_dim(np.ones((3, 3), np.float32), 0, [2, 0, 2], (4, 3))
    assert got.ravel().tolist() == [1, 1, 1, 0, 0, 0, 2, 2, 2, 0, 0, 0]


@pytest.mark.parametrize("dim", [0, 1, 2])
def test_index_add_dim_against_torch_and_the_adjoint(dim):
    shape = (3, 5, 4)
    idx = np.random.default_rng(41).integers(0, shape[dim], 9)  # with collisions
    src_shape = shape[:dim] + (9,) + shape[dim + 1:]
    src = np.random.default_rng(42).integers(-8, 9, src_shape).astype(np.float32)  # exact sums in any order
    got = so.index_add_dim(src, dim, idx, shape)
    want = torch.zeros(shape).index_add_(dim, torch.from_numpy(idx), torch.from_numpy(src)).numpy()
    assert np.array_equal(got, want)
    # index_add is the adjoint of index_select: <select(x), s> == <x, add(s)>
    x = np.random.default_rng(43).integers(-8, 9, shape).astype(np.float32)
    assert float((so.index_select_dim(x, dim, idx) * src).sum()) == float((x * got).sum())


def test_index_add_dim_f16_order():
    # ascending positions: (2048 + 1) + 1 == 2048 in f16, (1 + 1) + 2048 == 2050
    src = np.array([[2048.0, 1.0, 1.0]], np.float16).reshape(1, 3, 1)
    assert so.index_add_dim(src, 1, [0, 0, 0], (1, 2, 1)).ravel().tolist() == [2048.0, 0.0]
    src = np.array([[1.0, 1.0, 2048.0]], np.float16).reshape(1, 3, 1)
    assert so.index_add_dim(src, 1, [0, 0, 0], (1, 2, 1)).ravel().tolist() == [2050.0, 0.0]
