"""RoPE fused with the head split / merge (deers_rocm_rope_fwd / _bwd) against the numpy
restatement of apply_rotary_emb + permute (src/models/gpt.rs:49-73, 135-137)."""
import numpy as np
import pytest

import oracle
from deers_amd import rocm, synth

TOL = {np.dtype(np.float16): 5e-3, np.dtype(np.float32): 1e-4}

SHAPES = [(1, 1, 1, 32), (2, 5, 3, 32), (2, 33, 3, 64), (1, 130, 2, 128), (8, 1024, 12, 64),
          (2, 3, 2, 2), (1, 7, 3, 6), (2, 9, 2, 24), (1, 4, 2, 40)]  # the last four: one pair per thread


@pytest.fixture(scope="module", autouse=True)
def _init():
    if not rocm.available():
        pytest.skip("no gfx950 device")
    rocm.init(0)


def _inputs(B, T, H, D, dtype, seed):
    x = synth.normal((B, T, H, D), synth.tensor_seed(seed, "rope", "x"), 1.0).astype(dtype)
    dy = synth.normal((B, H, T, D), synth.tensor_seed(seed, "rope", "dy"), 1.0).astype(dtype)
    cos, sin = oracle.rope_tables(T, D, dtype=dtype)
    return x, dy, cos, sin


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("B,T,H,D", SHAPES)
def test_rope_fwd_bwd_match_oracle(dtype, B, T, H, D):
    x, dy, cos, sin = _inputs(B, T, H, D, dtype, 21)
    dx_, dc, ds = (rocm.DeviceBuffer.from_numpy(a) for a in (x, cos, sin))
    y = rocm.DeviceBuffer((B, H, T, D), dtype)
    rocm.rope_fwd_raw(dtype, dx_.ptr, dc.ptr, ds.ptr, y.ptr, B, T, H, D)
    want = oracle.rope_apply(x.astype(np.float32), cos.astype(np.float32),
                             sin.astype(np.float32)).transpose(0, 2, 1, 3)
    assert np.max(np.abs(y.numpy().astype(np.float64) - want)) <= TOL[np.dtype(dtype)]
    # position 0 passes through bit-exactly (cos = 1, sin = 0)
    assert np.array_equal(y.numpy()[:, :, 0], x.transpose(0, 2, 1, 3)[:, :, 0])

    ddy = rocm.DeviceBuffer.from_numpy(dy)
    gx = rocm.DeviceBuffer((B, T, H, D), dtype)
    rocm.rope_bwd_raw(dtype, ddy.ptr, dc.ptr, ds.ptr, gx.ptr, B, T, H, D)
    want_dx = oracle.rope_apply_bwd(dy.astype(np.float32).transpose(0, 2, 1, 3),
                                    cos.astype(np.float32), sin.astype(np.float32))
    assert np.max(np.abs(gx.numpy().astype(np.float64) - want_dx)) <= TOL[np.dtype(dtype)]


@pytest.mark.gpu
def test_rope_round_trip_and_norms_at_full_size():
    # size-independent properties at the C2 geometry: forward then backward is the identity
    # up to two f16 roundings, and every (x1_i, x2_i) pair keeps its norm
    B, T, H, D = 8, 1024, 12, 64
    x, _, cos, sin = _inputs(B, T, H, D, np.float16, 22)
    dx_, dc, ds = (rocm.DeviceBuffer.from_numpy(a) for a in (x, cos, sin))
    y = rocm.DeviceBuffer((B, H, T, D), np.float16)
    back = rocm.DeviceBuffer((B, T, H, D), np.float16)
    rocm.rope_fwd_raw(np.float16, dx_.ptr, dc.ptr, ds.ptr, y.ptr, B, T, H, D)
    rocm.rope_bwd_raw(np.float16, y.ptr, dc.ptr, ds.ptr, back.ptr, B, T, H, D)
    assert np.max(np.abs(back.numpy().astype(np.float32) - x.astype(np.float32))) <= 5e-3
    yn = y.numpy().astype(np.float32).transpose(0, 2, 1, 3)
    xf = x.astype(np.float32)
    n_in = xf[..., :32] ** 2 + xf[..., 32:] ** 2
    n_out = yn[..., :32] ** 2 + yn[..., 32:] ** 2
    # f16 rounding of the tables and of the result: a few 2^-11 relative on the squared norm
    assert np.all(np.abs(n_in - n_out) <= 4e-3 * n_in + 1e-3)


@pytest.mark.gpu
def test_rope_strided_views_and_errors():
    B, T, H, D = 2, 9, 3, 64
    x, dy, cos, sin = _inputs(B, T, H, D, np.float16, 23)
    dc, ds = rocm.DeviceBuffer.from_numpy(cos), rocm.DeviceBuffer.from_numpy(sin)
    # x as the q third of a fused [B,T,3,H,D] projection buffer
    qkv = np.zeros((B, T, 3, H, D), np.float16)
    qkv[:, :, 1] = x
    dq = rocm.DeviceBuffer.from_numpy(qkv)
    y = rocm.DeviceBuffer((B, H, T, D), np.float16)
    import ctypes
    off = ctypes.c_void_p(dq.ptr.value + H * D * 2)
    rocm.rope_fwd_raw(np.float16, off, dc.ptr, ds.ptr, y.ptr, B, T, H, D,
                      x_strides=(T * 3 * H * D, 3 * H * D, D, 1))
    ref = rocm.DeviceBuffer((B, H, T, D), np.float16)
    dx_ = rocm.DeviceBuffer.from_numpy(x)
    rocm.rope_fwd_raw(np.float16, dx_.ptr, dc.ptr, ds.ptr, ref.ptr, B, T, H, D)
    assert np.array_equal(y.numpy(), ref.numpy())
    # dy as the [B,T,H,D]-ordered gradient seen through its [B,H,T,D] view
    dy_bthd = np.ascontiguousarray(dy.transpose(0, 2, 1, 3))
    g1 = rocm.DeviceBuffer((B, T, H, D), np.float16)
    g2 = rocm.DeviceBuffer((B, T, H, D), np.float16)
    ddy, ddy_bthd = rocm.DeviceBuffer.from_numpy(dy), rocm.DeviceBuffer.from_numpy(dy_bthd)
    rocm.rope_bwd_raw(np.float16, ddy.ptr, dc.ptr, ds.ptr, g1.ptr, B, T, H, D)
    rocm.rope_bwd_raw(np.float16, ddy_bthd.ptr, dc.ptr, ds.ptr, g2.ptr, B, T, H, D,
                      dy_strides=(T * H * D, D, H * D, 1))
    assert np.array_equal(g1.numpy(), g2.numpy())
    with pytest.raises(rocm.RocmError):  # odd head width
        rocm.rope_fwd_raw(np.float16, dq.ptr, dc.ptr, ds.ptr, y.ptr, B, T, H, 23)
    with pytest.raises(rocm.RocmError):  # innermost stride must be 1
        rocm.rope_fwd_raw(np.float16, dq.ptr, dc.ptr, ds.ptr, y.ptr, B, T, H, D,
                          x_strides=(T * H * D, H * D, D, 2))
    with pytest.raises(rocm.RocmError):
        rocm.rope_fwd_raw(np.float16, None, dc.ptr, ds.ptr, y.ptr, B, T, H, D)


@pytest.mark.gpu
def test_rope_appends_rotated_keys_into_a_cache_and_copy_view_scatters_values():
    """The decode-time use: T_new rotated key rows written at row `pos` of a
    [B,H,L_cap,D] cache through output strides, value rows through copy_view."""
    import ctypes
    B, H, D, cap, pos, tn = 2, 3, 64, 20, 5, 4
    T = pos + tn
    x, _, cos, sin = _inputs(B, T, H, D, np.float16, 24)
    cache0 = synth.normal((B, H, cap, D), synth.tensor_seed(24, "rope", "cache"), 1.0).astype(np.float16)
    dcache = rocm.DeviceBuffer.from_numpy(cache0)
    dx = rocm.DeviceBuffer.from_numpy(np.ascontiguousarray(x[:, pos:]))
    dc, ds = rocm.DeviceBuffer.from_numpy(cos), rocm.DeviceBuffer.from_numpy(sin)
    el = 2
    row = lambda buf, r, width: ctypes.c_void_p(buf.ptr.value + r * width * el)
    rocm.rope_fwd_raw(np.float16, dx.ptr, row(dc, pos, D // 2), row(ds, pos, D // 2),
                      row(dcache, pos, D), B, tn, H, D, y_strides=(H * cap * D, cap * D, D, 1))
    ref = rocm.DeviceBuffer((B, H, T, D), np.float16)
    dfull = rocm.DeviceBuffer.from_numpy(x)
    rocm.rope_fwd_raw(np.float16, dfull.ptr, dc.ptr, ds.ptr, ref.ptr, B, T, H, D)
    got = dcache.numpy()
    assert np.array_equal(got[:, :, pos:pos + tn], ref.numpy()[:, :, pos:])  # same bits as the full pass
    assert np.array_equal(got[:, :, :pos], cache0[:, :, :pos])              # nothing else touched
    assert np.array_equal(got[:, :, pos + tn:], cache0[:, :, pos + tn:])
    # values: [B,tn,H,D] rows scattered to cache rows pos..pos+tn
    v = np.ascontiguousarray(x[:, pos:])
    dv = rocm.DeviceBuffer.from_numpy(v)
    dvc = rocm.DeviceBuffer.from_numpy(cache0)
    rocm.copy_view_raw(np.float16, dv.ptr, (tn * H * D, D, H * D, 1), row(dvc, pos, D),
                       (H * cap * D, cap * D, D, 1), (B, H, tn, D))
    gotv = dvc.numpy()
    assert np.array_equal(gotv[:, :, pos:pos + tn], v.transpose(0, 2, 1, 3))
    assert np.array_equal(gotv[:, :, :pos], cache0[:, :, :pos])
    with pytest.raises(rocm.RocmError):
        rocm.copy_view_raw(np.float16, dv.ptr, (1,) * 7, dvc.ptr, (1,) * 7, (1,) * 7)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("B,H,D", [(2, 3, 64), (32, 12, 64), (1, 5, 32), (3, 2, 128)])
def test_decode_qkv_is_two_ropes_and_a_copy_in_one_launch(dtype, B, H, D):
    """deers_rocm_decode_qkv against the separate entry points it replaces (same bits): q and k
    rotated at `pos` from the thirds of a fused [B, 3C] projection row, k and v written to row
    `pos` of [B,H,cap,D] caches, everything else untouched."""
    import ctypes
    cap, pos, C = 11, 7, H * D
    el = np.dtype(dtype).itemsize
    _, _, cos, sin = _inputs(1, cap, 1, D, dtype, 31)           # tables [cap, D/2]
    qkv = synth.normal((B, 3 * C), synth.tensor_seed(31, "decode", "qkv"), 1.0).astype(dtype)
    kc0 = synth.normal((B, H, cap, D), synth.tensor_seed(31, "decode", "kc"), 1.0).astype(dtype)
    vc0 = synth.normal((B, H, cap, D), synth.tensor_seed(31, "decode", "vc"), 1.0).astype(dtype)
    dqkv, dc, ds = (rocm.DeviceBuffer.from_numpy(a) for a in (qkv, cos, sin))
    at = lambda buf, elems: ctypes.c_void_p(buf.ptr.value + elems * el)
    cos_row, sin_row = at(dc, pos * (D // 2)), at(ds, pos * (D // 2))
    kv_strides = (H * cap * D, cap * D, D)
    # fused
    q1 = rocm.DeviceBuffer((B, H, D), dtype)
    k1, v1 = rocm.DeviceBuffer.from_numpy(kc0), rocm.DeviceBuffer.from_numpy(vc0)
    rocm.decode_qkv_raw(dtype, at(dqkv, 0), at(dqkv, C), at(dqkv, 2 * C), (3 * C, D), cos_row, sin_row,
                        q1.ptr, k1.ptr, v1.ptr, kv_strides, pos, cap, B, H, D)
    # separate
    q2 = rocm.DeviceBuffer((B, H, D), dtype)
    k2, v2 = rocm.DeviceBuffer.from_numpy(kc0), rocm.DeviceBuffer.from_numpy(vc0)
    xs = (3 * C, 3 * C, D, 1)
    rocm.rope_fwd_raw(dtype, at(dqkv, 0), cos_row, sin_row, q2.ptr, B, 1, H, D, x_strides=xs)
    rocm.rope_fwd_raw(dtype, at(dqkv, C), cos_row, sin_row, at(k2, pos * D), B, 1, H, D, x_strides=xs,
                      y_strides=(H * cap * D, cap * D, D, 1))
    rocm.copy_view_raw(dtype, at(dqkv, 2 * C), (3 * C, D, 1), at(v2, pos * D), (H * cap * D, cap * D, 1),
                       (B, H, D))
    assert np.array_equal(q1.numpy(), q2.numpy())
    assert np.array_equal(k1.numpy(), k2.numpy())
    assert np.array_equal(v1.numpy(), v2.numpy())
    # and against the oracle's rotation of the same rows
    want_q = oracle.rope_apply(qkv[:, :C].reshape(B, 1, H, D), cos[pos:pos + 1], sin[pos:pos + 1], dtype=dtype)
    tol = 5e-3 if dtype == np.float16 else 1e-5
    assert np.abs(q1.numpy().astype(np.float32) - want_q.reshape(B, H, D).astype(np.float32)).max() <= tol
    assert np.array_equal(v1.numpy()[:, :, pos], qkv[:, 2 * C:].reshape(B, H, D))
    assert np.array_equal(k1.numpy()[:, :, :pos], kc0[:, :, :pos]) and np.array_equal(k1.numpy()[:, :, pos + 1:], kc0[:, :, pos + 1:])
    with pytest.raises(rocm.RocmError):
        rocm.decode_qkv_raw(dtype, at(dqkv, 0), at(dqkv, C), at(dqkv, 2 * C), (3 * C, D), cos_row, sin_row,
                            q1.ptr, k1.ptr, v1.ptr, kv_strides, cap, cap, B, H, D)   # position past the cache
    with pytest.raises(rocm.RocmError):
        rocm.decode_qkv_raw(dtype, at(dqkv, 1), at(dqkv, C), at(dqkv, 2 * C), (3 * C, D), cos_row, sin_row,
                            q1.ptr, k1.ptr, v1.ptr, kv_strides, pos, cap, B, H, D)   # misaligned q


@pytest.mark.gpu
@pytest.mark.parametrize("B,H,D,cap,pos", [(2, 3, 64, 11, 7), (1, 2, 64, 5, 0), (3, 2, 128, 300, 299),
                                           (32, 12, 64, 700, 650), (1, 1, 64, 2100, 2000),
                                           (4, 6, 32, 40, 17), (1, 1, 32, 2100, 2000)])
def test_attn_decode_append_is_decode_qkv_then_attn_decode(B, H, D, cap, pos):
    """deers_rocm_attn_decode_append against the two launches it replaces: the caches end up
    bit-identical (same rotation arithmetic), the attention output agrees to the rounding of the
    f32 softmax sums (the new row is merged last instead of in stream order) and with the oracle
    on the same rows.  pos = 0 is the empty cache; the last case splits a head over workgroups."""
    import ctypes
    dtype = np.float16
    C = H * D
    _, _, cos, sin = _inputs(1, cap, 1, D, dtype, 37)           # tables [cap, D/2]
    qkv = synth.normal((B, 3 * C), synth.tensor_seed(37 + pos, "append", "qkv"), 1.0).astype(dtype)
    kc0 = synth.normal((B, H, cap, D), synth.tensor_seed(37 + pos, "append", "kc"), 1.0).astype(dtype)
    vc0 = synth.normal((B, H, cap, D), synth.tensor_seed(37 + pos, "append", "vc"), 1.0).astype(dtype)
    dqkv, dc, ds = (rocm.DeviceBuffer.from_numpy(a) for a in (qkv, cos, sin))
    at = lambda buf, elems: ctypes.c_void_p(buf.ptr.value + elems * 2)
    cos_row, sin_row = at(dc, pos * (D // 2)), at(ds, pos * (D // 2))
    kv_strides = (H * cap * D, cap * D, D)
    scale = rocm.default_scale(D)
    # one launch
    k1, v1 = rocm.DeviceBuffer.from_numpy(kc0), rocm.DeviceBuffer.from_numpy(vc0)
    o1 = rocm.DeviceBuffer((B, H, D), dtype)
    rocm.attn_decode_append_raw(dtype, at(dqkv, 0), at(dqkv, C), at(dqkv, 2 * C), (3 * C, D), cos_row, sin_row,
                                k1.ptr, v1.ptr, kv_strides, o1.ptr, pos, cap, B, H, D, scale)
    # two launches
    k2, v2 = rocm.DeviceBuffer.from_numpy(kc0), rocm.DeviceBuffer.from_numpy(vc0)
    q2, o2 = rocm.DeviceBuffer((B, H, D), dtype), rocm.DeviceBuffer((B, H, D), dtype)
    rocm.decode_qkv_raw(dtype, at(dqkv, 0), at(dqkv, C), at(dqkv, 2 * C), (3 * C, D), cos_row, sin_row,
                        q2.ptr, k2.ptr, v2.ptr, kv_strides, pos, cap, B, H, D)
    rocm.attn_decode_raw(dtype, q2.ptr, k2.ptr, v2.ptr, o2.ptr, B, H, pos + 1, D, scale, kv_strides=kv_strides)
    assert np.array_equal(k1.numpy(), k2.numpy())
    assert np.array_equal(v1.numpy(), v2.numpy())
    a, b = o1.numpy().astype(np.float32), o2.numpy().astype(np.float32)
    assert np.abs(a - b).max() <= 2e-3
    # the oracle on the rows the kernel saw
    kk, vv, qq = k2.numpy()[:, :, :pos + 1], v2.numpy()[:, :, :pos + 1], q2.numpy()
    want = oracle.attn_fwd(qq[:, :, None].astype(np.float32), kk.astype(np.float32), vv.astype(np.float32))[:, :, 0]
    assert np.abs(a - want).max() <= 5e-3
    with pytest.raises(rocm.RocmError):
        rocm.attn_decode_append_raw(dtype, at(dqkv, 0), at(dqkv, C), at(dqkv, 2 * C), (3 * C, D), cos_row, sin_row,
                                    k1.ptr, v1.ptr, kv_strides, o1.ptr, cap, cap, B, H, D, scale)
