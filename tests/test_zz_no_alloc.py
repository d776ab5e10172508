"""deers_rocm_attn_decode_noalloc against deers_rocm_attn_decode, through the C ABI.

The no-allocation entry point runs the decode kernels with the split partial results in a
static device array instead of the library's growing workspace.  Same kernels, same
arithmetic order: outputs must be bit-identical.  Two calls in a row, the second on a
smaller problem, show that what the first call left in the shared array does not leak into
the second; the oracle bounds both at the f16 tolerance of the path (5e-3 max abs).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL_F16 = 5e-3


def _decode_both(x, B, H, L, D, Lcap):
    from deers_amd import rocm
    scale = rocm.default_scale(D)
    bq = rocm.DeviceBuffer.from_numpy(x["q"][:, :, 0])
    bk = rocm.DeviceBuffer.from_numpy(x["k"])
    bv = rocm.DeviceBuffer.from_numpy(x["v"])
    strides = (H * Lcap * D, Lcap * D, D)
    # poison both outputs so that an entry point that wrote nothing cannot pass
    o_ref = rocm.DeviceBuffer.from_numpy(np.full((B, H, D), np.nan, np.float16))
    o_new = rocm.DeviceBuffer.from_numpy(np.full((B, H, D), np.nan, np.float16))
    rocm.attn_decode_raw(np.float16, bq.ptr, bk.ptr, bv.ptr, o_ref.ptr, B, H, L, D, scale,
                         kv_strides=strides)
    rocm.attn_decode_noalloc_raw(np.float16, bq.ptr, bk.ptr, bv.ptr, o_new.ptr, B, H, L, D, scale,
                                 kv_strides=strides)
    return o_ref.numpy(), o_new.numpy()


def test_noalloc_decode_matches_decode_on_two_calls_in_a_row():
    import oracle
    from deers_amd import rocm, synth
    if not rocm.available():
        pytest.fail("no gfx950 device")
    rocm.init(0)
    # (B, H, L, D): few heads, long caches => every head is split over several workgroups,
    # the case that uses the scratch array; the second call is smaller in every dimension
    for name, (B, H, L, D) in (("noalloc-a", (2, 3, 4096, 64)), ("noalloc-b", (1, 2, 1500, 32))):
        x = synth.attention_inputs(name, B, H, 1, D, np.float16, base_seed=7, kv_len=L,
                                   names=("q", "k", "v"))
        print(f"case {name} B={B} H={H} L={L} D={D}", flush=True)
        o_ref, o_new = _decode_both(x, B, H, L, D, L)
        assert np.isfinite(o_new.astype(np.float32)).all()
        assert np.array_equal(o_ref.view(np.uint16), o_new.view(np.uint16))
        want = oracle.attn_fwd(x["q"], x["k"], x["v"])[:, :, 0]
        err = float(np.max(np.abs(o_new.astype(np.float64) - want)))
        assert err <= TOL_F16, f"{name}: max abs err {err:.3e}"


def test_noalloc_decode_unsplit_heads_and_bad_arguments():
    from deers_amd import rocm, synth
    rocm.init(0)
    # enough heads that none is split: the scratch array is not touched at all
    B, H, L, D = 32, 12, 300, 64
    x = synth.attention_inputs("noalloc-c", B, H, 1, D, np.float16, base_seed=7, kv_len=L,
                               names=("q", "k", "v"))
    o_ref, o_new = _decode_both(x, B, H, L, D, L)
    assert np.array_equal(o_ref.view(np.uint16), o_new.view(np.uint16))
    # bad arguments are reported the same way as by the allocating entry point
    with pytest.raises(rocm.RocmError):
        rocm.attn_decode_noalloc_raw(np.float16, None, None, None, None, 1, 1, 16, 64, 0.125)
    with pytest.raises(rocm.RocmError):
        q = rocm.DeviceBuffer((1, 1, 48), np.float16)
        rocm.attn_decode_noalloc_raw(np.float16, q.ptr, q.ptr, q.ptr, q.ptr, 1, 1, 1, 48, 0.125)
