"""Device memory calls of the C ABI: the block cache behind alloc / free."""
import ctypes

import numpy as np
import pytest

from deers_amd import rocm


@pytest.fixture(scope="module", autouse=True)
def _init():
    if not rocm.available():
        pytest.skip("no gfx950 device")
    rocm.init(0)


def _alloc(nbytes, zeros=False):
    p = ctypes.c_void_p()
    fn = rocm.load().deers_rocm_alloc_zeros if zeros else rocm.load().deers_rocm_alloc
    rocm._check(fn(ctypes.c_size_t(nbytes), ctypes.byref(p)))
    return p


def _free(p):
    rocm._check(rocm.load().deers_rocm_free(p))


@pytest.mark.gpu
def test_freed_blocks_are_reused_by_size_and_in_stream_order():
    rocm.sync()
    rocm.empty_cache()
    a = _alloc(1000)           # rounds to 1024
    _free(a)
    b = _alloc(1024)           # same size class: the cached block comes back
    assert b.value == a.value
    c = _alloc(1024)           # a second one must be a different block
    assert c.value != b.value
    d = _alloc(4096)
    assert d.value not in (b.value, c.value)
    # work enqueued before a free still sees its data: fill, free, reallocate, read back
    # through a copy that was enqueued before the free
    n = 1 << 20
    src = rocm.DeviceBuffer((n,), np.float32)
    rocm.fill_raw(np.float32, src.ptr, n, 3.5)
    dst = rocm.DeviceBuffer((n,), np.float32)
    rocm._check(rocm.load().deers_rocm_dtod(dst.ptr, src.ptr, ctypes.c_size_t(4 * n)))
    held = src.ptr.value
    src.free()                                  # returns at once
    again = rocm.DeviceBuffer((n,), np.float32)  # the same block, refilled after the copy in stream order
    assert again.ptr.value == held
    rocm.fill_raw(np.float32, again.ptr, n, -1.0)
    assert (dst.numpy() == 3.5).all() and (again.numpy() == -1.0).all()
    for p in (b, c, d):
        _free(p)


@pytest.mark.gpu
def test_alloc_zeros_of_a_recycled_block_is_zero():
    p = _alloc(1 << 16)
    rocm.fill_raw(np.float32, p, 1 << 14, 9.0)
    _free(p)
    q = _alloc(1 << 16, zeros=True)
    assert q.value == p.value
    out = np.empty(1 << 14, np.float32)
    rocm._check(rocm.load().deers_rocm_dtoh(out.ctypes.data_as(ctypes.c_void_p), q, ctypes.c_size_t(1 << 16)))
    assert (out == 0).all()
    _free(q)


@pytest.mark.gpu
def test_free_rejects_what_it_did_not_hand_out():
    p = _alloc(512)
    _free(p)
    with pytest.raises(rocm.RocmError, match="not allocated"):
        _free(p)                                    # twice
    q = _alloc(2048)
    with pytest.raises(rocm.RocmError, match="not allocated"):
        _free(ctypes.c_void_p(q.value + 256))       # an interior pointer
    _free(q)
    _free(ctypes.c_void_p())                        # NULL is a no-op
    z = ctypes.c_void_p(1)
    rocm._check(rocm.load().deers_rocm_alloc(ctypes.c_size_t(0), ctypes.byref(z)))
    assert not z.value                              # zero bytes: NULL


@pytest.mark.gpu
def test_empty_cache_returns_blocks_to_the_driver():
    ps = [_alloc(1 << 20) for _ in range(4)]
    for p in ps:
        _free(p)
    rocm.empty_cache()
    rocm.empty_cache()  # idempotent
    p = _alloc(1 << 20)
    _free(p)
