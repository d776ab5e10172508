"""Hand-overs between workgroups: the selection rule (no device needed), the stream-ordered
forms against the single-launch ones, and the report of a wait that ran out.

The f16 backward publishes row statistics from one half of its grid to the other through
flags in one XCD's L2, and the few-rows GEMM sums K splits by last arrival the same way.
Both assume workgroup id % 8 == XCD; deers_rocm_init verifies the device facts that stand
behind that and otherwise takes two launches / an unsplit K.  A backend failure surfaces as an
error value in the reference (src/error.rs:40-41, capability checks at
src/storage/cuda.rs:492-528); here a wait that gives up is reported by the next
synchronising call."""
import numpy as np
import pytest

import oracle
from deers_amd import rocm, synth


def test_policy_takes_same_xcd_handover_only_on_a_whole_unmasked_mi355x():
    assert rocm.handover_policy(256, False) == rocm.HANDOVER_SAME_XCD
    assert rocm.handover_policy(256, True) == rocm.HANDOVER_STREAM_ORDER     # CU mask set
    for cus in (32, 64, 128, 228, 255, 257, 304, 0):                         # partitions, other parts
        assert rocm.handover_policy(cus, False) == rocm.HANDOVER_STREAM_ORDER
        assert rocm.handover_policy(cus, True) == rocm.HANDOVER_STREAM_ORDER


def test_mode_is_unknown_before_init():
    if rocm._inited:
        pytest.skip("runtime already initialised in this process")
    assert rocm.handover_mode() == -1


@pytest.fixture
def gpu():
    if not rocm.available():
        pytest.fail("no gfx950 device")
    rocm.init(0)
    yield
    rocm.debug_bwd_wait(1 << 20, False)
    rocm.set_handover_mode(-1)


@pytest.mark.gpu
def test_device_policy_matches_the_device(gpu):
    # the boxes these tests run on are whole MI355X: 256 CUs, no mask
    assert rocm.handover_mode() == rocm.HANDOVER_SAME_XCD


@pytest.mark.gpu
@pytest.mark.parametrize("B,H,T,D", [(2, 3, 300, 64), (1, 2, 129, 32), (1, 2, 257, 128), (3, 5, 1000, 64)])
def test_two_launch_backward_equals_single_launch_bit_for_bit(gpu, B, H, T, D):
    x = synth.attention_inputs(f"handover-{B}-{H}-{T}-{D}", B, H, T, D, np.float16, base_seed=11)
    rocm.set_handover_mode(rocm.HANDOVER_SAME_XCD)
    one = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])
    rocm.set_handover_mode(rocm.HANDOVER_STREAM_ORDER)
    two = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])
    rocm.sync()
    for a, b in zip(one, two):
        np.testing.assert_array_equal(a, b)
    rdq, rdk, rdv = oracle.attn_bwd(x["q"], x["k"], x["v"], x["do"])
    for got, want in zip(two[2:], (rdq, rdk, rdv)):
        assert np.max(np.abs(got.astype(np.float64) - want)) <= 5e-3


@pytest.mark.gpu
def test_more_than_64_query_blocks_per_head(gpu):
    """A dK/dV workgroup polls its flags one per lane: 66 query blocks take a second round of
    the 64-lane poll.  Single launch against two launches bit for bit, and one whole head
    against the oracle."""
    B, H, T, D = 1, 2, 8400, 64
    x = synth.attention_inputs("handover-long", B, H, T, D, np.float16, base_seed=13)
    print(f"case handover-long f16 B={B} H={H} T={T} D={D}", flush=True)
    rocm.set_handover_mode(rocm.HANDOVER_SAME_XCD)
    one = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])
    rocm.set_handover_mode(rocm.HANDOVER_STREAM_ORDER)
    two = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])
    rocm.sync()
    for a, b in zip(one, two):
        np.testing.assert_array_equal(a, b)
    sl = (slice(0, 1), slice(1, 2))
    rdq, rdk, rdv = oracle.attn_bwd(x["q"][sl], x["k"][sl], x["v"][sl], x["do"][sl])
    for name, got, want in zip(("dq", "dk", "dv"), one[2:], (rdq, rdk, rdv)):
        err = np.max(np.abs(got[sl].astype(np.float64) - want))
        assert err <= 5e-3, f"{name}: max abs err {err:.3e}"


@pytest.mark.gpu
def test_unsplit_few_rows_gemm_matches_split_within_rounding(gpu):
    m, n, k = 32, 768, 3072  # the shape whose K is split over workgroups
    rng = np.random.default_rng(5)
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = (rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float16)
    want = x.astype(np.float64) @ w.astype(np.float64)
    dx, dw = rocm.DeviceBuffer.from_numpy(x), rocm.DeviceBuffer.from_numpy(w)
    outs = []
    for mode in (rocm.HANDOVER_SAME_XCD, rocm.HANDOVER_STREAM_ORDER):
        rocm.set_handover_mode(mode)
        dy = rocm.DeviceBuffer.from_numpy(np.full((m, n), np.nan, np.float16))
        rocm.decode_linear_raw(np.float16, "plain", 0.0, dx.ptr, k, dw.ptr, n, dy.ptr, False, m, n, k)
        outs.append(dy.numpy().astype(np.float64))
    for got in outs:
        assert np.max(np.abs(got - want)) <= 5e-3
    # f32 sums in two different fixed orders, one rounding to f16 each
    assert np.max(np.abs(outs[0] - outs[1])) <= 2e-3


@pytest.mark.gpu
def test_a_wait_that_runs_out_is_reported_and_then_cleared(gpu):
    B, H, T, D = 1, 2, 200, 64
    x = synth.attention_inputs("handover-giveup", B, H, T, D, np.float16, base_seed=12)
    good = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])
    rocm.sync()
    # nobody publishes, the consumers poll 4 times and give up: every kernel exits normally
    rocm.set_handover_mode(rocm.HANDOVER_SAME_XCD)
    rocm.debug_bwd_wait(4, True)
    bufs = [rocm.DeviceBuffer.from_numpy(x[n]) for n in ("q", "k", "v", "do")]
    o = rocm.DeviceBuffer.from_numpy(good[0])
    lse = rocm.DeviceBuffer.from_numpy(good[1])
    grads = [rocm.DeviceBuffer((B, H, T, D), np.float16) for _ in range(3)]
    rocm.attn_bwd_raw(np.float16, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, o.ptr, lse.ptr, bufs[3].ptr,
                      grads[0].ptr, grads[1].ptr, grads[2].ptr, B, H, T, D, rocm.default_scale(D))
    with pytest.raises(rocm.RocmError, match="error 6"):
        rocm.sync()
    rocm.sync()  # reported once
    # normal operation again: same results as before, no error
    rocm.debug_bwd_wait(1 << 20, False)
    again = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])
    rocm.sync()
    for a, b in zip(good, again):
        np.testing.assert_array_equal(a, b)


@pytest.mark.gpu
def test_captured_backward_replays_correctly(gpu):
    """A replayed graph cannot be given a fresh hand-over epoch, so a backward that is being
    captured takes the two-launch form without the flags.  The captured backward is replayed
    three times, with eager backwards of another geometry and synchronisations between the
    replays, and every replay must give the eager result bit for bit."""
    import ctypes

    hip = ctypes.CDLL("libamdhip64.so")
    B, H, T, D = 2, 3, 300, 64
    x = synth.attention_inputs("handover-graph", B, H, T, D, np.float16, base_seed=14)
    y = synth.attention_inputs("handover-graph-other", 1, 2, 129, 32, np.float16, base_seed=15)
    rocm.set_handover_mode(rocm.HANDOVER_SAME_XCD)
    want = rocm.attn_fwd_bwd(x["q"], x["k"], x["v"], x["do"])  # also grows the workspace and the flags
    rocm.sync()
    bufs = [rocm.DeviceBuffer.from_numpy(x[n]) for n in ("q", "k", "v", "do")]
    o, lse = rocm.DeviceBuffer.from_numpy(want[0]), rocm.DeviceBuffer.from_numpy(want[1])
    grads = [rocm.DeviceBuffer((B, H, T, D), np.float16) for _ in range(3)]
    stream = ctypes.c_void_p(rocm.load().deers_rocm_stream())
    graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p()
    assert hip.hipStreamBeginCapture(stream, 2) == 0  # hipStreamCaptureModeRelaxed
    try:
        rocm.attn_bwd_raw(np.float16, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, o.ptr, lse.ptr, bufs[3].ptr,
                          grads[0].ptr, grads[1].ptr, grads[2].ptr, B, H, T, D, rocm.default_scale(D))
    finally:
        assert hip.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
    assert hip.hipGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, ctypes.c_size_t(0)) == 0
    nan = np.full((B, H, T, D), np.nan, np.float16)
    try:
        for replay in range(3):
            for gbuf in grads:  # poison the outputs
                rocm.load().deers_rocm_htod(gbuf.ptr, nan.ctypes.data_as(ctypes.c_void_p),
                                            ctypes.c_size_t(gbuf.nbytes))
            assert hip.hipGraphLaunch(graph_exec, stream) == 0
            rocm.sync()
            for name, gbuf, ref in zip(("dq", "dk", "dv"), grads, want[2:]):
                np.testing.assert_array_equal(gbuf.numpy(), ref, err_msg=f"replay {replay}: {name}")
            # eager work between the replays: other geometry, other flags, epochs move on
            rocm.attn_fwd_bwd(y["q"], y["k"], y["v"], y["do"])
            rocm.sync()
    finally:
        hip.hipGraphExecDestroy(graph_exec)
        hip.hipGraphDestroy(graph)
