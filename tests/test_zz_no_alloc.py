"""xfthip_attention_static (split-KV workspace in a statically allocated device array, no
allocation in the call) against xfthip_attention, through the C-ABI: two calls in a row, the
second with a smaller input, then a prefill, an INT8 cache and the rejection of a shape whose
split does not fit the static array."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
D = 128
SCALE = 1.0 / np.sqrt(D)


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init(0)
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def _filled(xh, orc, rng, int8, B, H, S, n):
    kc, vc = orc.KVCache(int8, B, H, S, D), orc.KVCache(int8, B, H, S, D)
    for b in range(B):
        kc.store(b, 0, rng.standard_normal((n, H * D)).astype(np.float32))
        vc.store(b, 0, rng.standard_normal((n, H * D)).astype(np.float32))
    dc = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, H, S, D)
    dc.load(0, kc.data, kc.scales)
    dc.load(1, vc.data, vc.scales)
    return kc, vc, dc


def _both(xh, orc, dc, q, B, S, qh, past):
    qd = xh.DeviceBuffer.from_numpy(orc.to_bf16(q))
    outs = []
    for fn in (xh.attention, xh.attention_static):
        od = xh.DeviceBuffer(q.size * 4)
        od.zero()
        fn(dc, qd.ptr, q.shape[1], od.ptr, q.shape[1], xh.F32, B, S, qh, SCALE, past)
        xh.synchronize()
        outs.append(od.to_numpy(np.float32, q.shape))
    return outs


@pytest.mark.parametrize("int8", [0, 1])
def test_static_scratch_attention_two_calls_in_a_row(xh, orc, int8):
    rng = np.random.default_rng(71 + int8)
    qh, kvh = 32, 8
    # first call: 4 sequences at context 1000 (the KV sequence is split over several workgroups)
    kc, vc, dc = _filled(xh, orc, rng, int8, 4, kvh, 1024, 1000)
    q = orc.round_bf16(rng.standard_normal((4, qh * D)))
    plain, static = _both(xh, orc, dc, q, 4, 1, qh, 999)
    ref = orc.attention_ref_f64(q, kc.as_f32(), vc.as_f32(), qh, kvh, D, [1] * 4, [999] * 4, SCALE)
    assert np.array_equal(plain, static)
    assert np.abs(static - ref).max() < 3e-3
    # second call, smaller: one sequence at context 300, over what the first call left in the array
    q2 = orc.round_bf16(rng.standard_normal((1, qh * D)))
    plain2, static2 = _both(xh, orc, dc, q2, 1, 1, qh, 299)
    ref2 = orc.attention_ref_f64(q2, kc.as_f32()[:1], vc.as_f32()[:1], qh, kvh, D, [1], [299], SCALE)
    assert np.array_equal(plain2, static2)
    assert np.abs(static2 - ref2).max() < 3e-3
    # and the first shape again
    plain3, static3 = _both(xh, orc, dc, q, 4, 1, qh, 999)
    assert np.array_equal(static3, static) and np.array_equal(plain3, plain)


def test_static_scratch_attention_prefill_and_widest_split(xh, orc):
    rng = np.random.default_rng(73)
    qh, kvh, B, S = 8, 2, 2, 100
    stride = (qh + 2 * kvh) * D
    qkv = orc.round_bf16(rng.standard_normal((B * S, stride)))
    dc = xh.KVCache(xh.FP16, B, kvh, 128, D)
    dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(qkv))
    xh.rope_kvstore(dc, dev.ptr, xh.BF16, stride, B, S, qh, None, 0)
    outs = []
    for fn in (xh.attention, xh.attention_static):
        od = xh.DeviceBuffer(B * S * qh * D * 4)
        fn(dc, dev.ptr, stride, od.ptr, qh * D, xh.F32, B, S, qh, SCALE, 0)
        xh.synchronize()
        outs.append(od.to_numpy(np.float32, (B * S, qh * D)))
    assert np.array_equal(outs[0], outs[1])
    # the widest split the library makes: 16 sequences x 8 KV heads = 128 column groups in 4 parts at 2048 tokens or
    # more = 512 of the array's 1024 slots (with as many column groups as CUs or more, nothing is split at all)
    big = xh.KVCache(xh.FP16, 16, 8, 2304, D)
    for which in (0, 1):
        big.load(which, orc.to_fp16(rng.standard_normal((16, 8, 2304, D), dtype=np.float32)))
    qd = xh.DeviceBuffer.from_numpy(orc.to_bf16(orc.round_bf16(rng.standard_normal((16, 32 * D)))))
    wide = []
    for fn in (xh.attention, xh.attention_static):
        od = xh.DeviceBuffer(16 * 32 * D * 4)
        fn(big, qd.ptr, 32 * D, od.ptr, 32 * D, xh.F32, 16, 1, 32, SCALE, 2200)
        xh.synchronize()
        wide.append(od.to_numpy(np.float32, (16, 32 * D)))
    assert np.array_equal(wide[0], wide[1])


def test_static_scratch_attention_records_into_a_graph(xh, orc):
    """The property the entry point exists for: nothing in the call allocates.  A device allocation (or any
    other synchronising call) while a stream is being captured makes the capture fail, so a split shape is
    recorded into a graph and the graph replayed three times, with eager work between the replays, against
    the eager result."""
    rng = np.random.default_rng(79)
    qh, kvh, B, ctx = 32, 8, 2, 900
    kc, vc, dc = _filled(xh, orc, rng, 0, B, kvh, 1024, ctx)
    q = orc.round_bf16(rng.standard_normal((B, qh * D)))
    qd = xh.DeviceBuffer.from_numpy(orc.to_bf16(q))
    eager = xh.DeviceBuffer(q.size * 4)
    xh.attention_static(dc, qd.ptr, qh * D, eager.ptr, qh * D, xh.F32, B, 1, qh, SCALE, ctx - 1)
    xh.synchronize()
    want = eager.to_numpy(np.float32, q.shape)
    ref = orc.attention_ref_f64(q, kc.as_f32(), vc.as_f32(), qh, kvh, D, [1] * B, [ctx - 1] * B, SCALE)
    assert np.abs(want - ref).max() < 3e-3
    st = xh.Stream()
    od = xh.DeviceBuffer(q.size * 4)
    with xh.Graph(st) as g:
        xh.attention_static(dc, qd.ptr, qh * D, od.ptr, qh * D, xh.F32, B, 1, qh, SCALE, ctx - 1, stream=st.h)
    for replay in range(3):
        od.zero()
        xh.synchronize()
        g.launch()
        st.synchronize()
        assert np.array_equal(od.to_numpy(np.float32, q.shape), want), replay
        # eager work of the same kind between the replays (shares the scratch array, one call at a time)
        xh.attention_static(dc, qd.ptr, qh * D, eager.ptr, qh * D, xh.F32, B, 1, qh, SCALE, ctx - 1)
        xh.synchronize()
    g.free()
