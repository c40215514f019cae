"""GPU parity of the attention kernel (decode, prefill, chunked prefill; FP16 and INT8 KV;
GQA and MHA) against the CPU oracle and the float64 textbook attention, through the C-ABI.
Shapes follow the reference's own tests (tests/ut/cross_attention_test.cpp:276-296,
attention_kernels_test.cpp:484-540) and the decode sweep of the benchmark configuration."""
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


def _cos(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def _filled(xh, orc, rng, int8, B, H, S, n):
    """Host oracle caches and a device cache holding the same n rows per sequence."""
    kc, vc = orc.KVCache(int8, B, H, S, D), orc.KVCache(int8, B, H, S, D)
    for b in range(B):
        kc.store(b, 0, rng.standard_normal((n, H * D)).astype(np.float32))
        vc.store(b, 0, rng.standard_normal((n, H * D)).astype(np.float32))
    dc = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, H, S, D)
    dc.load(0, kc.data, kc.scales)
    dc.load(1, vc.data, vc.scales)
    return kc, vc, dc


def _attend(xh, orc, dc, q, B, S, qh, past, out_dtype=None):
    out_dtype = xh.F32 if out_dtype is None else out_dtype
    qd = xh.DeviceBuffer.from_numpy(orc.to_bf16(q))
    od = xh.DeviceBuffer(q.size * 4)
    od.zero()
    xh.attention(dc, qd.ptr, q.shape[1], od.ptr, q.shape[1], out_dtype, B, S, qh, SCALE, past)
    xh.synchronize()
    if out_dtype == xh.F32:
        return od.to_numpy(np.float32, q.shape)
    return orc.from_bf16(od.to_numpy(np.uint16, q.shape))


@pytest.mark.parametrize("int8", [0, 1])
@pytest.mark.parametrize("qh,kvh", [(32, 8), (32, 32), (8, 1)])
@pytest.mark.parametrize("present", [1, 31, 32, 33, 100, 1000])
def test_decode_vs_textbook(xh, orc, int8, qh, kvh, present):
    print(f"case int8={int8} qh={qh} kvh={kvh} present={present}", flush=True)
    rng = np.random.default_rng(present * 7 + qh + int8)
    B = 2
    kc, vc, dc = _filled(xh, orc, rng, int8, B, kvh, 1024, present)
    q = orc.round_bf16(rng.standard_normal((B, qh * D)))
    got = _attend(xh, orc, dc, q, B, 1, qh, present - 1)
    ref = orc.attention_ref_f64(q, kc.as_f32(), vc.as_f32(), qh, kvh, D, [1] * B, [present - 1] * B, SCALE)
    # reference tests use 1e-3 / 3e-3 here (cross_attention_test.cpp:108-113)
    assert np.abs(got - ref).max() < 3e-3, np.abs(got - ref).max()
    assert _cos(got, ref) >= 0.9999
    # the oracle's restatement of the sharded-head kernel agrees too
    sh = orc.cross_attn_sharded_head(q, present, qh, kvh, D, SCALE, 2, kc, vc) if present >= 2 else ref
    assert np.abs(got - sh).max() < 3e-3


@pytest.mark.parametrize("int8", [0, 1])
@pytest.mark.parametrize("B,ctx", [(1, 1024), (16, 4096), (4, 16384)])
def test_decode_sweep_shapes(xh, orc, int8, B, ctx):
    print(f"case int8={int8} B={B} ctx={ctx}", flush=True)
    rng = np.random.default_rng(ctx + B)
    qh, kvh = 32, 8
    kc, vc, dc = _filled(xh, orc, rng, int8, B, kvh, ctx, ctx)
    q = orc.round_bf16(rng.standard_normal((B, qh * D)))
    got = _attend(xh, orc, dc, q, B, 1, qh, ctx - 1)
    ref = orc.attention_ref_f64(q, kc.as_f32(), vc.as_f32(), qh, kvh, D, [1] * B, [ctx - 1] * B, SCALE)
    assert np.abs(got - ref).max() < 3e-3
    assert _cos(got, ref) >= 0.9999
    got16 = _attend(xh, orc, dc, q, B, 1, qh, ctx - 1, xh.BF16)
    assert (np.abs(got16 - ref) <= 3e-3 + np.abs(ref) * 2.0 ** -8).all()


@pytest.mark.parametrize("int8", [0, 1])
def test_decode_step_with_store_vs_reference_semantics(xh, orc, int8):
    """One whole decode step: RoPE-free append of the new K/V row then attention, against the
    restatement of crossAttnByHead (which stores, then lets non-leader heads read the
    unrounded new row)."""
    rng = np.random.default_rng(21)
    B, qh, kvh, past, S = 3, 32, 8, 77, 256
    kc, vc, dc = _filled(xh, orc, rng, int8, B, kvh, S, past)
    stride = (qh + 2 * kvh) * D
    qkv = orc.round_bf16(rng.standard_normal((B, stride)))
    dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(qkv))
    xh.rope_kvstore(dc, dev.ptr, xh.BF16, stride, B, 1, qh, None, past)
    od = xh.DeviceBuffer(B * qh * D * 4)
    xh.attention(dc, dev.ptr, stride, od.ptr, qh * D, xh.F32, B, 1, qh, SCALE, past)
    xh.synchronize()
    got = od.to_numpy(np.float32, (B, qh * D))
    exp = orc.cross_attn_by_head(qkv[:, :qh * D].copy(), qkv[:, qh * D:(qh + kvh) * D].copy(),
                                 qkv[:, (qh + kvh) * D:].copy(), qh, kvh, D, [1] * B, [past] * B, SCALE, kc, vc)
    assert np.abs(got - exp).max() < (2e-2 if int8 else 3e-3)
    assert _cos(got, exp) >= 0.9999
    # leaders read exactly what we read
    lead = np.concatenate([np.arange(D) + h * D for h in range(0, qh, qh // kvh)])
    assert np.abs(got[:, lead] - exp[:, lead]).max() < 1e-3


@pytest.mark.parametrize("qh,kvh", [(2, 2), (6, 2), (8, 2), (32, 8)])
@pytest.mark.parametrize("S", [80, 100, 33, 257])
def test_prefill_vs_textbook(xh, orc, qh, kvh, S):
    print(f"case qh={qh} kvh={kvh} S={S}", flush=True)
    rng = np.random.default_rng(S + qh)
    B = 2
    stride = (qh + 2 * kvh) * D
    qkv = orc.round_bf16(rng.standard_normal((B * S, stride)))
    dc = xh.KVCache(xh.FP16, B, kvh, 300, D)
    dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(qkv))
    xh.rope_kvstore(dc, dev.ptr, xh.BF16, stride, B, S, qh, None, 0)
    od = xh.DeviceBuffer(B * S * qh * D * 4)
    xh.attention(dc, dev.ptr, stride, od.ptr, qh * D, xh.F32, B, S, qh, SCALE, 0)
    xh.synchronize()
    got = od.to_numpy(np.float32, (B * S, qh * D))
    q = qkv[:, :qh * D].copy()
    K4 = orc.from_fp16(orc.to_fp16(qkv[:, qh * D:(qh + kvh) * D])).reshape(B, S, kvh, D).transpose(0, 2, 1, 3).copy()
    V4 = orc.from_fp16(orc.to_fp16(qkv[:, (qh + kvh) * D:])).reshape(B, S, kvh, D).transpose(0, 2, 1, 3).copy()
    ref = orc.attention_ref_f64(q, K4, V4, qh, kvh, D, [S] * B, [0] * B, SCALE)
    assert np.abs(got - ref).max() < 3e-3
    # and within the reference test's 1e-2 of its flash-style path (bf16 K/V, bf16 probabilities)
    fl = orc.flash_prefill(q, orc.to_bf16(qkv[:, qh * D:(qh + kvh) * D]), orc.to_bf16(qkv[:, (qh + kvh) * D:]), qh,
                           kvh, D, [S] * B, [0] * B, SCALE)
    assert np.abs(got - fl).max() < 1e-2


@pytest.mark.parametrize("int8", [0, 1])
def test_chunked_prefill_over_cache(xh, orc, int8):
    rng = np.random.default_rng(31)
    B, qh, kvh, past, S = 2, 32, 8, 200, 48
    kc, vc, dc = _filled(xh, orc, rng, int8, B, kvh, 256, past)
    stride = (qh + 2 * kvh) * D
    qkv = orc.round_bf16(rng.standard_normal((B * S, stride)))
    dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(qkv))
    xh.rope_kvstore(dc, dev.ptr, xh.BF16, stride, B, S, qh, None, past)
    od = xh.DeviceBuffer(B * S * qh * D * 4)
    xh.attention(dc, dev.ptr, stride, od.ptr, qh * D, xh.F32, B, S, qh, SCALE, past)
    xh.synchronize()
    got = od.to_numpy(np.float32, (B * S, qh * D))
    exp = orc.cross_attn_by_head(qkv[:, :qh * D].copy(), qkv[:, qh * D:(qh + kvh) * D].copy(),
                                 qkv[:, (qh + kvh) * D:].copy(), qh, kvh, D, [S] * B, [past] * B, SCALE, kc, vc)
    assert np.abs(got - exp).max() < (2e-2 if int8 else 3e-3)
    assert _cos(got, exp) >= 0.9999


@pytest.mark.parametrize("int8", [0, 1])
def test_short_chunk_over_a_long_cache(xh, orc, int8):
    """Three new tokens per sequence over 3000 cached ones, one sequence, 8 KV heads: 12 columns in one column group,
    the sequence cut into 24 parts whose merge is a launch of its own over those 12 columns."""
    rng = np.random.default_rng(35)
    B, qh, kvh, past, S = 1, 32, 8, 3000, 3
    kc, vc, dc = _filled(xh, orc, rng, int8, B, kvh, 3072, past)
    stride = (qh + 2 * kvh) * D
    qkv = orc.round_bf16(rng.standard_normal((B * S, stride)))
    dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(qkv))
    xh.rope_kvstore(dc, dev.ptr, xh.BF16, stride, B, S, qh, None, past)
    od = xh.DeviceBuffer(B * S * qh * D * 4)
    xh.attention(dc, dev.ptr, stride, od.ptr, qh * D, xh.F32, B, S, qh, SCALE, past)
    xh.synchronize()
    got = od.to_numpy(np.float32, (B * S, qh * D))
    exp = orc.cross_attn_by_head(qkv[:, :qh * D].copy(), qkv[:, qh * D:(qh + kvh) * D].copy(),
                                 qkv[:, (qh + kvh) * D:].copy(), qh, kvh, D, [S] * B, [past] * B, SCALE, kc, vc)
    assert np.abs(got - exp).max() < (2e-2 if int8 else 3e-3)
    assert _cos(got, exp) >= 0.9999


@pytest.mark.parametrize("n,S", [(900, 1024), (4000, 4096)])
def test_split_count_independence(xh, orc, n, S):
    """The same query against the same rows gives the same answer whether the sequence is left whole (a large batch:
    one workgroup per sequence and KV head) or split: 8 parts merged by the last workgroup to finish at 900 tokens,
    32 parts merged by a launch of their own at 4000."""
    rng = np.random.default_rng(41)
    qh, kvh = 32, 8
    rows_k = rng.standard_normal((n, kvh * D)).astype(np.float32)
    rows_v = rng.standard_normal((n, kvh * D)).astype(np.float32)
    q = orc.round_bf16(rng.standard_normal((1, qh * D)))
    outs = []
    for B in (1, 40):  # 320 (sequence, KV head) pairs: more than the device has CUs, nothing is split
        kc, vc = orc.KVCache(0, 1, kvh, S, D), orc.KVCache(0, 1, kvh, S, D)
        kc.store(0, 0, rows_k)
        vc.store(0, 0, rows_v)
        dc = xh.KVCache(xh.FP16, B, kvh, S, D)
        dc.load(0, np.repeat(kc.data, B, 0))
        dc.load(1, np.repeat(vc.data, B, 0))
        outs.append(_attend(xh, orc, dc, np.repeat(q, B, 0), B, 1, qh, n - 1)[0])
        dc.free()
    # probabilities are narrowed to fp16 relative to a different running max per split
    assert np.abs(outs[0] - outs[1]).max() < 1e-4


def test_two_streams_each_merge_their_splits_in_their_own_workspace(xh, orc):
    """Split launches on two streams, queued alternately without a wait in between, over different caches and
    queries: each stream's results equal what the same call gives alone (the partial results and tickets of plain
    calls belong to the stream they are made on)."""
    rng = np.random.default_rng(77)
    qh, kvh, n = 32, 8, 3000  # batch 1: 24 parts, merged by a launch of their own
    cases = []
    for i in range(2):
        kc, vc, dc = _filled(xh, orc, rng, 0, 1, kvh, 3072, n)
        q = orc.round_bf16(rng.standard_normal((1, qh * D)))
        alone = _attend(xh, orc, dc, q, 1, 1, qh, n - 1)
        cases.append((dc, xh.DeviceBuffer.from_numpy(orc.to_bf16(q)), xh.DeviceBuffer(q.size * 4), alone, q.shape))
    streams = [xh.Stream(), xh.Stream()]
    for rep in range(20):
        for (dc, qd, od, _, shape), st in zip(cases, streams):
            xh.attention(dc, qd.ptr, shape[1], od.ptr, shape[1], xh.F32, 1, 1, qh, SCALE, n - 1, None, st.h)
    for st in streams:
        st.synchronize()
    for dc, qd, od, alone, shape in cases:
        assert np.array_equal(od.to_numpy(np.float32, shape), alone)
    for st in streams:
        st.free()


def test_past_from_device_memory(xh, orc):
    rng = np.random.default_rng(51)
    B, qh, kvh = 3, 32, 8
    kc, vc, dc = _filled(xh, orc, rng, 0, B, kvh, 512, 400)
    q = orc.round_bf16(rng.standard_normal((B, qh * D)))
    pasts = np.array([399, 17, 250], np.int32)
    pd = xh.DeviceBuffer.from_numpy(pasts)
    qd = xh.DeviceBuffer.from_numpy(orc.to_bf16(q))
    od = xh.DeviceBuffer(q.size * 4)
    xh.attention(dc, qd.ptr, qh * D, od.ptr, qh * D, xh.F32, B, 1, qh, SCALE, 0, pd.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, q.shape)
    ref = orc.attention_ref_f64(q, kc.as_f32(), vc.as_f32(), qh, kvh, D, [1] * B, list(pasts), SCALE)
    assert np.abs(got - ref).max() < 3e-3
