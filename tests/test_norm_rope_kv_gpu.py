"""GPU parity of RMSNorm, RoPE and the KV-cache append (FP16 convert / INT8 quantise) against
the CPU oracle, through the C-ABI.  Integer and conversion results must match bit for bit."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init(0)
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


@pytest.mark.parametrize("rows,cols", [(1, 4096), (7, 4096), (3, 100), (128, 4096), (2, 11008)])
def test_rmsnorm(xh, orc, rows, cols):
    rng = np.random.default_rng(rows * 1000 + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    exp = orc.rmsnorm(x, w, 1e-6)
    xd, wd = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(w)
    od = xh.DeviceBuffer(rows * cols * 4)
    xh.rmsnorm(od.ptr, xh.F32, xd.ptr, xh.F32, wd.ptr, rows, cols)
    xh.synchronize()
    got = od.to_numpy(np.float32, (rows, cols))
    assert np.abs(got - exp).max() <= 4e-6 * np.abs(exp).max()
    # bf16 output: the fp32 result narrowed round-to-nearest-even
    xh.rmsnorm(od.ptr, xh.BF16, xd.ptr, xh.F32, wd.ptr, rows, cols)
    xh.synchronize()
    got16 = od.to_numpy(np.uint16, (rows, cols))
    assert np.abs(orc.from_bf16(got16) - exp).max() <= 2.0 ** -8 * np.abs(exp).max()
    # bf16 input
    xb = orc.to_bf16(x)
    xbd = xh.DeviceBuffer.from_numpy(xb)
    xh.rmsnorm(od.ptr, xh.F32, xbd.ptr, xh.BF16, wd.ptr, rows, cols)
    xh.synchronize()
    exp_b = orc.rmsnorm(orc.from_bf16(xb), w, 1e-6)
    assert np.abs(od.to_numpy(np.float32, (rows, cols)) - exp_b).max() <= 4e-6 * np.abs(exp_b).max()


def test_rmsnorm_strided(xh, orc):
    rng = np.random.default_rng(5)
    rows, cols, istr, ostr = 4, 256, 300, 512
    x = rng.standard_normal((rows, istr)).astype(np.float32)
    w = np.ones(cols, np.float32)
    xd, wd = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(w)
    od = xh.DeviceBuffer(rows * ostr * 4)
    od.zero()
    xh.rmsnorm(od.ptr, xh.F32, xd.ptr, xh.F32, wd.ptr, rows, cols, istr, ostr)
    xh.synchronize()
    got = od.to_numpy(np.float32, (rows, ostr))
    assert np.abs(got[:, :cols] - orc.rmsnorm(x[:, :cols].copy(), w)).max() < 1e-5
    assert not got[:, cols:].any()


def test_rope_tables_bit_exact(xh, orc):
    for dim, mp in ((128, 2048), (2, 10), (64, 300)):
        t = xh.RopeTables(dim, mp)
        c, s = t.to_numpy()
        ec, es = orc.rope_tables(dim, mp)
        assert np.array_equal(c, ec) and np.array_equal(s, es)


def test_rotary_embedding_golden_and_bit_exact(xh, orc):
    # golden constants of the reference unit test (tests/ut/rotary_embedding_test.cpp:28-57)
    q = np.array([4, 4, 4, 4, 3, 2, 1, 1, 4, 4, 2, 1, 4, 1, 3, 0], np.float32)
    k = np.ones(16, np.float32)
    qg = np.array([-1.20467, 5.52709, -1.20467, 5.52709, 3, 2, 1, 1, -1.20467, 5.52709, 0.239134, 2.22324, 4, 1, 3, 0])
    kg = np.array([-0.301169, 1.38177, -0.301169, 1.38177, 1, 1, 1, 1, -0.301169, 1.38177, -0.301169, 1.38177, 1, 1,
                   1, 1])
    t = xh.RopeTables(2, 10)
    qd, kd = xh.DeviceBuffer.from_numpy(q), xh.DeviceBuffer.from_numpy(k)
    pos = xh.DeviceBuffer.from_numpy(np.array([1, 0, 1, 0], np.int32))
    xh.rotary_embedding(xh.F32, pos.ptr, qd.ptr, kd.ptr, t, 2, 4, 4, 4, 2, 2, 2)
    xh.synchronize()
    assert np.abs(qd.to_numpy(np.float32, 16) - qg).max() < 1e-3
    assert np.abs(kd.to_numpy(np.float32, 16) - kg).max() < 1e-3
    # Llama shape, fp32 in place: identical bits to the oracle (same fused multiply-adds)
    rng = np.random.default_rng(7)
    T, qh, kh, D = 9, 32, 8, 128
    stride = (qh + 2 * kh) * D
    qkv = rng.standard_normal((T, stride)).astype(np.float32)
    positions = rng.integers(0, 512, T).astype(np.int32)
    t = xh.RopeTables(D, 512)
    cos, sin = orc.rope_tables(D, 512)
    exp = qkv.copy()
    orc.lib.orc_rope_apply_tokens(C.c_void_p(exp.ctypes.data), C.c_void_p(exp.ctypes.data + qh * D * 4), orc.p(cos),
                                  orc.p(sin), stride, stride, D, T, qh, kh, orc.p(positions))
    dev = xh.DeviceBuffer.from_numpy(qkv)
    pd = xh.DeviceBuffer.from_numpy(positions)
    xh.rotary_embedding(xh.F32, pd.ptr, dev.ptr, dev.at(qh * D * 4), t, D, stride, stride, T, qh, D, kh)
    xh.synchronize()
    assert np.array_equal(dev.to_numpy(np.float32, (T, stride)).view(np.uint32), exp.view(np.uint32))


@pytest.mark.parametrize("int8", [0, 1])
@pytest.mark.parametrize("rope", [0, 1])
@pytest.mark.parametrize("S,past,max_seq", [(5, 33, 70), (75, 13, 128), (64, 32, 96), (16, 0, 40)])
def test_kv_append_bit_exact(xh, orc, int8, rope, S, past, max_seq):
    """(From 16 tokens on a rotating append takes the kernel that works by 32-token cache blocks: 75 tokens behind 13
    fill their first and last block partly, 64 behind 32 fill two blocks exactly, 16 from 0 half of one.)"""
    rng = np.random.default_rng(11 + int8 + S)
    B, qh, kh, D = 2, 8, 2, 128
    stride = (qh + 2 * kh) * D
    qkv = orc.round_bf16(rng.standard_normal((B * S, stride)) * 3.0)
    qkv[1, qh * D:(qh + 1) * D] = 0.0  # an all-zero key row: scale 0, codes 0
    cache = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, kh, max_seq, D)
    tables = xh.RopeTables(D, 128) if rope else None
    dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(qkv))
    xh.rope_kvstore(cache, dev.ptr, xh.BF16, stride, B, S, qh, tables, past)
    xh.synchronize()
    # oracle: rotate q and k in fp32, store k and v rows
    exp = qkv.copy()
    if rope:
        cos, sin = orc.rope_tables(D, 128)
        orc.lib.orc_rope_apply(C.c_void_p(exp.ctypes.data), C.c_void_p(exp.ctypes.data + qh * D * 4), stride, stride,
                               orc.p(cos), orc.p(sin), D // 2, orc.p(np.array([B, S, qh, D, kh], np.int32)),
                               orc.p(np.arange(past, past + S, dtype=np.int32)))
    kc, vc = orc.KVCache(int8, B, kh, max_seq, D), orc.KVCache(int8, B, kh, max_seq, D)
    for b in range(B):
        rows = exp[b * S:(b + 1) * S]
        kc.store(b, past, rows[:, qh * D:(qh + kh) * D].copy())
        vc.store(b, past, rows[:, (qh + kh) * D:].copy())
    kd, ks = cache.export(0)
    vd, vs = cache.export(1)
    assert np.array_equal(kd, kc.data) and np.array_equal(vd, vc.data)
    if int8:
        assert np.array_equal(ks.view(np.uint32), kc.scales.view(np.uint32))
        assert np.array_equal(vs.view(np.uint32), vc.scales.view(np.uint32))
    # the query block is rotated in place and narrowed to bf16; key/value columns untouched
    got = orc.from_bf16(dev.to_numpy(np.uint16, (B * S, stride)))
    assert np.array_equal(got[:, :qh * D], orc.round_bf16(exp[:, :qh * D]))
    assert np.array_equal(got[:, qh * D:], qkv[:, qh * D:])


@pytest.mark.parametrize("int8", [0, 1])
def test_kv_import_export_roundtrip(xh, orc, int8):
    rng = np.random.default_rng(13)
    B, H, S, D = 3, 2, 45, 128
    cache = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, H, S, D)
    if int8:
        data = rng.integers(-127, 128, (B, H, S, D)).astype(np.int8)
    else:
        data = orc.to_fp16(rng.standard_normal((B, H, S, D)))
    scales = rng.uniform(0.01, 0.1, (B, H, S)).astype(np.float32)
    for which in (0, 1):
        cache.load(which, data, scales)
        d, s = cache.export(which)
        assert np.array_equal(d, data)
        if int8:
            assert np.array_equal(s, scales)
        # the reference's other layout, [S][B][H][D] (ENABLE_KV_TRANS off, kvcache_tensor.h:113-117): out of the same cache,
        # and into a fresh one
        sbhd = np.ascontiguousarray(data.transpose(2, 0, 1, 3))
        d2, s2 = cache.export(which, sbhd=True)
        assert np.array_equal(d2, sbhd) and (not int8 or np.array_equal(s2, scales))
        other = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, H, S, D)
        other.load(which, sbhd, scales, sbhd=True)
        d3, s3 = other.export(which)
        assert np.array_equal(d3, data) and (not int8 or np.array_equal(s3, scales))
        other.free()


# index vectors of the reference's own reorder test (tests/ut/kv_reorder_test.cpp:64-124): the fixed ones of
# reorder4 / reorder6, samples of reorder8 (beam size 4, two user sequences) and of reorder6More
REORDER_CASES = [
    [0, 2, 1, 3], [0, 0, 0, 0], [1, 1, 0, 0], [1, 0, 2, 1], [0, 1, 0, 1],
    [0, 2, 1, 4, 3, 3], [1, 2, 3, 4, 5, 0], [1, 3, 2, 4, 3, 5], [2, 1, 0, 4, 5, 0], [2, 0, 1, 5, 5, 4],
    [3, 0, 0, 2, 5, 7, 7, 4], [1, 1, 3, 2, 6, 6, 4, 5], [2, 3, 0, 1, 7, 4, 5, 6],
    [0, 0, 0, 0, 5, 4], [3, 2, 1, 0, 5, 4], [1, 3, 3, 1, 5, 4],
]


@pytest.mark.parametrize("int8", [0, 1])
def test_kv_reorder_reference_cases(xh, orc, int8):
    """Every (position, row, head) holds a value of its own (the reference test's fill, :29-40); after
    reorder(idx) row b must hold what row idx[b] held (:44-55), for keys, values and INT8 scales alike.
    Positions outside [pos0, pos1) rounded to 32-token blocks stay what they were."""
    H, S, D = 4, 70, 128
    for case, idx in enumerate(REORDER_CASES):
        B = len(idx)
        cache = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, H, S, D)
        seq, row, head = np.meshgrid(np.arange(S), np.arange(B), np.arange(H), indexing="ij")
        val = (seq * B + row) + 0.01 * head  # [S][B][H]
        val = np.transpose(val, (1, 2, 0))  # [B][H][S]
        if int8:
            data = np.broadcast_to(((seq * B + row) % 251 - 125).transpose(1, 2, 0)[..., None], (B, H, S, D)).astype(np.int8)
            scales = (0.001 * (1 + val)).astype(np.float32)
        else:
            data = orc.to_fp16(np.broadcast_to(val[..., None], (B, H, S, D)))
            scales = np.zeros((B, H, S), np.float32)
        for which in (0, 1):
            cache.load(which, data + (which if int8 else 0), scales * (1 + which))
        pos0, pos1 = (0, S) if case % 2 == 0 else (33, 64)  # whole cache / the second 32-token block only
        cache.reorder(list(range(B)), idx, pos0, pos1)
        lo, hi = pos0 // 32 * 32, min(S, (pos1 + 31) // 32 * 32)
        for which in (0, 1):
            d, sc = cache.export(which)
            want_d = (data + (which if int8 else 0)).copy()
            want_s = (scales * (1 + which)).copy()
            src_d, src_s = want_d.copy(), want_s.copy()
            for b in range(B):
                want_d[b, :, lo:hi] = src_d[idx[b], :, lo:hi]
                want_s[b, :, lo:hi] = src_s[idx[b], :, lo:hi]
            assert np.array_equal(d[:, :, :S], want_d), (case, which)
            if int8:
                assert np.array_equal(sc[:, :, :S], want_s), (case, which)
        cache.free()


def test_kvstore_rejects_overflow(xh):
    cache = xh.KVCache(xh.FP16, 1, 2, 16, 128)
    dev = xh.DeviceBuffer(4 * (8 + 4) * 128 * 2)
    with pytest.raises(xh.XftHipError):
        xh.rope_kvstore(cache, dev.ptr, xh.BF16, (8 + 4) * 128, 1, 4, 8, None, 14)
    with pytest.raises(xh.XftHipError):
        xh.rope_kvstore(cache, dev.ptr, xh.BF16, (8 + 4) * 128, 2, 1, 8, None, 0)


def test_copy_kernel_copies_and_checks_alignment(xh):
    rng = np.random.default_rng(17)
    a = rng.integers(0, 2 ** 31, 3 * 4096 + 4, dtype=np.int64).astype(np.uint32)
    src = xh.DeviceBuffer.from_numpy(a)
    dst = xh.DeviceBuffer(a.nbytes)
    dst.zero()
    xh.copy_kernel(dst.ptr, src.ptr, a.nbytes)
    xh.synchronize()
    assert np.array_equal(dst.to_numpy(np.uint32, a.shape), a)
    with pytest.raises(xh.XftHipError):
        xh.copy_kernel(dst.ptr, src.ptr, 24)  # not a multiple of 16 bytes
