"""GPU parity of the two decode-step fusions of the M <= 32 weight-only GEMM against the CPU
oracle's separate steps (RMSNorm -> bf16 -> GEMM [-> bf16 -> RoPE -> cache append]), through the
C-ABI: xfthip_gemm_gateup_silu_rmsnorm and xfthip_gemm_qkv_rmsnorm_rope."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

KINDS = {"int8": 0, "uint4": 1, "nf4": 2}


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


def _quant(orc, kind, K, N, seed, asym_int8=False):
    rng = np.random.default_rng(seed)
    w = orc.quantize(kind, (rng.standard_normal((K, N)) * 0.02).astype(np.float32))
    if asym_int8:
        w.zero = (rng.standard_normal(N) * 0.01).astype(np.float32)
    return w


@pytest.mark.parametrize("kind", ["int8", "uint4", "nf4"])
@pytest.mark.parametrize("M,K,I", [(1, 4096, 11008), (4, 4096, 1408), (3, 512, 96)])
def test_gateup_silu_with_norm_prologue(xh, orc, kind, M, K, I):
    k = KINDS[kind]
    w = _quant(orc, k, K, 2 * I, 80)
    rng = np.random.default_rng(81 + M)
    x = (rng.standard_normal((M, K)) * 1.7).astype(np.float32)
    g = rng.uniform(0.5, 1.5, K).astype(np.float32)
    dw = xh.Weight(k, K, 2 * I, w.q, w.scale, w.zero, flags=xh.WF_GATEUP)
    xd, gd = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(g)
    od = xh.DeviceBuffer(M * I * 4)
    xh.gemm_gateup_silu_rmsnorm(dw, xd.ptr, M, K, gd.ptr, 1e-6, od.ptr, I, xh.F32)
    xh.synchronize()
    got = od.to_numpy(np.float32, (M, I))
    n = orc.round_bf16(orc.rmsnorm(x, g, 1e-6))
    exp = orc.silu_sum(orc.qgemm(w, n))
    # the norm's fp32 sum runs in another order than the oracle's, which moves a bf16 rounding of
    # the normalised input now and then: one such flip is worth |w| * 2^-8 in the output
    assert np.abs(got - exp).max() < 4e-3 + 2e-3 * np.abs(exp).max()
    assert _cos(got, exp) >= 0.9999
    dw.free()


@pytest.mark.parametrize("kind,asym", [("int8", False), ("int8", True), ("uint4", False), ("nf4", False)])
@pytest.mark.parametrize("M,qh,kh,K", [(1, 32, 32, 4096), (3, 8, 2, 512), (4, 4, 4, 1024)])
def test_qkv_with_norm_prologue_and_rope_epilogue(xh, orc, kind, asym, M, qh, kh, K):
    k = KINDS[kind]
    D, max_seq = 128, 96
    N = (qh + 2 * kh) * D
    w = _quant(orc, k, K, N, 90, asym_int8=asym)
    rng = np.random.default_rng(91 + M)
    x = (rng.standard_normal((M, K)) * 1.3).astype(np.float32)
    g = rng.uniform(0.5, 1.5, K).astype(np.float32)
    pos = rng.integers(0, max_seq, M).astype(np.int32)
    dw = xh.Weight(k, K, N, w.q, w.scale, w.zero)
    cache = xh.KVCache(xh.FP16, 4, kh, max_seq, D)
    tables = xh.RopeTables(D, 128)
    xd, gd = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(g)
    qd = xh.DeviceBuffer(M * qh * D * 2)
    pd = xh.DeviceBuffer.from_numpy(pos)
    xh.gemm_qkv_rmsnorm_rope(dw, cache, xd.ptr, M, K, gd.ptr, 1e-5, qd.ptr, qh * D, qh, tables, 0, pos_dev=pd.ptr)
    xh.synchronize()
    # oracle: the separate steps with their bf16 hand-over points
    n = orc.round_bf16(orc.rmsnorm(x, g, 1e-5))
    qkv = orc.round_bf16(orc.qgemm(w, n))
    cos, sin = orc.rope_tables(D, 128)
    exp = qkv.copy()
    for m in range(M):  # every row is its own sequence at its own position
        row = exp[m:m + 1]
        orc.lib.orc_rope_apply(C.c_void_p(row.ctypes.data), C.c_void_p(row.ctypes.data + qh * D * 4), N, N, orc.p(cos), orc.p(sin),
                               D // 2, orc.p(np.array([1, 1, qh, D, kh], np.int32)), orc.p(pos[m:m + 1].copy()))
    got_q = orc.from_bf16(qd.to_numpy(np.uint16, (M, qh * D)))
    exp_q = orc.round_bf16(exp[:, :qh * D])
    kd, _ = cache.export(0)
    vd, _ = cache.export(1)
    got_k = np.stack([kd[m, :, pos[m], :] for m in range(M)]).view(np.float16).astype(np.float32).reshape(M, kh * D)
    got_v = np.stack([vd[m, :, pos[m], :] for m in range(M)]).view(np.float16).astype(np.float32).reshape(M, kh * D)
    exp_k = exp[:, qh * D:(qh + kh) * D].astype(np.float16).astype(np.float32)
    exp_v = exp[:, (qh + kh) * D:].astype(np.float16).astype(np.float32)
    # a flipped bf16 rounding of the normalised input moves a projection output by about 1e-3; an
    # output that then rounds the other way in bf16 differs by one bf16 step of its magnitude
    for got, ex in ((got_q, exp_q), (got_k, exp_k), (got_v, exp_v)):
        assert np.abs(got - ex).max() <= 4e-3 + np.abs(ex).max() * 2.0 ** -7
        assert _cos(got, ex) >= 0.9999
    # nothing but the M new rows was written
    mask = np.ones(kd.shape[:3], bool)
    for m in range(M):
        mask[m, :, pos[m]] = False
    assert not kd[mask].any() and not vd[mask].any()
    dw.free()


def test_fused_entry_points_reject_bad_arguments(xh, orc):
    w = _quant(orc, 0, 512, (4 + 4) * 128, 95)
    dw = xh.Weight(0, 512, 1024, w.q, w.scale, w.zero)
    gw = xh.Weight(0, 512, 1024, w.q, w.scale, w.zero, flags=xh.WF_GATEUP)
    x = xh.DeviceBuffer(8 * 512 * 4)
    g = xh.DeviceBuffer(512 * 4)
    o = xh.DeviceBuffer(8 * 1024 * 4)
    tables = xh.RopeTables(128, 64)
    fp16_cache = xh.KVCache(xh.FP16, 2, 2, 32, 128)
    int8_cache = xh.KVCache(xh.INT8, 2, 2, 32, 128)
    with pytest.raises(xh.XftHipError):
        xh.gemm_gateup_silu_rmsnorm(gw, x.ptr, 5, 512, g.ptr, 1e-6, o.ptr, 512, xh.F32)  # more than 4 rows
    with pytest.raises(xh.XftHipError):
        xh.gemm_gateup_silu_rmsnorm(dw, x.ptr, 1, 512, g.ptr, 1e-6, o.ptr, 512, xh.F32)  # not a gate/up weight
    with pytest.raises(xh.XftHipError):
        xh.gemm_qkv_rmsnorm_rope(dw, int8_cache, x.ptr, 1, 512, g.ptr, 1e-6, o.ptr, 512, 4, tables, 0)  # INT8 cache
    with pytest.raises(xh.XftHipError):
        xh.gemm_qkv_rmsnorm_rope(dw, fp16_cache, x.ptr, 3, 512, g.ptr, 1e-6, o.ptr, 512, 4, tables, 0)  # rows > cache batch
    with pytest.raises(xh.XftHipError):
        xh.gemm_qkv_rmsnorm_rope(dw, fp16_cache, x.ptr, 1, 512, g.ptr, 1e-6, o.ptr, 512, 6, tables, 0)  # head counts do not match N
    with pytest.raises(xh.XftHipError):
        xh.gemm_qkv_rmsnorm_rope(dw, fp16_cache, x.ptr, 1, 512, g.ptr, 1e-6, o.ptr, 512, 4, tables, 40)  # position past max_seq
