"""Cells of the benchmark configurations that the other GPU test files reach only at reduced sizes or not at
all, each at its full size:
  config 2 (weight-only GEMM sweep): (N, K) = (4096, 11008) at M in {1, 8, 32} for INT8 / UINT4 / NF4 with the
            plain epilogue, and (11008, 4096) at M = 8;
  config 3 (GQA decode attention, 32 query / 8 KV heads): batch 1 x {4096, 16384}, batch 16 x {1024, 16384} and
            batch 64 x 4096 tokens of context, FP16 and INT8 caches;
  config 1 (one Llama-2-7B-shape layer through the layer API): the xft::invokeLayerLLaMA symbol itself at hidden
            4096 / intermediate 11008 with dt = int8, a 128-token prefill and two decode steps.
Oracles: the scalar restatement of the reference's GEMM on sampled columns plus a BLAS product on the dequantised
weight for all of them; float64 textbook attention over what the cache holds; the oracle's decoder layer."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
D = 128
SCALE = 1.0 / np.sqrt(D)
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


_W = {}


def _weight(xh, orc, kind, K, N):
    key = (kind, K, N)
    if key not in _W:
        _W.clear()  # one large weight at a time
        rng = np.random.default_rng(2000 + K + N + KINDS[kind])
        w = orc.quantize(KINDS[kind], (rng.standard_normal((K, N)) * 0.02).astype(np.float32))
        _W[key] = (w, xh.Weight(KINDS[kind], K, N, w.q, w.scale, w.zero), orc.dequant(w))
    return _W[key]


# ------------------------------------------------------------------ config 2
@pytest.mark.parametrize("kind", ["int8", "uint4", "nf4"])
@pytest.mark.parametrize("M,K,N", [(1, 11008, 4096), (8, 11008, 4096), (32, 11008, 4096), (8, 4096, 11008)])
def test_gemm_sweep_few_rows_full_shapes(xh, orc, kind, M, K, N):
    print(f"case kind={kind} M={M} K={K} N={N}", flush=True)
    w, dw, Wd = _weight(xh, orc, kind, K, N)
    A = orc.round_bf16(np.random.default_rng(11 * M + K).standard_normal((M, K)))
    a_dev = xh.DeviceBuffer.from_numpy(orc.to_bf16(A))
    for c_dtype in (xh.F32, xh.BF16):
        c_dev = xh.DeviceBuffer(M * N * 4)
        c_dev.zero()
        xh.gemm(dw, a_dev.ptr, M, K, c_dev.ptr, N, c_dtype)
        xh.synchronize()
        got = c_dev.to_numpy(np.float32, (M, N)) if c_dtype == xh.F32 else xh.bf16_bits_to_f32(c_dev.to_numpy(np.uint16, (M, N)))
        assert np.isfinite(got).all()
        blas = A.astype(np.float64) @ Wd.astype(np.float64)
        slack = 0.0 if c_dtype == xh.F32 else np.abs(blas) * 2.0 ** -8
        assert (np.abs(got - blas) <= 2e-3 + slack).all(), float(np.abs(got - blas).max())
        assert _cos(got, blas) >= 0.9999
        # the scalar restatement of the reference's arithmetic (all rows, K = 11008 takes a few seconds)
        exp = orc.qgemm(w, A)
        assert (np.abs(got - exp) <= 2e-3 + slack).all(), float(np.abs(got - exp).max())


# ------------------------------------------------------------------ config 3
@pytest.mark.parametrize("int8", [0, 1])
@pytest.mark.parametrize("B,ctx", [(1, 4096), (1, 16384), (16, 1024), (16, 16384), (64, 4096)])
def test_decode_attention_open_cells(xh, orc, int8, B, ctx):
    """Every sequence holds the same random rows rolled by its index (bounded host time); sampled sequences are
    compared with the float64 attention over what the cache holds."""
    print(f"case int8={int8} B={B} ctx={ctx}", flush=True)
    qh, kvh = 32, 8
    rng = np.random.default_rng(3 * ctx + B + int8)
    base_k = rng.standard_normal((ctx, kvh * D), dtype=np.float32)
    base_v = rng.standard_normal((ctx, kvh * D), dtype=np.float32)
    sample = sorted(set([0, B - 1, B // 2, B // 3]))
    kc, vc = orc.KVCache(int8, B, kvh, ctx, D), orc.KVCache(int8, B, kvh, ctx, D)
    for b in range(B):
        kc.store(b, 0, np.roll(base_k, 53 * b, 0))
        vc.store(b, 0, np.roll(base_v, 53 * b, 0))
    dc = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, kvh, ctx, D)
    dc.load(0, kc.data, kc.scales)
    dc.load(1, vc.data, vc.scales)
    q = orc.round_bf16(rng.standard_normal((B, qh * D)))
    qd = xh.DeviceBuffer.from_numpy(orc.to_bf16(q))
    od = xh.DeviceBuffer(q.size * 4)
    od.zero()
    xh.attention(dc, qd.ptr, qh * D, od.ptr, qh * D, xh.F32, B, 1, qh, SCALE, ctx - 1)
    xh.synchronize()
    got = od.to_numpy(np.float32, q.shape)
    assert np.isfinite(got).all()
    for b in sample:
        def rows(c):
            if int8:
                return c.data[b:b + 1].astype(np.float32) * c.scales[b:b + 1, :, :, None]
            return orc.from_fp16(c.data[b:b + 1])
        ref = orc.attention_ref_f64(q[b:b + 1], rows(kc), rows(vc), qh, kvh, D, [1], [ctx - 1], SCALE)
        err = float(np.abs(got[b] - ref[0]).max())
        # the reference's own tolerance here is 1e-3 / 3e-3 (cross_attention_test.cpp:108-113)
        assert err < 3e-3 and _cos(got[b], ref[0]) >= 0.9999, (b, err)


# ------------------------------------------------------------------ config 1
def test_invoke_layer_llama_7b_shape_int8(orc):
    """xft::invokeLayerLLaMA (include/layers_decoder.h, reference src/layers/decoder_layer.cpp:161-208) at the
    Llama-2-7B layer shape with dt = int8: fp32 host weights quantised by the library on first sight (per output
    channel, symmetric), a 128-token prompt and two decode steps with the caller-supplied pastSeqLen, as
    tests/ut/layers_decoder_test.cpp:25-60 drives it.  The oracle's layer gets the same weights quantised by the
    oracle's definition of the same quantiser."""
    INT8, SILU, RMS = 3, 3, 0
    P, I = C.c_void_p, C.c_int
    C.CDLL(os.path.join(ROOT, "xfastertransformer_amd", "libxft_hip.so"), mode=C.RTLD_GLOBAL)
    lib = C.CDLL(os.path.join(ROOT, "xfastertransformer_amd", "libxft_layers.so"))
    layer = getattr(lib, "_ZN3xft16invokeLayerLLaMAENS_8DataTypeENS_14ActivationTypeENS_8NormTypeEiiiiiiiiiiiiPviPKviPKfS7_S5_S5_S5_S5_S7_S7_S5_S5_S5_S7_S7_S7_S7_")
    layer.argtypes = [I] * 15 + [P, I, P, I] + [P] * 15
    layer.restype = None
    hidden, inter, qh, kvh = 4096, 11008, 32, 32
    rng = np.random.default_rng(0)
    qkv = (rng.standard_normal((hidden, (qh + 2 * kvh) * D), dtype=np.float32) * 0.02)
    wo = (rng.standard_normal((qh * D, hidden), dtype=np.float32) * 0.02)
    gate = (rng.standard_normal((hidden, inter), dtype=np.float32) * 0.02)
    up = (rng.standard_normal((hidden, inter), dtype=np.float32) * 0.02)
    down = (rng.standard_normal((inter, hidden), dtype=np.float32) * 0.02)
    ones = np.ones(hidden, np.float32)
    ow = [orc.quantize(0, w) for w in (qkv, wo, np.concatenate([gate, up], 1), down)]
    max_pos = 160
    ref = orc.LlamaLayerOracle(hidden, inter, qh, kvh, D, *ow, ones, ones, max_seq=max_pos, rounding="bf16", gemm="blas",
                               prefill_attention="cache")
    ptr = lambda a: a.ctypes.data_as(C.c_void_p)
    qcols = kvcols = qh * D
    past = 0
    for step, S in enumerate((128, 1, 1)):
        x = orc.round_bf16(rng.standard_normal((S, hidden)))
        out = np.zeros_like(x)
        layer(INT8, SILU, RMS, 1, S, D, qh, kvh, max_pos, max_pos, past, past + S, step, hidden, inter, ptr(out), hidden, ptr(x), hidden,
              ptr(ones), None, ptr(qkv), C.c_void_p(qkv.ctypes.data + qcols * 4), C.c_void_p(qkv.ctypes.data + (qcols + kvcols) * 4),
              ptr(wo), ptr(ones), None, ptr(gate), ptr(up), ptr(down), None, None, None, None)
        exp = ref.forward(x, 1, S, past)
        err = np.abs(out - exp)
        print(f"step {step} (S = {S}): max-abs {err.max():.3e} rms {np.sqrt((err ** 2).mean()):.3e} cosine {_cos(out, exp):.6f} "
              f"(|y| max {np.abs(exp).max():.2f})", flush=True)
        # the whole-layer bars of the layer tests: cosine 0.9999, rms 1e-2, max-abs 5e-2 (one bf16 ulp of |y| ~ 8 is 0.0625)
        assert _cos(out, exp) >= 0.9999 and np.sqrt((err ** 2).mean()) < 1e-2 and err.max() < 5e-2, (step, float(err.max()))
        past += S
    orc.clear_blas_cache()
