"""Attention over a block-paged BF16 KV cache (xft::invokeAttention, include/layers_attention.h:22-59,
src/kernels/attention_kernels.cpp:24-157) on the GPU against the CPU oracle: decode over ragged
contexts through shuffled block tables (MHA and grouped heads, several block sizes, strided rows),
prefill of ragged sequences, and the host entry point driven as a serving loop would drive it
(prefill, then decode steps that grow the tables).  The reference has no test of this function; the
oracle is pinned against float64 brute force in tests/test_oracle_pins.py.
Tolerance: outputs are bf16 (relative step 2^-8); |d| <= 2e-2 and cosine >= 0.9999 on N(0,1) inputs."""
import ctypes as C
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init()
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def _cos(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def _bf(orc, rng, shape):
    return orc.round_bf16(rng.standard_normal(shape).astype(np.float32))


def _tables(rng, ctx, block_size, block_num, extra=1):
    """Disjoint random blocks for every sequence, enough for ctx[b] + extra tokens."""
    need = [(c + extra + block_size - 1) // block_size for c in ctx]
    assert sum(need) <= block_num
    perm = rng.permutation(block_num)
    tab = np.zeros((len(ctx), max(need)), np.int32)
    at = 0
    for b, n in enumerate(need):
        tab[b, :n] = perm[at:at + n]
        at += n
    return tab, np.asarray(need, np.int32)


@pytest.mark.parametrize("B,qH,kvH,block_size,max_ctx", [(1, 32, 32, 4, 700), (5, 32, 8, 16, 3000), (32, 32, 32, 16, 300),
                                                       (3, 8, 2, 1, 40), (2, 32, 8, 64, 9000)])
def test_paged_decode_matches_oracle(xh, orc, B, qH, kvH, block_size, max_ctx):
    D = 128
    rng = np.random.default_rng(B * 1000 + block_size)
    ctx = rng.integers(0, max_ctx, B).astype(np.int32)
    ctx[0] = max_ctx - 1
    if B > 1:
        ctx[1] = 0  # a sequence whose only token is the new one
    if B > 2:
        ctx[2] = (ctx[2] // block_size) * block_size  # the new token opens a block
    block_num = int(sum((c + 1 + block_size - 1) // block_size for c in ctx)) + 3
    tab, _ = _tables(rng, ctx, block_size, block_num)
    slots = np.asarray([tab[b, ctx[b] // block_size] * block_size + ctx[b] % block_size for b in range(B)], np.int32)
    kc, vc = _bf(orc, rng, (block_num, block_size, kvH, D)), _bf(orc, rng, (block_num, block_size, kvH, D))
    q_stride, kv_stride = qH * D + 64, kvH * D + 8
    q, k, v = _bf(orc, rng, (B, q_stride)), _bf(orc, rng, (B, kv_stride)), _bf(orc, rng, (B, kv_stride))
    dev = lambda a: xh.DeviceBuffer.from_numpy(np.ascontiguousarray(a))
    dkc, dvc = dev(orc.to_bf16(kc)), dev(orc.to_bf16(vc))
    dq, dk, dv = dev(orc.to_bf16(q)), dev(orc.to_bf16(k)), dev(orc.to_bf16(v))
    dt, dc, ds = dev(tab), dev(ctx), dev(slots)
    out = xh.DeviceBuffer(B * qH * D * 2)
    scale = 1.0 / np.sqrt(D)
    xh.paged_attention_decode(out.ptr, dq.ptr, dk.ptr, dv.ptr, qH, kvH, D, q_stride, kv_stride, qH * D, scale, B, dkc.ptr, dvc.ptr,
                              block_num, block_size, dt.ptr, tab.shape[1], dc.ptr, ds.ptr, int(ctx.max()))
    xh.synchronize()
    got = orc.from_bf16(out.to_numpy(np.uint16, (B, qH, D)))
    ref = orc.paged_attention_decode(q[:, :qH * D].reshape(B, qH, D), k[:, :kvH * D].reshape(B, kvH, D),
                                     v[:, :kvH * D].reshape(B, kvH, D), kc, vc, tab, ctx, slots, scale)
    # the new rows reached their slots, nothing else moved (kc / vc were updated in place by the oracle)
    assert np.array_equal(orc.from_bf16(dkc.to_numpy(np.uint16, kc.shape)), kc)
    assert np.array_equal(orc.from_bf16(dvc.to_numpy(np.uint16, vc.shape)), vc)
    err = float(np.abs(got - ref).max())
    print(f"paged decode B={B} heads {qH}/{kvH} block {block_size}: max-abs {err:.2e}, cosine {_cos(got, ref):.6f}", flush=True)
    assert err <= 2e-2 and _cos(got, ref) >= 0.9999


@pytest.mark.parametrize("qH,kvH,lens,block_size", [(32, 32, [7, 128, 300], 16), (32, 8, [1, 1024], 4), (8, 8, [33], 8)])
def test_paged_prefill_matches_oracle(xh, orc, qH, kvH, lens, block_size):
    D = 128
    rng = np.random.default_rng(sum(lens))
    T = sum(lens)
    block_num = sum((L + block_size - 1) // block_size for L in lens) + 2
    tab, _ = _tables(rng, [L - 1 for L in lens], block_size, block_num)
    slots = np.concatenate([[tab[b, t // block_size] * block_size + t % block_size for t in range(L)] for b, L in enumerate(lens)]).astype(np.int32)
    kc, vc = _bf(orc, rng, (block_num, block_size, kvH, D)), _bf(orc, rng, (block_num, block_size, kvH, D))
    q, k, v = _bf(orc, rng, (T, qH, D)), _bf(orc, rng, (T, kvH, D)), _bf(orc, rng, (T, kvH, D))
    dev = lambda a: xh.DeviceBuffer.from_numpy(np.ascontiguousarray(a))
    dkc, dvc = dev(orc.to_bf16(kc)), dev(orc.to_bf16(vc))
    dq, dk, dv, ds = dev(orc.to_bf16(q)), dev(orc.to_bf16(k)), dev(orc.to_bf16(v)), dev(slots)
    out = xh.DeviceBuffer(T * qH * D * 2)
    scale = 1.0 / np.sqrt(D)
    xh.paged_attention_prefill(out.ptr, dq.ptr, dk.ptr, dv.ptr, qH, kvH, D, qH * D, kvH * D, qH * D, scale, lens, dkc.ptr, dvc.ptr,
                               block_num, block_size, ds.ptr)
    xh.synchronize()
    got = orc.from_bf16(out.to_numpy(np.uint16, (T, qH, D)))
    ref = orc.paged_attention_prefill(q, k, v, lens, kc, vc, slots, scale)
    assert np.array_equal(orc.from_bf16(dkc.to_numpy(np.uint16, kc.shape)), kc)
    assert np.array_equal(orc.from_bf16(dvc.to_numpy(np.uint16, vc.shape)), vc)
    err = float(np.abs(got - ref).max())
    print(f"paged prefill heads {qH}/{kvH} lens {lens}: max-abs {err:.2e}, cosine {_cos(got, ref):.6f}", flush=True)
    assert err <= 2e-2 and _cos(got, ref) >= 0.9999


def test_invoke_attention_serving_loop(orc):
    """xft::invokeAttention on host buffers: prefill of two sequences, then decode steps that append to
    the paged cache; outputs against the oracle and the caller's cache arrays kept current."""
    C.CDLL(os.path.join(ROOT, "xfastertransformer_amd", "libxft_hip.so"), mode=C.RTLD_GLOBAL)
    lib = C.CDLL(os.path.join(ROOT, "xfastertransformer_amd", "libxft_layers.so"))
    fn = getattr(lib, "_ZN3xft15invokeAttentionENS_8DataTypeEPvPKvS3_S3_PiS4_iifiPKiS3_S3_S4_S4_S4_S4_ibS4_")
    P, I = C.c_void_p, C.c_int
    fn.argtypes = [I, P, P, P, P, P, P, I, I, C.c_float, I, P, P, P, P, P, P, P, I, C.c_bool, P]
    fn.restype = None
    ptr = lambda a: a.ctypes.data_as(P)
    BF16 = 1
    qH, kvH, D, bs, block_num = 32, 8, 128, 16, 24
    rng = np.random.default_rng(77)
    lens = [37, 100]
    scale = 1.0 / np.sqrt(D)
    kc_f, vc_f = np.zeros((block_num, bs, kvH, D), np.float32), np.zeros((block_num, bs, kvH, D), np.float32)
    kc_h, vc_h = orc.to_bf16(kc_f), orc.to_bf16(vc_f)  # the caller's bf16 arrays
    blocks = [[3, 9, 17, 1], [5, 2, 11, 20, 7, 14, 8, 22]]
    slot_of = lambda b, t: blocks[b][t // bs] * bs + t % bs
    # prefill
    T = sum(lens)
    q, k, v = _bf(orc, rng, (T, qH, D)), _bf(orc, rng, (T, kvH, D)), _bf(orc, rng, (T, kvH, D))
    slots = np.asarray([slot_of(b, t) for b, L in enumerate(lens) for t in range(L)], np.int32)
    out = np.zeros((T, qH * D), np.uint16)
    qb, kb, vb = orc.to_bf16(q), orc.to_bf16(k), orc.to_bf16(v)
    qs = np.asarray([T, qH, D], np.int32)
    ks = np.asarray([T, kvH, D], np.int32)
    cs = np.asarray([block_num, bs, kvH, D], np.int32)
    tl = np.asarray(lens, np.int32)
    fn(BF16, ptr(out), ptr(qb), ptr(kb), ptr(vb), ptr(qs), ptr(ks), qH * D, kvH * D, scale, 2, ptr(tl), ptr(kc_h), ptr(vc_h), ptr(cs),
       None, None, None, 0, True, ptr(slots))
    ref = orc.paged_attention_prefill(q, k, v, lens, kc_f, vc_f, slots, scale)
    got = orc.from_bf16(out).reshape(T, qH, D)
    assert np.abs(got - ref).max() <= 2e-2 and _cos(got, ref) >= 0.9999
    assert np.array_equal(orc.from_bf16(kc_h), kc_f) and np.array_equal(orc.from_bf16(vc_h), vc_f)
    # decode steps: the second sequence crosses a block boundary at 112
    ctx = np.asarray(lens, np.int32)
    for step in range(14):
        q, k, v = _bf(orc, rng, (2, qH, D)), _bf(orc, rng, (2, kvH, D)), _bf(orc, rng, (2, kvH, D))
        nums = np.asarray([(c + 1 + bs - 1) // bs for c in ctx], np.int32)
        tab = np.zeros((2, int(nums.max())), np.int32)
        for b in range(2):
            tab[b, :nums[b]] = blocks[b][:nums[b]]
        slots = np.asarray([slot_of(b, int(ctx[b])) for b in range(2)], np.int32)
        out = np.zeros((2, qH * D), np.uint16)
        qb, kb, vb = orc.to_bf16(q), orc.to_bf16(k), orc.to_bf16(v)
        qs = np.asarray([2, qH, D], np.int32)
        ks = np.asarray([2, kvH, D], np.int32)
        fn(BF16, ptr(out), ptr(qb), ptr(kb), ptr(vb), ptr(qs), ptr(ks), qH * D, kvH * D, scale, 2, None, ptr(kc_h), ptr(vc_h), ptr(cs),
           ptr(tab), ptr(nums), ptr(ctx), 0, False, ptr(slots))
        ref = orc.paged_attention_decode(q, k, v, kc_f, vc_f, tab, ctx, slots, scale)
        got = orc.from_bf16(out).reshape(2, qH, D)
        assert np.abs(got - ref).max() <= 2e-2 and _cos(got, ref) >= 0.9999, step
        assert np.array_equal(orc.from_bf16(kc_h), kc_f) and np.array_equal(orc.from_bf16(vc_h), vc_f)
        ctx = ctx + 1
