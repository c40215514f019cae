"""GPU parity of the Mixtral-style sparse MLP (router, top-2 with 2-way softmax, gather, expert
SwiGLU MLPs, weighted scatter-add) against the oracle's restatement of MixtralMLP
(reference src/layers/mlp_mixtral.h:85-283)."""
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


def test_top2_selection_and_weights(xh, orc):
    rng = np.random.default_rng(1)
    logits = rng.standard_normal((300, 8)).astype(np.float32)
    logits[5] = [1, 5, 5, 0, 5, -1, 2, 2]  # ties: the lower index wins
    logits[6] = [3, 3, 3, 3, 3, 3, 3, 3]
    dev = xh.DeviceBuffer.from_numpy(logits)  # kept alive across the call: a temporary would be freed before the kernel runs
    sel, w = xh.moe_top2(dev.ptr, 300, 8)
    esel, ew = orc.moe_top2(logits)
    assert np.array_equal(sel, esel)
    assert list(sel[5]) == [1, 2] and list(sel[6]) == [0, 1]
    assert np.abs(w - ew).max() < 1e-6
    assert np.abs(w.sum(1) - 1).max() < 1e-6


def _experts(orc, rng, kind, hidden, inter, E):
    out = []
    for _ in range(E):
        gu = orc.quantize(kind, (rng.standard_normal((hidden, 2 * inter)) * 0.02).astype(np.float32))
        dn = orc.quantize(kind, (rng.standard_normal((inter, hidden)) * 0.02).astype(np.float32))
        out.append((gu, dn))
    return out


@pytest.mark.parametrize("tokens", [1, 7, 64, 200])
@pytest.mark.parametrize("override", [False, True])
def test_mixtral_mlp_vs_oracle(xh, orc, tokens, override):
    hidden, inter, E = 1024, 3584, 8
    rng = np.random.default_rng(tokens)
    experts = _experts(orc, rng, 0, hidden, inter, E)
    router = (rng.standard_normal((hidden, E)) * 0.05).astype(np.float32)
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32) if override else None
    moe = xh.MoE(hidden, inter, E, tokens, router, ln)
    for e, (gu, dn) in enumerate(experts):
        moe.set_expert(e, xh.Weight(0, gu.K, gu.N, gu.q, gu.scale, gu.zero, flags=xh.WF_GATEUP),
                       xh.Weight(0, dn.K, dn.N, dn.q, dn.scale, dn.zero))
    xd = xh.DeviceBuffer.from_numpy(x)
    od = xh.DeviceBuffer(x.nbytes)
    lod = None if lo is None else xh.DeviceBuffer.from_numpy(lo)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, None if lod is None else lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    # output over the input (the residual is read where it is written): the same bits
    sel2, w2 = moe.forward(xd.ptr, xd.ptr, tokens, True, None if lod is None else lod.ptr)
    xh.synchronize()
    assert np.array_equal(sel, sel2) and np.array_equal(w, w2)
    assert np.array_equal(xd.to_numpy(np.float32, x.shape), got)
    exp, esel, ew = orc.mixtral_mlp(x, ln, router, experts, lo, rounding="bf16")
    if override:
        assert np.array_equal(sel, esel)
    else:
        # router logits come from bf16 activations on both sides; a flip needs a near-tie
        same = (sel == esel).all(1)
        assert same.mean() > 0.97
        got, exp = got[same], exp[same]
        w, ew = w[same], ew[same]
    assert np.abs(w - ew).max() < 2e-3
    assert np.abs(got - exp).max() < 2e-2 and _cos(got, exp) >= 0.9999
    e32, _, _ = orc.mixtral_mlp(x, ln, router, experts, lo, rounding="fp32")
    if override:
        assert _cos(got, e32) >= 0.9999


@pytest.mark.parametrize("kind", [1, 2])
@pytest.mark.parametrize("tokens", [9, 150])
def test_mixtral_mlp_four_bit_experts(xh, orc, kind, tokens):
    """UINT4 and NF4 experts, through the per-expert launches (18 gathered rows) and through the launch
    that serves all experts at once (300 gathered rows), with two experts that get no token."""
    hidden, inter, E = 1024, 3584, 8
    rng = np.random.default_rng(100 * kind + tokens)
    experts = _experts(orc, rng, kind, hidden, inter, E)
    router = np.zeros((hidden, E), np.float32)
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32)
    lo[:, 3] = lo[:, 6] = -20.0
    moe = xh.MoE(hidden, inter, E, tokens, router, ln)
    for e, (gu, dn) in enumerate(experts):
        moe.set_expert(e, xh.Weight(kind, gu.K, gu.N, gu.q, gu.scale, gu.zero, flags=xh.WF_GATEUP),
                       xh.Weight(kind, dn.K, dn.N, dn.q, dn.scale, dn.zero))
    xd, lod = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(lo)
    od = xh.DeviceBuffer(x.nbytes)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    exp, esel, ew = orc.mixtral_mlp(x, ln, router, experts, lo, rounding="bf16")
    assert np.array_equal(sel, esel) and not np.isin(sel, (3, 6)).any()
    assert np.abs(w - ew).max() < 1e-6
    assert np.abs(got - exp).max() < 2e-2 and _cos(got, exp) >= 0.9999


@pytest.mark.parametrize("tokens", [6, 40])
def test_mixtral_mlp_bf16_experts(xh, orc, tokens):
    """BF16 expert weights (no codes to widen), per-expert launches and the launch that serves all experts: against a
    float64 restatement with the same bf16 hand-over points (normalised input, hidden activations)."""
    hidden, inter, E = 512, 1024, 8
    rng = np.random.default_rng(500 + tokens)
    Wgu = [orc.round_bf16(rng.standard_normal((hidden, 2 * inter)) * 0.05) for _ in range(E)]
    Wdn = [orc.round_bf16(rng.standard_normal((inter, hidden)) * 0.05) for _ in range(E)]
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32)
    moe = xh.MoE(hidden, inter, E, tokens, np.zeros((hidden, E), np.float32), ln)
    for e in range(E):
        moe.set_expert(e, xh.Weight(xh.W_BF16, hidden, 2 * inter, orc.to_bf16(Wgu[e]), flags=xh.WF_GATEUP),
                       xh.Weight(xh.W_BF16, inter, hidden, orc.to_bf16(Wdn[e])))
    xd, lod = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(lo)
    od = xh.DeviceBuffer(x.nbytes)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    esel, ew = orc.moe_top2(lo)
    assert np.array_equal(sel, esel) and np.abs(w - ew).max() < 1e-6
    xn = orc.round_bf16(orc.rmsnorm(x, ln)).astype(np.float64)
    exp = x.astype(np.float64).copy()
    for t in range(tokens):
        for s_ in range(2):
            e = int(esel[t, s_])
            gu = xn[t] @ Wgu[e].astype(np.float64)
            g, u = gu[:inter], gu[inter:]
            h = orc.round_bf16((g / (1.0 + np.exp(-g)) * u).astype(np.float32)[None])[0].astype(np.float64)
            exp[t] += float(ew[t, s_]) * (h @ Wdn[e].astype(np.float64))
    assert np.abs(got - exp).max() < 2e-2 and _cos(got, exp) >= 0.9999


@pytest.mark.parametrize("tokens", [12, 70])
def test_mixtral_mlp_experts_of_different_layouts(xh, orc, tokens):
    """Experts that cannot share a launch (some INT8 weights carry a zero-point vector, some do not) go through the
    per-expert launches with device-side row counts."""
    hidden, inter, E = 1024, 3584, 8
    rng = np.random.default_rng(700 + tokens)
    experts = _experts(orc, rng, 0, hidden, inter, E)
    router = np.zeros((hidden, E), np.float32)
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32)
    moe = xh.MoE(hidden, inter, E, tokens, router, ln)
    for e, (gu, dn) in enumerate(experts):
        zg, zd = (gu.zero, dn.zero) if e % 3 else (None, None)  # all zeros either way: same values, other kernel form
        moe.set_expert(e, xh.Weight(0, gu.K, gu.N, gu.q, gu.scale, zg, flags=xh.WF_GATEUP), xh.Weight(0, dn.K, dn.N, dn.q, dn.scale, zd))
    xd, lod = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(lo)
    od = xh.DeviceBuffer(x.nbytes)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    exp, esel, ew = orc.mixtral_mlp(x, ln, router, experts, lo, rounding="bf16")
    assert np.array_equal(sel, esel) and np.abs(w - ew).max() < 1e-6
    assert np.abs(got - exp).max() < 2e-2 and _cos(got, exp) >= 0.9999


def test_mixtral_shape_full_size_spot_check(xh, orc):
    """Mixtral-8x7B shape (hidden 4096, FFN 14336, 8 INT8 experts, 256 tokens, overridden N(0,1)
    logits): routing must equal the oracle's, and a handful of tokens are recomputed by the oracle."""
    hidden, inter, E, tokens = 4096, 14336, 8, 256
    rng = np.random.default_rng(4)
    # one expert's random codes shared by all experts keeps host time short; scales differ per expert
    q_gu = rng.integers(-127, 128, (hidden, 2 * inter)).astype(np.int8)
    q_dn = rng.integers(-127, 128, (inter, hidden)).astype(np.int8)
    experts = []
    for e in range(E):
        s_gu = np.full(2 * inter, 0.02 * 1.7 / 127 * (1 + 0.05 * e), np.float32)
        s_dn = np.full(hidden, 0.02 * 1.7 / 127 * (1 - 0.03 * e), np.float32)
        experts.append((orc.QWeight(0, hidden, 2 * inter, q_gu, s_gu, np.zeros(2 * inter, np.float32)),
                        orc.QWeight(0, inter, hidden, q_dn, s_dn, np.zeros(hidden, np.float32))))
    router = np.zeros((hidden, E), np.float32)
    ln = np.ones(hidden, np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32)
    moe = xh.MoE(hidden, inter, E, tokens, router, ln)
    for e, (gu, dn) in enumerate(experts):
        moe.set_expert(e, xh.Weight(0, gu.K, gu.N, gu.q, gu.scale, None, flags=xh.WF_GATEUP),
                       xh.Weight(0, dn.K, dn.N, dn.q, dn.scale, None))
    xd, lod = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(lo)
    od = xh.DeviceBuffer(x.nbytes)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    esel, ew = orc.moe_top2(lo)
    assert np.array_equal(sel, esel) and np.abs(w - ew).max() < 1e-6
    assert np.isfinite(got).all()
    for t in (0, 17, 255):
        xn = orc.round_bf16(orc.rmsnorm(x[t:t + 1], ln))
        ref = x[t:t + 1].copy()
        for s in range(2):
            gu, dn = experts[esel[t, s]]
            h = orc.round_bf16(orc.silu_sum(orc.qgemm(gu, xn)))
            ref = ref + ew[t, s] * orc.qgemm(dn, h)
        assert np.abs(got[t] - ref[0]).max() < 2e-2 * max(1.0, np.abs(ref).max()), t
        assert _cos(got[t], ref[0]) >= 0.9999


def test_layer_without_routing_output_is_capturable(xh, orc):
    """Asked for no routing output, the layer never waits for the device (the per-expert row counts stay in
    device memory), so it can be recorded into a graph: every replay, on fresh inputs and with eager work
    between the replays, must give the eager call's result bit for bit."""
    hidden, inter, E, tokens = 1024, 3584, 8, 96
    rng = np.random.default_rng(11)
    experts = _experts(orc, rng, 0, hidden, inter, E)
    router = (rng.standard_normal((hidden, E)) * 0.05).astype(np.float32)
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    moe = xh.MoE(hidden, inter, E, tokens, router, ln)
    for e, (gu, dn) in enumerate(experts):
        moe.set_expert(e, xh.Weight(0, gu.K, gu.N, gu.q, gu.scale, gu.zero, flags=xh.WF_GATEUP),
                       xh.Weight(0, dn.K, dn.N, dn.q, dn.scale, dn.zero))
    xs = [orc.round_bf16(rng.standard_normal((tokens, hidden))) for _ in range(3)]
    los = [rng.standard_normal((tokens, E)).astype(np.float32) for _ in range(3)]
    # the third input sends every token to experts 0 and 1 only: six experts get no rows at all
    los[2][:, 0], los[2][:, 1], los[2][:, 2:] = 9.0, 8.0, -5.0
    xd, lod = xh.DeviceBuffer.from_numpy(xs[0]), xh.DeviceBuffer.from_numpy(los[0])
    od = xh.DeviceBuffer(xs[0].nbytes)
    eager = []
    for x, lo in zip(xs, los):
        xd.upload(x)
        lod.upload(lo)
        od.zero()
        sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
        xh.synchronize()
        eager.append(od.to_numpy(np.float32, x.shape).copy())
        exp, esel, _ = orc.mixtral_mlp(x, ln, router, experts, lo, rounding="bf16")
        assert np.array_equal(sel, esel) and np.abs(eager[-1] - exp).max() < 2e-2
    assert set(np.unique(orc.moe_top2(los[2])[0])) == {0, 1}
    side = xh.Stream()
    xh.synchronize()
    with xh.Graph(side) as graph:
        got = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr, stream=side.h, want_routing=False)
    assert got == (None, None)
    for i in (2, 0, 1, 2):
        xd.upload(xs[i])
        lod.upload(los[i])
        od.zero()
        xh.synchronize()
        graph.launch()
        side.synchronize()
        assert np.array_equal(od.to_numpy(np.float32, xs[i].shape), eager[i]), i
    graph.free()
    side.free()


def test_graph_helpers_reject_the_null_stream(xh):
    """Capture needs a stream of the caller's own: the null stream and null handles are refused with a message,
    nothing is recorded."""
    import ctypes as C
    assert xh.lib.xfthip_graph_begin(None) != 0
    assert b"null stream" in xh.lib.xfthip_last_error()
    g = C.c_void_p()
    assert xh.lib.xfthip_graph_end(None, C.byref(g)) != 0
    assert xh.lib.xfthip_graph_launch(None, None) != 0
    assert xh.lib.xfthip_graph_destroy(None) == 0


@pytest.mark.parametrize("kind,hidden,inter", [(0, 1056, 1104), (1, 1088, 1168)])
@pytest.mark.parametrize("tokens", [3, 8])
def test_mixtral_mlp_few_tokens_k_not_a_whole_tile(xh, orc, kind, hidden, inter, tokens):
    """Up to 32 tokens with a hidden / intermediate size that is not a whole number of weight tiles along K (64 rows
    for INT8, 128 for the 4-bit kinds): the one-launch form of the few-row GEMM has no K-tail variant, so these
    shapes go expert by expert; every expert's rows must still be multiplied."""
    E = 8
    rng = np.random.default_rng(hidden + tokens)
    experts = _experts(orc, rng, kind, hidden, inter, E)
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32)
    moe = xh.MoE(hidden, inter, E, tokens, np.zeros((hidden, E), np.float32), ln)
    for e, (gu, dn) in enumerate(experts):
        moe.set_expert(e, xh.Weight(kind, gu.K, gu.N, gu.q, gu.scale, gu.zero, flags=xh.WF_GATEUP),
                       xh.Weight(kind, dn.K, dn.N, dn.q, dn.scale, dn.zero))
    xd, lod = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(lo)
    od = xh.DeviceBuffer(x.nbytes)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    exp, esel, ew = orc.mixtral_mlp(x, ln, np.zeros((hidden, E), np.float32), experts, lo, rounding="bf16")
    assert np.array_equal(sel, esel)
    assert len(set(sel.ravel().tolist())) >= 3  # several experts take part
    assert np.abs(got - exp).max() < 2e-2 and _cos(got, exp) >= 0.9999


@pytest.mark.parametrize("tokens", [5, 70])
def test_mixtral_mlp_token_without_two_choices(xh, orc, tokens):
    """Router logits that are NaN (no comparison is true: no expert) or all -inf but one (a single expert): such a
    choice takes no row, as in the reference, whose loop over the experts never matches index -1
    (mlp_mixtral.h:165-186, 262-283); the token keeps its residual plus what its valid choice adds, and the
    other tokens are not disturbed."""
    hidden, inter, E = 512, 1024, 8
    rng = np.random.default_rng(900 + tokens)
    experts = _experts(orc, rng, 0, hidden, inter, E)
    ln = rng.uniform(0.8, 1.2, hidden).astype(np.float32)
    x = orc.round_bf16(rng.standard_normal((tokens, hidden)))
    lo = rng.standard_normal((tokens, E)).astype(np.float32)
    lo[1] = np.nan
    lo[3] = -np.inf
    lo[3, 5] = 0.25
    moe = xh.MoE(hidden, inter, E, tokens, np.zeros((hidden, E), np.float32), ln)
    for e, (gu, dn) in enumerate(experts):
        moe.set_expert(e, xh.Weight(0, gu.K, gu.N, gu.q, gu.scale, gu.zero, flags=xh.WF_GATEUP),
                       xh.Weight(0, dn.K, dn.N, dn.q, dn.scale, dn.zero))
    xd, lod = xh.DeviceBuffer.from_numpy(x), xh.DeviceBuffer.from_numpy(lo)
    od = xh.DeviceBuffer(x.nbytes)
    sel, w = moe.forward(xd.ptr, od.ptr, tokens, True, lod.ptr)
    xh.synchronize()
    got = od.to_numpy(np.float32, x.shape)
    assert list(sel[1]) == [-1, -1] and list(sel[3]) == [5, -1]
    assert np.array_equal(got[1], x[1]), "a token without an expert keeps its input"
    # the well-formed tokens: as the oracle computes them from finite logits
    keep = np.ones(tokens, bool)
    keep[[1, 3]] = False
    lo_ok = lo.copy()
    lo_ok[1] = 0.0
    lo_ok[3] = 0.0
    exp, esel, _ = orc.mixtral_mlp(x, ln, np.zeros((hidden, E), np.float32), experts, lo_ok, rounding="bf16")
    assert np.array_equal(sel[keep], esel[keep])
    assert np.abs(got[keep] - exp[keep]).max() < 2e-2
    # token 3: residual + weight 1 (exp(-inf) = 0 for the missing one) times expert 5 alone
    lo_one = lo_ok.copy()
    lo_one[3] = -40.0
    lo_one[3, 5] = 40.0  # the second choice's weight underflows to 0
    exp1, _, _ = orc.mixtral_mlp(x, ln, np.zeros((hidden, E), np.float32), experts, lo_one, rounding="bf16")
    assert np.isfinite(got[3]).all() and np.abs(got[3] - exp1[3]).max() < 2e-2
