"""GPU parity of the full-size benchmark model: 32 layers of the Llama-2-7B shape, vocabulary
32000, 512-token prompt, 32 greedy decode steps, INT8 and UINT4 weight-only, batch 1 and 32.

Host time is bounded in three ways, none of which changes what the GPU runs: (i) the 32 layers
share ONE set of quantised N(0, 0.02) weight matrices (each layer has its own RMSNorm weights, so
the layers still differ); (ii) the oracle multiplies through numpy's sgemm on the weight
dequantised once (pyoracle gemm="blas", compared with the scalar oracle GEMM in the CPU tests);
(iii) at batch 32 the oracle follows two of the 32 independent sequences.  The oracle narrows
activations to bf16 where the GPU pipeline does, runs its prefill attention at the precision of the
FP16 cache (the reference's route for a prefill over a past; its flash-style route for a first
prefill narrows K, V and the probabilities to bf16, and through 32 randomly initialised layers that
one point alone moves the logits by ~0.2, which the INT8 batch-1 case prints), and is teacher-forced
with the GPU's tokens, so every step is checked against the GPU's own logits of that step:
  * prompt logits: cosine >= 0.9997, max-abs <= 0.15 (|logit| reaches 6);
  * every decode step's logits: max-abs <= 0.2, cosine >= 0.9995 (a step attends over 512 + t cached rows
    that already carry the prompt pass's differences, and the maximum is taken over 32 steps x 32000 (x 2)
    logits instead of one set; measured at worst 0.182 and 0.99966, UINT4 at batch 32 / batch 1);
  * a GPU token that is not the oracle's best must lie within 0.75 x that step's measured max-abs
    logit difference of the oracle's best (in the oracle's logits; measured at worst 0.37): the two
    pipelines then disagree only about a pair they cannot tell apart;
  * at least 70 % of the choices are the oracle's best.  With 32000 logits of unit spread the best two
    of a step lie ~0.2 apart on average and closer than 0.04 in one step of six, and the logits differ
    by ~0.02 rms, so a few of the 33 choices fall on such a pair by chance (measured: 26 to 33 of 33
    between builds that differ only in the rounding order of the prompt pass); the gap rule above is
    what bounds each of them."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HIDDEN, INTER, QH, KVH, D, LAYERS, VOCAB = 4096, 11008, 32, 32, 128, 32, 32000
PROMPT, STEPS = 512, 32
COS_BAR, STEP_COS_BAR, ABS_BAR, STEP_ABS_BAR, GAP_FACTOR, EXACT_SHARE = 0.9997, 0.9995, 0.15, 0.2, 0.75, 0.70


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


@pytest.fixture(scope="module")
def head(orc):
    rng = np.random.default_rng(3)
    emb = orc.to_fp16(rng.standard_normal((VOCAB, HIDDEN), dtype=np.float32) * 0.02)
    lm = orc.round_bf16(rng.standard_normal((HIDDEN, VOCAB), dtype=np.float32) * 0.02)
    fn = np.ones(HIDDEN, np.float32)
    return emb, lm, fn


def _build(xh, orc, head, kind, B_gpu, B_orc, also_flash=False):
    emb, lm, fn = head
    rng = np.random.default_rng(30 + kind)
    shapes = [(HIDDEN, (QH + 2 * KVH) * D), (QH * D, HIDDEN), (HIDDEN, 2 * INTER), (INTER, HIDDEN)]
    ws = [orc.quantize(kind, rng.standard_normal(s, dtype=np.float32) * 0.02) for s in shapes]
    dws = [xh.Weight(kind, w.K, w.N, w.q, w.scale, w.zero, flags=xh.WF_GATEUP if i == 2 else xh.WF_NONE)
           for i, w in enumerate(ws)]
    max_seq = PROMPT + STEPS + 1
    model = xh.Model(LAYERS, HIDDEN, INTER, QH, KVH, D, vocab=VOCAB, max_batch=B_gpu, max_seq=max_seq,
                     max_tokens=B_gpu * PROMPT)
    olayers, flayers = [], []
    for l in range(LAYERS):
        ln1 = rng.uniform(0.9, 1.1, HIDDEN).astype(np.float32)
        ln2 = rng.uniform(0.9, 1.1, HIDDEN).astype(np.float32)
        model.set_layer(l, *dws, ln1, ln2)
        olayers.append(orc.LlamaLayerOracle(HIDDEN, INTER, QH, KVH, D, *ws, ln1, ln2, batch=B_orc, max_seq=max_seq,
                                            rounding="bf16", gemm="blas", prefill_attention="cache"))
        if also_flash:
            flayers.append(orc.LlamaLayerOracle(HIDDEN, INTER, QH, KVH, D, *ws, ln1, ln2, batch=B_orc, max_seq=max_seq,
                                                rounding="bf16", gemm="blas"))
    lmw = xh.Weight(xh.W_BF16, HIDDEN, VOCAB, orc.to_bf16(lm))
    model.set_head(emb, fn, lmw)
    flash = orc.LlamaModelOracle(flayers, emb, fn, lm) if also_flash else None
    return model, orc.LlamaModelOracle(olayers, emb, fn, lm), flash, (dws, lmw)


@pytest.mark.parametrize("kind,B", [(0, 1), (1, 1), (0, 32), (1, 32)])
def test_full_model_greedy_32_steps(xh, orc, head, kind, B):
    print(f"case kind={kind} B={B}", flush=True)
    t0 = time.time()
    follow = [0] if B == 1 else [5, 31]  # sequences of the batch that the oracle follows
    model, ref, flash, keep = _build(xh, orc, head, kind, B, len(follow), also_flash=(kind == 0 and B == 1))
    ids = np.random.default_rng(3).integers(0, VOCAB, (B, PROMPT)).astype(np.int32)
    first, logits = model.prefill(ids, want_logits=True)
    got, glogits = [], []
    for t in range(STEPS):  # one graph replay a step, so that every step's logits can be read
        got.append(model.decode(1, B)[0])
        glogits.append(model.logits(B)[follow].copy())
    assert model.decode_mode() == 1  # replays of the captured decode graph
    t1 = time.time()
    Bo = len(follow)
    elogits, _ = ref.step(ids[follow], Bo, PROMPT, 0)
    err = float(np.abs(logits[follow] - elogits).max())
    cos = _cos(logits[follow], elogits)
    print(f"prefill logits: max-abs {err:.3e} cosine {cos:.6f} (|logit| max {np.abs(elogits).max():.2f})", flush=True)
    # Through 32 randomly initialised layers every bf16 hand-over re-rounds the difference it
    # receives (an intermediate that differs by 5e-5 lands on the neighbouring bf16 value in a few
    # per cent of the elements), so one layer's 5e-3 rms grows to ~2e-2 rms on the logits.
    assert cos >= COS_BAR and err <= ABS_BAR
    if flash is not None:
        flogits, _ = flash.step(ids[follow], Bo, PROMPT, 0)
        print(f"oracle with the flash-style prefill (bf16 K/V/probabilities): differs from the cache-precision oracle by "
              f"{np.abs(flogits - elogits).max():.3e}, from the GPU by {np.abs(flogits - logits[follow]).max():.3e} "
              f"(cosine {_cos(logits[follow], flogits):.6f})", flush=True)
        assert _cos(logits[follow], flogits) >= 0.999

    worst = dict(err=err, cos=cos, gap_ratio=0.0)
    misses = []

    def check(g, gpu_lg, lg, what, cos_bar=STEP_COS_BAR, abs_bar=STEP_ABS_BAR):
        """g: the GPU's tokens; gpu_lg / lg: the GPU's and the oracle's logits of the same step."""
        same = 0
        step_err = float(np.abs(gpu_lg - lg).max())
        step_cos = _cos(gpu_lg, lg)
        worst["err"], worst["cos"] = max(worst["err"], step_err), min(worst["cos"], step_cos)
        assert step_cos >= cos_bar and step_err <= abs_bar, (what, step_cos, step_err)
        for j in range(Bo):
            assert int(g[j]) == int(gpu_lg[j].argmax()), (what, j)  # the device arg-max picked the GPU's own best logit
            best = int(lg[j].argmax())
            gap = float(lg[j, best] - lg[j, g[j]])
            worst["gap_ratio"] = max(worst["gap_ratio"], gap / step_err)
            assert gap <= GAP_FACTOR * step_err, (what, j, int(g[j]), best, gap, step_err)
            same += int(g[j] == best)
            if g[j] != best:
                misses.append((what, j, round(gap, 4), round(step_err, 4)))
        return same

    exact = check(first[follow], logits[follow], elogits, "prompt", COS_BAR, ABS_BAR)
    cur = first[follow]
    for t in range(STEPS):
        elogits, _ = ref.step(cur.reshape(Bo, 1), Bo, 1, PROMPT + t)
        exact += check(got[t][follow], glogits[t], elogits, f"step {t}")
        cur = got[t][follow]
    total = (STEPS + 1) * Bo
    print(f"greedy ids equal to the oracle's best in {exact} of {total} choices; worst step: max-abs {worst['err']:.3e}, cosine "
          f"{worst['cos']:.6f}, gap / max-abs {worst['gap_ratio']:.2f}; gpu {t1 - t0:.1f} s, oracle {time.time() - t1:.1f} s", flush=True)
    print("choices that are not the oracle's best (step, sequence, oracle's gap, step max-abs):", misses, flush=True)
    assert exact >= EXACT_SHARE * total
    orc.clear_blas_cache()
    model.free()
