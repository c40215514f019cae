"""Continuous batching in the model driver (xfthip_model_seq_*): sequences of different prompt
lengths enter cache rows of their own, step in changing subsets, end and hand their row to a new
sequence; every sequence must produce what it produces when it runs alone (same kernels, so the
logits agree to fp32 summation order and the greedy ids are the same).  Stands in for
CommonDecoder::forward(seqs) over the reference's per-sequence KV caches
(src/models/common_decoder.h, src/common/kvcache_mgr.h:37-194, src/layers/attention.h:501-730)."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init()
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def _alone(model, prompt, steps):
    """ids and logits of one sequence run by itself (batch 1, lockstep API)."""
    first, logits = model.prefill(np.asarray(prompt, np.int32)[None, :], want_logits=True)
    ids, lg = [int(first[0])], [logits[0].copy()]
    for _ in range(steps):
        ids.append(int(model.decode(1, 1)[0, 0]))
        lg.append(model.logits(1)[0].copy())
    return ids, lg


@pytest.mark.parametrize("kind,kv", [(0, "fp16"), (1, "fp16"), (0, "int8")])
def test_sequences_come_and_go(xh, orc, kind, kv):
    from test_layer_model_gpu import make_layer_weights, to_device_weights
    layers, hidden, inter, qh, kvh, D, vocab, rows, max_seq = 2, 512, 1408, 4, 2, 128, 1000, 6, 160
    rng = np.random.default_rng(91)
    model = xh.Model(layers, hidden, inter, qh, kvh, D, vocab=vocab, max_batch=rows, max_seq=max_seq, max_tokens=rows * max_seq,
                     kv_dtype=xh.INT8 if kv == "int8" else xh.FP16)
    for l in range(layers):
        ws = make_layer_weights(orc, rng, kind, hidden, inter, qh, kvh, D)
        model.set_layer(l, *to_device_weights(xh, ws, kind), rng.uniform(0.8, 1.2, hidden).astype(np.float32),
                        rng.uniform(0.8, 1.2, hidden).astype(np.float32))
    lm = orc.round_bf16(rng.standard_normal((hidden, vocab)) * 0.05)
    model.set_head(orc.to_fp16(rng.standard_normal((vocab, hidden)) * 0.5), rng.uniform(0.8, 1.2, hidden).astype(np.float32),
                   xh.Weight(xh.W_BF16, hidden, vocab, orc.to_bf16(lm)))
    prompts = {name: rng.integers(0, vocab, n).tolist() for name, n in (("a", 9), ("b", 30), ("c", 17), ("d", 5), ("e", 64))}
    steps = 24
    alone = {name: _alone(model, p, steps) for name, p in prompts.items()}

    # the schedule: a, b, c start; b sits out some steps; a ends early and d takes its row; e joins in a high row
    got = {name: [] for name in prompts}
    lg = {name: [] for name in prompts}
    row = {"a": 0, "b": 1, "c": 2}

    def start(name, r):
        row[name] = r
        logits = model.seq_prefill(r, prompts[name], want_logits=True)
        got[name].append(int(model.last_ids(rows)[r]))
        lg[name].append(logits)

    def step(names):
        rr = [row[n] for n in names]
        ids = model.seq_decode(rr)
        for n, t in zip(names, ids):
            got[n].append(int(t))
            lg[n].append(model.seq_logits(row[n]))

    for n in ("a", "b", "c"):
        start(n, row[n])
    for t in range(4):
        step(["a", "b", "c"])
    for t in range(3):
        step(["a", "c"])  # b waits
    step(["b"])
    model.seq_release(row["a"])  # a ends after 8 tokens
    start("d", 0)  # and d takes over its row
    start("e", 5)
    for t in range(10):
        step(["b", "c", "d", "e"])
    model.seq_release(row["c"])
    for t in range(6):
        step(["e", "d", "b"])
    checked = 0
    for name in prompts:
        ref_ids, ref_lg = alone[name]
        n = len(got[name])
        assert n >= 8
        assert got[name] == ref_ids[:n], (name, got[name], ref_ids[:n])
        for i in range(n):
            # the batch changes the attention's split count, hence the fp32 merge order; a bf16 hand-over
            # point that rounds the other way moves a logit by a few 1e-3
            err = float(np.abs(lg[name][i] - ref_lg[i]).max())
            assert err < 2e-2, (name, i, err)
            checked += 1
    print(f"{checked} steps of 5 sequences equal to their solo runs ({kind=}, {kv=})", flush=True)
    # the lockstep API still works afterwards and resets the rows
    first, _ = model.prefill(np.asarray(prompts["b"], np.int32)[None, :])
    assert int(first[0]) == alone["b"][0][0]


@pytest.mark.parametrize("kv", ["fp16", "int8"])
def test_cache_rows_copied_and_reordered_for_beams(xh, orc, kv):
    """xfthip_model_seq_reorder, the device half of KVCacheTensor::expandAllSequence / ::reorder
    (src/common/kvcache_tensor.h:147-286): three prompts run in rows 0, 2, 4, every row is copied to its
    neighbour (two beams), forced tokens are fed to all six rows, and three times the rows are re-mapped
    the way a beam searcher does (a row may be read and overwritten in the same call).  Every row must then
    produce the logits of its own token history run alone."""
    from test_layer_model_gpu import make_layer_weights, to_device_weights
    layers, hidden, inter, qh, kvh, D, vocab, rows, max_seq = 2, 512, 1408, 4, 2, 128, 1000, 6, 96
    rng = np.random.default_rng(123)
    model = xh.Model(layers, hidden, inter, qh, kvh, D, vocab=vocab, max_batch=rows, max_seq=max_seq, max_tokens=rows * max_seq,
                     kv_dtype=xh.INT8 if kv == "int8" else xh.FP16)
    for l in range(layers):
        ws = make_layer_weights(orc, rng, 0, hidden, inter, qh, kvh, D)
        model.set_layer(l, *to_device_weights(xh, ws, 0), rng.uniform(0.8, 1.2, hidden).astype(np.float32),
                        rng.uniform(0.8, 1.2, hidden).astype(np.float32))
    lm = orc.round_bf16(rng.standard_normal((hidden, vocab)) * 0.05)
    model.set_head(orc.to_fp16(rng.standard_normal((vocab, hidden)) * 0.5), rng.uniform(0.8, 1.2, hidden).astype(np.float32),
                   xh.Weight(xh.W_BF16, hidden, vocab, orc.to_bf16(lm)))
    S, steps = 20, 18  # the generated part crosses the 32-token block boundary
    prompts = [rng.integers(0, vocab, S).tolist() for _ in range(3)]
    toks = rng.integers(0, vocab, (steps, rows))
    remaps = {3: [1, 1, 2, 3, 5, 4], 9: [0, 0, 3, 2, 5, 5], 14: [1, 0, 2, 2, 4, 5]}
    # the plan on the host: which history every row ends with
    hist = [list(prompts[r // 2]) for r in range(rows)]
    for k in range(steps):
        if k in remaps:
            hist = [list(hist[s]) for s in remaps[k]]
        for r in range(rows):
            hist[r].append(int(toks[k, r]))
    want = []
    for r in range(rows):  # each history alone, lockstep interface
        model.prefill(np.asarray(hist[r][:S], np.int32)[None, :])
        for t in hist[r][S:]:
            model.set_next_ids([t])
            model.decode(1, 1)
        want.append(model.logits(1)[0].copy())
    # the same through cache rows
    for b in range(3):
        model.seq_prefill(2 * b, prompts[b])
    model.seq_reorder([1, 3, 5], [0, 2, 4], 0, S)
    for k in range(steps):
        if k in remaps:
            model.seq_reorder(list(range(rows)), remaps[k], S, S + k)
        for r in range(rows):
            model.seq_set_next_id(r, int(toks[k, r]))
        model.seq_decode(list(range(rows)))
    for r in range(rows):
        got = model.seq_logits(r)
        err = float(np.abs(got - want[r]).max())
        assert err < 2e-2, (r, err)
    print(f"six rows agree with their solo runs after three re-mappings ({kv=})", flush=True)


def test_lockstep_and_per_sequence_decode_alternate_at_one_batch(xh, orc):
    """The captured decode step differs between the two modes (the per-sequence one carries the mask of
    the rows that sit out), so a change of mode at an unchanged batch, stream and split count must not
    replay the other mode's step: a subset decode that leaves a zero in the mask, then a lockstep
    prompt + decode at the same batch, and the reverse order, each compared with a fresh model."""
    from test_layer_model_gpu import make_layer_weights, to_device_weights
    layers, hidden, inter, qh, kvh, D, vocab, rows, max_seq = 2, 512, 1408, 4, 2, 128, 1000, 2, 96

    def build():
        rng = np.random.default_rng(77)
        model = xh.Model(layers, hidden, inter, qh, kvh, D, vocab=vocab, max_batch=rows, max_seq=max_seq, max_tokens=rows * max_seq)
        for l in range(layers):
            ws = make_layer_weights(orc, rng, 0, hidden, inter, qh, kvh, D)
            model.set_layer(l, *to_device_weights(xh, ws, 0), rng.uniform(0.8, 1.2, hidden).astype(np.float32),
                            rng.uniform(0.8, 1.2, hidden).astype(np.float32))
        lm = orc.round_bf16(rng.standard_normal((hidden, vocab)) * 0.05)
        model.set_head(orc.to_fp16(rng.standard_normal((vocab, hidden)) * 0.5), rng.uniform(0.8, 1.2, hidden).astype(np.float32),
                       xh.Weight(xh.W_BF16, hidden, vocab, orc.to_bf16(lm)))
        return model

    rng = np.random.default_rng(5)
    pa, pb = rng.integers(0, vocab, 11).tolist(), rng.integers(0, vocab, 11).tolist()
    both = np.asarray([pa, pb], np.int32)
    steps = 6

    def lockstep(model):
        first, _ = model.prefill(both)
        out = model.decode(steps, 2)
        return [int(first[0]), int(first[1])], out.tolist()

    def per_sequence(model):
        model.seq_prefill(0, pa)
        model.seq_prefill(1, pb)
        ids = [[int(t) for t in model.last_ids(2)]]
        for _ in range(2):
            ids.append([int(t) for t in model.seq_decode([0, 1])])
        only_b = [int(model.seq_decode([1])[0]) for _ in range(3)]  # row 0 sits out: the mask ends as [0, 1]
        return ids, only_b

    want_lock = lockstep(build())
    want_seq = per_sequence(build())
    # (in the per-sequence run row 0 must stay where it was while it sat out)
    m = build()
    assert per_sequence(m) == want_seq
    assert lockstep(m) == want_lock, "a lockstep decode replayed the masked step of the per-sequence mode"
    assert per_sequence(m) == want_seq, "a per-sequence decode replayed the unmasked lockstep step"
    m2 = build()
    assert lockstep(m2) == want_lock
    got_ids, got_b = per_sequence(m2)
    assert (got_ids, got_b) == want_seq
    # row 0 sat out three steps: stepping it now continues from its own position
    a_next = int(m2.seq_decode([0])[0])
    fresh = build()
    fresh.seq_prefill(0, pa)
    solo = [int(fresh.seq_decode([0])[0]) for _ in range(3)]
    assert a_next == solo[2], (a_next, solo)
