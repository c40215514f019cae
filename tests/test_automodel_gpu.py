"""xft::AutoModel on the GPU: a model directory in the reference's on-disk format (written by
tests/golden/make_llama_fixture.py) is loaded, and generation through the reference's loop
(config / input / generate until isDone / finalize, src/models/models.cpp:99-135, 834-846) must give
  * exactly the ids of a device model built directly from the same arrays (which pins the loader:
    file names, shapes, element types, the Q|K|V and gate|up concatenations, the lm_head transpose),
  * prompt logits within the layer tolerance of the CPU oracle fed the same weights,
and the searchers must behave as GreedySearch / SampleSearch do (src/searchers/greedy_search.cpp:78-134,
270-287, sample_search.cpp, search_utils.cpp:22-99): EOS then padding, stop words, repetition penalty."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

KIND = {"int8": 0, "int4": 1, "nf4": 2, "w8a8": 3, "bf16": 4, "fp16": 4}


@pytest.fixture(scope="module")
def xh():
    from xfastertransformer_amd import capi
    capi.init()
    return capi


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


@pytest.fixture(scope="module")
def am():
    from xfastertransformer_amd import automodel
    return automodel


def _device_weight(xh, orc, held, kind, flags=0):
    """(device weight, oracle weight) of one matrix: pre-quantised codes as they are when the
    requested kind is the files' own, else quantised from the fp32 values the files hold."""
    w = held["w"]
    K, N = w.shape
    if kind == xh.W_BF16:
        return xh.Weight(kind, K, N, orc.to_bf16(w), flags=flags), orc.round_bf16(w)
    if "q" in held and ((kind == xh.W_INT8 and held["q"].dtype == np.int8) or (kind == xh.W_UINT4 and held["q"].dtype == np.uint8)):
        q = held["q"] if kind == xh.W_INT8 else (held["q"][:, 0::2] | (held["q"][:, 1::2] << 4)).astype(np.uint8)
        return xh.Weight(kind, K, N, q, held["scale"], held["zero"], flags=flags), orc.QWeight(kind, K, N, q, held["scale"], held["zero"])
    q, s, z = xh.quantize_weight(kind, w)
    ow = orc.QWeight(kind, K, N, q, s, z)
    if kind == xh.W_W8A8:
        ow = orc.quantize(kind, w)
        assert np.array_equal(ow.q, q.view(np.int8).reshape(K, N))
    return xh.Weight(kind, K, N, q, s, z, flags=flags), ow


def _cat(a, b):
    out = {"w": np.concatenate([a["w"], b["w"]], 1)}
    if "q" in a:
        out.update(q=np.concatenate([a["q"], b["q"]], 1), scale=np.concatenate([a["scale"], b["scale"]]),
                   zero=np.concatenate([a["zero"], b["zero"]]))
    return out


def _direct(xh, orc, held, dtype, kv, B, max_seq, with_oracle=True):
    c = held["cfg"]
    kind = KIND[dtype]
    model = xh.Model(c["layers"], c["hidden"], c["inter"], c["heads"], c["kv_heads"], c["head"], vocab=c["vocab"], max_batch=B,
                     max_seq=max_seq, max_tokens=B * max_seq, max_pos_embed=c["max_pos"], rope_base=int(c["rope_theta"]),
                     kv_dtype=xh.INT8 if kv == "int8" else xh.FP16, rms_eps=c["eps"])
    olayers = []
    for l, lay in enumerate(held["layers"]):
        pairs = [_device_weight(xh, orc, lay["qkv"], kind), _device_weight(xh, orc, lay["o"], kind),
                 _device_weight(xh, orc, _cat(lay["gate"], lay["up"]), kind, 0 if kind == xh.W_W8A8 else xh.WF_GATEUP),
                 _device_weight(xh, orc, lay["down"], kind)]
        model.set_layer(l, *[p[0] for p in pairs], lay["ln1"], lay["ln2"])
        if with_oracle and kind in (0, 1, 2):
            olayers.append(orc.LlamaLayerOracle(c["hidden"], c["inter"], c["heads"], c["kv_heads"], c["head"], *[p[1] for p in pairs],
                                                lay["ln1"], lay["ln2"], kv_int8=int(kv == "int8"), batch=B, max_seq=max_seq,
                                                eps=c["eps"], rope_base=int(c["rope_theta"]), max_pos=c["max_pos"], rounding="bf16",
                                                prefill_attention="cache"))
    emb = orc.to_fp16(held["wte"])
    lm = orc.round_bf16(np.ascontiguousarray(held["lm_head"].T))
    model.set_head(emb, held["final_norm"], xh.Weight(xh.W_BF16, c["hidden"], c["vocab"], orc.to_bf16(lm)))
    ref = orc.LlamaModelOracle(olayers, emb, held["final_norm"], lm) if olayers else None
    return model, ref


CASES = [("fp32", None, "int8", "fp16"), ("fp16", None, "bf16", "fp16"), ("bf16", None, "int4", "int8"),
         ("fp32", "int8", "int8", "fp16"), ("fp32", "uint4", "int4", "fp16"), ("fp32", None, "nf4", "fp16"),
         ("fp32", None, "w8a8", "fp16"), ("fp32", "int8", "bf16", "fp16"), ("fp32", None, "fp16", "fp16")]


@pytest.mark.parametrize("weight_type,quant,dtype,kv", CASES)
def test_loaded_model_generates_what_the_directly_built_model_does(xh, orc, am, tmp_path, weight_type, quant, dtype, kv):
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 3, weight_type, quant)
    B, S, max_len = 2, 10, 26
    ids = np.random.default_rng(5).integers(0, held["cfg"]["vocab"], (B, S)).astype(np.int32)
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype=dtype, kv_cache_dtype=kv)
    assert model.vocab_size == held["cfg"]["vocab"] and model.max_seq_len == held["cfg"]["max_pos"]
    out = model.generate(ids, max_length=max_len)
    assert out.shape == (B, max_len) and np.array_equal(out[:, :S], ids)
    direct, ref = _direct(xh, orc, held, dtype, kv, B, max_len)
    first, logits = direct.prefill(ids, want_logits=True)
    rest = direct.decode(max_len - S - 1, B)
    expect = np.concatenate([ids, first.reshape(B, 1), rest.T], 1)
    assert np.array_equal(out, expect)
    # Model::forward(false): the prompt's logits, equal to the direct model's and near the oracle's
    model.input(ids)
    got = model.logits()
    assert np.array_equal(got, logits)
    if ref is not None:
        elogits, _ = ref.step(ids, B, S, 0)
        err = float(np.abs(got - elogits).max())
        print(f"{weight_type}/{quant}/{dtype}/{kv}: prompt logits max-abs error vs oracle {err:.3e}", flush=True)
        assert err < 3e-2  # bf16 hand-over points between layers: see the layer tests for the per-stage bars
    model.free()


def test_torch_tensors_in_and_out(am, tmp_path):
    import torch
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 4)
    ids = torch.randint(0, held["cfg"]["vocab"], (1, 7), generator=torch.Generator().manual_seed(1))
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8")
    out = model.generate(ids, max_length=12)
    assert isinstance(out, torch.Tensor) and out.dtype == torch.int64 and tuple(out.shape) == (1, 12)
    assert torch.equal(out[:, :7], ids)
    model.free()


def test_eos_padding_stop_words_and_early_finish(am, tmp_path):
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 6)
    B, S, max_len = 2, 8, 30
    ids = np.random.default_rng(8).integers(0, held["cfg"]["vocab"], (B, S)).astype(np.int32)
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8")
    # an EOS id the model never emits here (the default would be config.ini's end_id)
    free_run = model.generate(ids, max_length=max_len, eos_token_id=497)
    assert 497 not in free_run[:, S:]
    # EOS: the token sequence 0 emits at step 3 ends it there; the rest of its row is padding
    # (greedy_search.cpp:270-281) and the other sequence is untouched
    eos, pad = int(free_run[0, S + 3]), 499
    assert eos not in free_run[0, S:S + 3] and eos not in free_run[1, S:]
    out = model.generate(ids, max_length=max_len, eos_token_id=eos, pad_token_id=pad)
    assert np.array_equal(out[0, :S + 4], free_run[0, :S + 4]) and np.all(out[0, S + 4:] == pad)
    assert np.array_equal(out[1], free_run[1])
    # pad defaults to EOS; with every sequence finished the loop ends before max_length (isDone)
    out = model.generate(ids[:1], max_length=max_len, eos_token_id=eos)
    assert out.shape == (1, S + 4) and out[0, -1] == eos
    # stop word of two tokens: the step after it is forced to EOS, then padding (search_utils.cpp:77-99)
    stop = [int(free_run[1, S + 5]), int(free_run[1, S + 6])]
    eos2 = 498
    out = model.generate(ids, max_length=max_len, eos_token_id=eos2, pad_token_id=pad, stop_words_ids=[stop])
    first = next(t for t in range(S + 1, max_len) if list(free_run[1, t - 1:t + 1]) == stop and t - 1 >= S)
    assert np.array_equal(out[1, :first + 1], free_run[1, :first + 1])
    assert out[1, first + 1] == eos2 and np.all(out[1, first + 2:] == pad)
    # max_length no longer than the prompt: one token is still produced, as in the reference
    out = model.generate(ids, max_length=S, eos_token_id=497)
    assert out.shape == (B, S + 1) and np.array_equal(out, free_run[:, :S + 1])
    model.free()


def test_repetition_penalty_and_sampling(xh, orc, am, tmp_path, monkeypatch):
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 9)
    B, S, max_len, pen = 2, 9, 24, 1.7
    V = held["cfg"]["vocab"]
    ids = np.random.default_rng(10).integers(0, V, (B, S)).astype(np.int32)
    monkeypatch.setenv("XFT_SEED", "1234")
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8")
    never = dict(eos_token_id=V + 7)  # no id ends a sequence in this test
    greedy = model.generate(ids, max_length=max_len, **never)
    out = model.generate(ids, max_length=max_len, repetition_penalty=pen, **never)
    assert not np.array_equal(out, greedy)
    # the same loop by hand on the directly built model: penalise every id seen so far, first maximum
    direct, _ = _direct(xh, orc, held, "int8", "fp16", B, max_len, with_oracle=False)
    direct.prefill(ids)
    seq = ids.copy()
    for t in range(max_len - S):
        lg = direct.logits(B)
        for b in range(B):
            seen = np.unique(seq[b])
            lg[b, seen] = np.where(lg[b, seen] < 0, lg[b, seen] * np.float32(pen), lg[b, seen] / np.float32(pen))
        nxt = lg.argmax(1).astype(np.int32)
        seq = np.concatenate([seq, nxt[:, None]], 1)
        if t + 1 < max_len - S:
            direct.set_next_ids(nxt)
            direct.decode(1, B)
    assert np.array_equal(out, seq)
    def replay(tokens, check):
        """feeds `tokens` to the directly built model and hands every step's logits to check(b, t, logits)"""
        direct.prefill(ids)
        for t in range(max_len - S):
            lg = direct.logits(B)
            for b in range(B):
                check(b, t, lg[b])
            if t + 1 < max_len - S:
                direct.set_next_ids(tokens[:, S + t])
                direct.decode(1, B)

    # sampling at a temperature that leaves the best token (or a tie within 0.02 of it) all the probability
    out = model.generate(ids, max_length=max_len, do_sample=True, temperature=1e-3, top_k=5, **never)

    def near_best(b, t, lg):
        assert lg[out[b, S + t]] >= lg.max() - 2e-2, (b, t)
    replay(out, near_best)
    # at temperature 1 every drawn token is one of the top-k of the logits the direct model has for
    # the same history
    a = model.generate(ids, max_length=max_len, do_sample=True, top_k=4, top_p=0.95, **never)

    def in_candidates(b, t, lg):
        cand, _ = am.sample_candidates(lg, 4, 0.95, 1.0)
        assert a[b, S + t] in cand, (b, t)
    replay(a, in_candidates)
    assert not np.array_equal(a, greedy)
    model.free()


def test_continuous_batching_through_the_model_class(am, tmp_path):
    """Model::set_input / generate / freeSeqs (models.cpp:278-410, 847-903): ragged prompts, sequences that
    sit out steps, an early free and a late joiner each reproduce their own lockstep run."""
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 12)
    V = held["cfg"]["vocab"]
    rng = np.random.default_rng(13)
    prompts = [rng.integers(0, V, n).astype(np.int32) for n in (6, 19, 11, 4)]
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8")
    never = V + 3
    solo = [model.generate(p[None, :], max_length=len(p) + 12, eos_token_id=never)[0] for p in prompts]
    pen = [model.generate(p[None, :], max_length=len(p) + 12, eos_token_id=never, repetition_penalty=1.5)[0] for p in prompts]

    ids = model.set_input_cb([prompts[0], prompts[1], prompts[2]], max_length=40, eos_token_id=never)
    assert len(ids) == 3 and len(set(ids)) == 3
    got = {i: [] for i in ids}
    for i, t in zip(ids, model.forward_cb()):  # the prompts
        got[i].append(t)
    for step in range(3):
        model.set_input_cb(seq_ids=ids, max_length=40, eos_token_id=never)
        for i, t in zip(ids, model.forward_cb()):
            got[i].append(t)
    # only two of them step; then the first one is freed and a new sequence takes a row
    for step in range(2):
        model.set_input_cb(seq_ids=ids[1:], max_length=40, eos_token_id=never)
        for i, t in zip(ids[1:], model.forward_cb()):
            got[i].append(t)
    assert model.free_seqs(ids[:1]) and not model.free_seqs(ids[:1])
    late = model.set_input_cb([prompts[3]], max_length=40, eos_token_id=never)
    got[late[0]] = list(model.forward_cb())
    everyone = ids[1:] + late
    for step in range(5):
        model.set_input_cb(seq_ids=everyone, max_length=40, eos_token_id=never)
        for i, t in zip(everyone, model.forward_cb()):
            got[i].append(t)
    for k, i in enumerate(ids + late):
        n = len(got[i])
        assert n >= 4 and got[i] == solo[k][len(prompts[k]):len(prompts[k]) + n].tolist(), (k, got[i], solo[k])
    # finalize returns prompt + generated of the working sequences and frees them
    model.set_input_cb(seq_ids=everyone, max_length=40, eos_token_id=never)
    flat = model.finalize().ravel().tolist()
    expect = []
    for k, i in zip((1, 2, 3), everyone):
        expect += prompts[k].tolist() + got[i]
    assert flat == expect
    assert not model.free_seqs(everyone)  # already gone
    # EOS and maxLen end a sequence (sampling.cpp:134-154), repetition penalty as on the lockstep path
    eos = int(solo[0][len(prompts[0]) + 3])
    assert eos not in solo[0][len(prompts[0]):len(prompts[0]) + 3]
    a = model.set_input_cb([prompts[0]], max_length=40, eos_token_id=eos)
    toks = list(model.forward_cb())
    while not model.is_done():
        model.set_input_cb(seq_ids=a, max_length=40, eos_token_id=eos)
        toks += model.forward_cb()
    assert toks == solo[0][len(prompts[0]):len(prompts[0]) + 4].tolist()
    model.free_seqs(a)
    b = model.set_input_cb([prompts[1], prompts[2]], max_length=len(prompts[1]) + 5, eos_token_id=never, repetition_penalty=1.5)
    out = {i: [t] for i, t in zip(b, model.forward_cb())}
    while not model.is_done():
        model.set_input_cb(seq_ids=b, max_length=len(prompts[1]) + 5, eos_token_id=never, repetition_penalty=1.5)
        for i, t in zip(b, model.forward_cb()):
            out[i].append(t)
    # the longer prompt is done with the token that brings it to maxLen (5 new ones) and emits EOS from then
    # on, the shorter one goes on to its own limit
    assert out[b[0]][:5] == pen[1][len(prompts[1]):len(prompts[1]) + 5].tolist() and all(t == never for t in out[b[0]][5:])
    assert len(out[b[1]]) == 13 and out[b[1]][:12] == pen[2][len(prompts[2]):len(prompts[2]) + 12].tolist()
    model.free()


@pytest.mark.parametrize("kv", ["fp16", "int8"])
def test_beam_search_through_the_model_class(xh, orc, am, tmp_path, kv):
    """numBeams > 1 (BeamSearch, src/searchers/beam_search.cpp): every step's tokens and the final hypotheses must
    be those of the pinned restatement of the searcher fed with the logits the directly built device model has
    for each beam row's token history (recomputed from scratch - the prompt, then one decode step per generated
    token, so the cache copies and re-mappings behind Model::generate are what is under test).  The EOS id is the first sequence's most likely first token, so a
    hypothesis closes in the first step; two hypotheses are returned per sequence."""
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 11)
    B, S, nb, keep, max_len = 2, 6, 3, 2, 15
    V = held["cfg"]["vocab"]
    ids = np.random.default_rng(12).integers(0, V, (B, S)).astype(np.int32)
    direct, _ = _direct(xh, orc, held, "int8", kv, B * nb, max_len, with_oracle=False)
    _, lg0 = direct.prefill(np.repeat(ids, nb, 0), want_logits=True)
    eos, pad = int(lg0[0].argmax()), 1
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8", kv_cache_dtype=kv)
    model.config(max_length=max_len, num_beams=nb, num_return_sequences=keep, eos_token_id=eos, pad_token_id=pad)
    model.input(ids)
    ref = orc.BeamSearchOracle(ids, nb, max_len, eos, pad, V, keep=keep)
    steps = 0
    while not ref.is_done():
        assert not model.is_done()
        hist = np.asarray(ref.rows, np.int32)
        _, lg = direct.prefill(hist[:, :S], want_logits=True)
        for t in range(S, hist.shape[1]):
            direct.set_next_ids(hist[:, t])
            direct.decode(1, B * nb)
            lg = direct.logits(B * nb)
        want, _ = ref.step(lg)
        got = model.forward().ravel().tolist()
        assert got == want, (steps, got, want)
        steps += 1
    assert model.is_done() and steps >= 3
    out = model.finalize()
    exp = ref.finalize()
    assert out.shape == exp.shape == (B * keep, exp.shape[1]) and np.array_equal(out, exp)
    assert len(ref.hyps[0]) >= 1 and ref.hyps[0][0][1] == ids[0].tolist() or any(h[1] == ids[0].tolist() for h in ref.hyps[0])
    # the one-call form gives the same
    again = model.generate(ids, max_length=max_len, num_beams=nb, num_return_sequences=keep, eos_token_id=eos, pad_token_id=pad)
    assert np.array_equal(again, exp)
    # and greedy search still works on the same object afterwards
    g = model.generate(ids, max_length=S + 4, eos_token_id=V + 3)
    assert g.shape == (B, S + 4)
    model.free()


def _layer_sets(xh, orc, held, kind):
    sets = []
    for lay in held["layers"]:
        sets.append([_device_weight(xh, orc, lay["qkv"], kind)[0], _device_weight(xh, orc, lay["o"], kind)[0],
                     _device_weight(xh, orc, _cat(lay["gate"], lay["up"]), kind, 0 if kind == xh.W_W8A8 else xh.WF_GATEUP)[0],
                     _device_weight(xh, orc, lay["down"], kind)[0]])
    return sets


@pytest.mark.parametrize("dtype", ["bf16_int8", "w8a8_int4", "bf16_nf4"])
def test_first_token_and_next_token_weight_types(xh, orc, am, tmp_path, dtype):
    """The mixed types (HybridModel, src/models/hybrid_model.h:25-84): the prompt runs on the first type's
    weights, every later token on the second type's, over one KV cache.  Checked against a model that is
    switched by hand: built with the first type, prompt run, then its layers replaced by the second type's
    weights (the cache stays) and decoded; the prompt's logits must be the first type's own."""
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 21)
    first, nxt = dtype.split("_")
    B, S, max_len = 2, 9, 20
    V = held["cfg"]["vocab"]
    ids = np.random.default_rng(22).integers(0, V, (B, S)).astype(np.int32)
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype=dtype)
    out = model.generate(ids, max_length=max_len, eos_token_id=V + 5)
    model.input(ids)
    prompt_logits = model.logits()
    # by hand
    hand, _ = _direct(xh, orc, held, first, "fp16", B, max_len, with_oracle=False)
    tok0, lg0 = hand.prefill(ids, want_logits=True)
    assert np.array_equal(prompt_logits, lg0)
    for l, ws in enumerate(_layer_sets(xh, orc, held, KIND[nxt])):
        hand.set_layer(l, *ws, held["layers"][l]["ln1"], held["layers"][l]["ln2"])
    rest = hand.decode(max_len - S - 1, B)
    expect = np.concatenate([ids, tok0.reshape(B, 1), rest.T], 1)
    assert np.array_equal(out, expect)
    # and it differs from both pure types somewhere (the test would not notice a silent single-type model otherwise)
    pure = [am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype=t).generate(ids, max_length=max_len, eos_token_id=V + 5)
            for t in (first, nxt)]
    print(f"{dtype}: equal to pure {first}: {np.array_equal(out, pure[0])}, to pure {nxt}: {np.array_equal(out, pure[1])}", flush=True)
    model.free()


def test_every_set_input_overload_through_the_cpp_api(am, tmp_path):
    """tests/set_input_driver.cpp (built with the libraries) calls all nine Model::set_input overloads of
    include/models.h, generate(), forward(false / true) and freeSeqs the way a program written against the
    reference's header does (include/models.h:40-73, src/models/models.cpp:238-683) and checks that every
    sequence continues as it does alone.  Here: it must pass, and its lockstep ids must be the ones the
    Python face gets for the same prompts."""
    import subprocess
    import make_llama_fixture as fx
    driver = os.path.join(ROOT, "xfastertransformer_amd", "csrc", "build", "set_input_driver")
    assert os.path.exists(driver), "tests/set_input_driver.cpp is not built; run `python -m xfastertransformer_amd.build`"
    held = fx.write_model_dir(str(tmp_path / "model"), None, 31)
    V = held["cfg"]["vocab"]
    run = subprocess.run([driver, str(tmp_path / "model"), "int8", str(V)], capture_output=True, text=True, timeout=300)
    print(run.stdout[-3000:], run.stderr[-2000:], flush=True)
    assert run.returncode == 0 and "PASSED" in run.stdout and "FAIL" not in run.stdout.replace("FAILED", "")
    alone = [[int(t) for t in line.split()[1:]] for line in run.stdout.splitlines() if line.startswith("ALONE")]
    assert len(alone) == 3 and all(len(a) == 6 for a in alone)

    def prompt_of(n, salt):  # the driver's generator (xorshift64)
        s = (88172645463325252 + salt * 7919) & (2 ** 64 - 1)
        out = []
        for _ in range(n):
            s ^= (s << 13) & (2 ** 64 - 1)
            s ^= s >> 7
            s ^= (s << 17) & (2 ** 64 - 1)
            out.append(s % V)
        return np.asarray(out, np.int32)

    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8")
    for k, (n, salt) in enumerate(((7, 1), (7, 2), (12, 3))):
        p = prompt_of(n, salt)
        out = model.generate(p[None, :], max_length=n + 6, eos_token_id=V + 5)
        assert out[0, n:].tolist() == alone[k], (k, out[0, n:].tolist(), alone[k])
    model.free()
