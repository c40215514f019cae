"""Beam search, host half (CPU only): the restatement in oracle/pyoracle.py against brute force, and the
library's BeamSearcher (the C++ behind Model::generate for numBeams > 1) against the restatement on the same
logits.  Follows src/searchers/beam_search.cpp of the reference."""
import itertools

import numpy as np
import pytest

from oracle import pyoracle as orc


def toy_lm(history, vocab, seed):
    """Deterministic logits of the next token given a token history."""
    h = seed
    for t in history[-3:]:
        h = (h * 1000003 + int(t) + 17) % (2 ** 31 - 1)
    return np.random.default_rng(h).standard_normal(vocab).astype(np.float32) * 2.0


def log_softmax(x):
    x = x.astype(np.float64)
    return x - (x.max() + np.log(np.exp(x - x.max()).sum()))


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5])
def test_oracle_beam_search_is_exhaustive_with_enough_beams(seed):
    """With vocab ** (steps - 1) beams no prefix is ever dropped, so the best hypothesis must be the best of all
    vocab ** steps continuations under the sum of log-probabilities (no EOS in play: equal lengths)."""
    vocab, steps, prompt = 3, 3, [1, 0, 2, 1]
    nb = vocab ** (steps - 1)
    best, best_score = None, -1e30
    for cont in itertools.product(range(vocab), repeat=steps):
        hist, score = list(prompt), 0.0
        for t in cont:
            score += log_softmax(toy_lm(hist, vocab, seed))[t]
            hist.append(t)
        if score > best_score:
            best, best_score = list(cont), score
    bs = orc.BeamSearchOracle([prompt], nb, len(prompt) + steps, eos=-1, pad=0, vocab=vocab)
    while not bs.is_done():
        bs.step(np.stack([toy_lm(r, vocab, seed) for r in bs.rows]))
    out = bs.finalize()
    assert out.shape == (1, len(prompt) + steps)
    assert out[0].tolist() == prompt + best
    # and the kept score is that sum (length penalty 1: divided by the length)
    top = max(bs.hyps[0], key=lambda h: h[0])
    assert abs(top[0] * (len(prompt) + steps) - best_score) < 1e-4


def test_oracle_beam_search_eos_bookkeeping():
    """EOS among the best numBeams candidates closes a hypothesis (score = sum / length ** penalty over the ids
    WITHOUT the EOS), EOS ranked lower is skipped, a finished user sequence feeds the pad token from row 0, and
    the output row is hypothesis + EOS + padding."""
    vocab, eos, pad, prompt = 5, 4, 3, [2, 2]
    # step 1: EOS is the best token; tokens 0 and 1 follow
    l1 = np.array([2.0, 1.0, -5.0, -5.0, 3.0], np.float32)
    bs = orc.BeamSearchOracle([prompt], 2, 6, eos, pad, vocab, len_penalty=1.0, early=True)
    toks, idx = bs.step(np.stack([l1, l1]))
    assert toks == [0, 1] and idx == [0, 0]
    lp = log_softmax(l1)
    assert len(bs.hyps[0]) == 1 and bs.hyps[0][0][1] == prompt
    assert abs(bs.hyps[0][0][0] - lp[4] / 2) < 1e-5
    assert not bs.done[0]
    # step 2: EOS best again from beam 0 -> second hypothesis [2, 2, 0]; early stopping ends the sequence
    toks, idx = bs.step(np.stack([l1, l1 - 10]))
    assert bs.done[0] and len(bs.hyps[0]) == 2
    assert sorted(h[1] for h in bs.hyps[0]) == [[2, 2], [2, 2, 0]]
    assert bs.is_done()
    toks, idx = bs.step(np.stack([l1, l1]))  # a finished sequence: pad from row 0, nothing else changes
    assert toks == [pad, pad] and idx == [0, 0] and len(bs.hyps[0]) == 2
    out = bs.finalize()
    # scores: [2, 2] -> lp[4] / 2, [2, 2, 0] -> (lp[0] + lp[4]) / 3; the larger one wins
    s_a, s_b = lp[4] / 2, (lp[0] + lp[4]) / 3
    want = [2, 2] if s_a > s_b else [2, 2, 0]
    assert out[0].tolist()[:len(want) + 1] == want + [eos]
    assert all(t == pad for t in out[0].tolist()[len(want) + 1:])


@pytest.mark.parametrize("batch,nb,keep,pen,early,eos", [(1, 2, 1, 1.0, False, 0), (2, 3, 2, 1.0, False, 5), (3, 4, 1, 0.6, True, 1),
                                                          (2, 2, 2, 2.0, False, -1), (1, 5, 3, 1.0, True, 7)])
def test_library_searcher_matches_oracle(batch, nb, keep, pen, early, eos):
    from xfastertransformer_amd.automodel import BeamSearcher
    vocab, seq, max_len, pad = 12, 4, 14, 2
    rng = np.random.default_rng(batch * 100 + nb)
    prompts = rng.integers(0, vocab, (batch, seq))
    ref = orc.BeamSearchOracle(prompts, nb, max_len, eos, pad, vocab, keep=keep, len_penalty=pen, early=early)
    lib = BeamSearcher(prompts, nb, max_len, eos, pad, vocab, num_return_sequences=keep, length_penalty=pen, early_stopping=early)
    steps = 0
    while not ref.is_done():
        assert not lib.is_done()
        logits = np.stack([toy_lm(r, vocab, 99 + batch) for r in ref.rows])
        t_ref, i_ref = ref.step(logits)
        t_lib, i_lib, s_lib = lib.step(logits)
        assert t_lib == t_ref and i_lib == i_ref, steps
        assert np.allclose(s_lib, ref.scores, atol=1e-4)
        steps += 1
    assert lib.is_done() and steps >= 1
    assert np.array_equal(lib.finalize(), ref.finalize())
