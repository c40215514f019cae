"""torch.classes.xfastertransformer.AutoModel (libxft_pt.so), the Torch custom class the reference's Python
package binds (src/pytorch/pytorch_warpper.cpp:18-34, src/pytorch/auto_model.h:25-360): the same method
names and tensor conventions over this library's xft::AutoModel.  Checked against the ctypes face of the
same C++ class (whose ids are pinned against a directly built device model and the oracle in
test_automodel_gpu.py), against causality for the logits of every prompt position, and, for the
sequence-id interface (set_input_cb / forward_cb / free_seqs), against each sequence's own lockstep run."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
LIB = os.path.join(ROOT, "xfastertransformer_amd", "libxft_pt.so")


@pytest.fixture(scope="module")
def torch_class():
    import torch
    from xfastertransformer_amd import capi  # libxft_hip.so first (RTLD_GLOBAL), or the import raises
    capi.init()
    assert os.path.exists(LIB), "libxft_pt.so is not built; run `python -m xfastertransformer_amd.build`"
    torch.classes.load_library(LIB)
    return torch.classes.xfastertransformer.AutoModel


@pytest.fixture(scope="module")
def am():
    from xfastertransformer_amd import automodel
    return automodel


@pytest.fixture(scope="module")
def model_dir(tmp_path_factory):
    import make_llama_fixture as fx
    path = str(tmp_path_factory.mktemp("torch_class") / "model")
    held = fx.write_model_dir(path, None, 21)
    return path, held


def test_generation_loop_equals_the_ctypes_face(torch_class, am, model_dir):
    import torch
    path, held = model_dir
    V = held["cfg"]["vocab"]
    B, S, max_len = 2, 9, 24
    ids = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(3))
    ref_model = am.AutoModel.from_pretrained(path, dtype="int8")
    want = ref_model.generate(ids, max_length=max_len, eos_token_id=V + 1)
    ref_model.free()
    m = torch_class(path, "int8", "fp16")
    assert m.get_rank() == 0
    m.config(max_len, 1, 1, 1.0, False, V + 1, None, False, 1.0, 50, 1.0, 1.0, None)
    m.input(ids)
    steps = []
    while not m.is_done():
        t = m.generate()
        assert t.dtype == torch.int64 and tuple(t.shape) == (B, 1)
        steps.append(t)
    out = m.finalize()
    assert out.dtype == torch.int64 and tuple(out.shape) == (B, max_len)
    assert torch.equal(out, want)
    assert torch.equal(torch.cat(steps, 1), want[:, S:])
    # beam search through the same calls: rows = batch x hypotheses kept
    m.config(S + 6, 3, 2, 1.0, False, V + 1, None, False, 1.0, 50, 1.0, 1.0, None)
    m.input(ids)
    while not m.is_done():
        assert tuple(m.generate().shape) == (B, 3)
    beams = m.finalize()
    ref_model = am.AutoModel.from_pretrained(path, dtype="int8")
    want_beams = ref_model.generate(ids, max_length=S + 6, num_beams=3, num_return_sequences=2, eos_token_id=V + 1)
    ref_model.free()
    assert torch.equal(beams, want_beams.reshape(beams.shape))
    with pytest.raises(Exception):
        torch_class(path, "int9", "fp16")
    with pytest.raises(Exception):
        torch_class(path, "int8", "fp8")


def test_forward_returns_the_logits_of_every_position(torch_class, model_dir):
    """forward(ids) -> [batch, seqLen, vocab].  The last position is what the generation loop samples from
    (checked against the oracle elsewhere); an earlier position t must equal the last position of the prompt
    cut after t + 1 tokens (causal attention), up to the rounding of a different batch shape."""
    import torch
    path, held = model_dir
    V = held["cfg"]["vocab"]
    B, S = 2, 12
    ids = torch.randint(0, V, (B, S), generator=torch.Generator().manual_seed(8))
    m = torch_class(path, "int8", "fp16")
    full = m.forward(ids).clone()
    assert tuple(full.shape) == (B, S, V) and full.dtype == torch.float32 and torch.isfinite(full).all()
    for t in (0, 4, S - 1):
        cut = m.forward(ids[:, :t + 1].contiguous()).clone()
        err = float((cut[:, t] - full[:, t]).abs().max())
        assert err < 2e-2, (t, err)
        assert torch.equal(cut[:, t].argmax(-1), full[:, t].argmax(-1)) or err < 1e-3
    # rows differ from each other (no row was written twice or skipped)
    assert float((full[:, 1:] - full[:, :-1]).abs().max()) > 1e-2


def test_prefix_sharing_through_the_class(torch_class, model_dir):
    """set_prefix / unset_prefix (src/pytorch/auto_model.h: setPrefix / unsetPrefix): generation over a shared prefix
    gives the ids of generation from the whole prompts (FP16 cache: the same keys and values bit for bit)."""
    import torch
    path, held = model_dir
    V = held["cfg"]["vocab"]
    B, n, tail, max_len = 2, 33, 5, 50
    g = torch.Generator().manual_seed(12)
    prefix = torch.randint(0, V, (1, n), generator=g)
    ids = torch.cat([prefix.repeat(B, 1), torch.randint(0, V, (B, tail), generator=g)], 1)

    def run(m):
        m.config(max_len, 1, 1, 1.0, False, V + 1, None, False, 1.0, 50, 1.0, 1.0, None)
        m.input(ids)
        while not m.is_done():
            m.generate()
        return m.finalize()

    m = torch_class(path, "int8", "fp16")
    whole = run(m)
    m.set_prefix(prefix)
    shared = run(m)
    m.unset_prefix()
    again = run(m)
    assert torch.equal(shared, whole) and torch.equal(again, whole)
    with pytest.raises(Exception):
        m.set_prefix(ids)  # one prompt only


def test_sequence_id_interface(torch_class, am, model_dir):
    """set_input_cb with ragged prompts (1-D ids + lengths), forward_cb, tokens chosen by the caller fed back
    with set_input_cb(ids, None, seqIDs, None), a sequence that sits out, free_seqs: every sequence follows
    its own lockstep greedy run."""
    import torch
    path, held = model_dir
    V = held["cfg"]["vocab"]
    rng = np.random.default_rng(17)
    prompts = [rng.integers(0, V, n).astype(np.int64) for n in (5, 13, 8)]
    ref_model = am.AutoModel.from_pretrained(path, dtype="int8")
    solo = [ref_model.generate(p[None, :].astype(np.int32), max_length=len(p) + 8, eos_token_id=V + 1)[0] for p in prompts]
    ref_model.free()
    m = torch_class(path, "int8", "fp16")
    flat = torch.from_numpy(np.concatenate(prompts))
    lens = torch.tensor([len(p) for p in prompts])
    seq = m.set_input_cb(flat, lens, None, torch.tensor([40]))
    assert seq.dtype == torch.int64 and tuple(seq.shape) == (3,) and len(set(seq.tolist())) == 3
    logits = m.forward_cb()
    assert tuple(logits.shape) == (3, V)
    got = [[int(t)] for t in logits.argmax(-1)]
    for step in range(3):
        nxt = torch.tensor([[g[-1]] for g in got])
        assert torch.equal(m.set_input_cb(nxt, None, seq, None), seq)
        for g, t in zip(got, m.forward_cb().argmax(-1)):
            g.append(int(t))
    # the middle sequence sits out two steps
    pair = seq[[0, 2]]
    for step in range(2):
        nxt = torch.tensor([[got[0][-1]], [got[2][-1]]])
        m.set_input_cb(nxt, None, pair, None)
        lg = m.forward_cb()
        assert tuple(lg.shape) == (2, V)
        got[0].append(int(lg[0].argmax()))
        got[2].append(int(lg[1].argmax()))
    assert m.free_seqs(seq[:1]) and not m.free_seqs(seq[:1])
    m.set_input_cb(torch.tensor([[got[1][-1]]]), None, seq[1:2], None)
    got[1].append(int(m.forward_cb()[0].argmax()))
    for k, g in enumerate(got):
        n = len(prompts[k])
        assert g == solo[k][n:n + len(g)].tolist(), (k, g, solo[k][n:])
    # 2-D prompts of one length, with the logits of every position when asked through forward()
    same = torch.from_numpy(np.stack([prompts[1][:6], prompts[2][:6]]))
    ids2 = m.set_input_cb(same, None, None, torch.tensor([30, 36]))  # (room within the rows the live sequences hold)
    assert tuple(m.forward_cb().shape) == (2, V)
    assert m.free_seqs(torch.cat([seq[1:], ids2]))
    # with every sequence gone the model may grow: no maximum length = the model's own
    ids3 = m.set_input_cb(same, None, None, None)
    lg = m.forward_cb()
    assert tuple(lg.shape) == (2, V) and torch.isfinite(lg).all()
    assert m.free_seqs(ids3)
