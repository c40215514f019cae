"""Host-side checks of the model loader / searcher layer that need no GPU: the deterministic half of
the sampler against a numpy restatement of SampleSearch::sample (src/searchers/sample_search.cpp:154-243)
and against what the mathematics fixes, the Python face's argument checks (automodel.py:21-39 of the
reference) and the loader's rejection messages (src/models/models.cpp:1014-1035)."""
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))
PKG = os.path.join(ROOT, "xfastertransformer_amd")
pytestmark = pytest.mark.skipif(not os.path.exists(os.path.join(PKG, "libxft_layers.so")), reason="host library not built")


def _np_candidates(logits, top_k, top_p, temperature):
    """sample_search.cpp:154-226 in numpy: candidates ordered by (value, id) descending."""
    top_k = min(max(top_k, 2), logits.size)
    order = sorted(range(logits.size), key=lambda j: (logits[j], j), reverse=True)[:top_k]
    vals = logits[order].astype(np.float32)
    tinv = np.float32(1) / np.float32(temperature)
    if tinv != 1:
        vals = vals * tinv
    n = top_k
    if top_p < 1.0:
        pr = np.exp(vals.astype(np.float32))
        inv = np.float32(1) / pr.sum(dtype=np.float32)
        cur = np.float32(0)
        for i in range(top_k):
            cur += pr[i] * inv
            if cur > np.float32(top_p):
                n = i if i > 2 else 2
                break
    e = np.exp(vals[:n] - vals[:n].max())
    return np.asarray(order[:n], np.int32), (e / e.sum()).astype(np.float32)


@pytest.mark.parametrize("top_k,top_p,temperature", [(50, 1.0, 1.0), (50, 0.9, 1.0), (8, 0.5, 0.7), (1, 0.1, 1.0),
                                                     (5, 0.999, 2.0), (40, 0.3, 0.25)])
def test_sample_candidates_match_numpy_restatement(top_k, top_p, temperature):
    from xfastertransformer_amd import automodel
    rng = np.random.default_rng(top_k * 7 + int(top_p * 100))
    for trial in range(20):
        logits = (rng.standard_normal(997) * 3).astype(np.float32)
        if trial % 4 == 0:  # ties: the higher id comes first
            logits[rng.integers(0, 997, 3)] = logits.max()
        ids, probs = automodel.sample_candidates(logits, top_k, top_p, temperature)
        eids, eprobs = _np_candidates(logits, top_k, top_p, temperature)
        assert np.array_equal(ids, eids)
        assert np.allclose(probs, eprobs, rtol=1e-5, atol=1e-7)
        assert abs(float(probs.sum()) - 1.0) < 1e-5 and len(ids) >= 2
        assert np.all(np.diff(probs) <= 1e-7)  # candidates come in descending probability


def test_sample_candidates_closed_forms():
    from xfastertransformer_amd import automodel
    # equal logits: uniform over top_k candidates, highest ids first
    ids, probs = automodel.sample_candidates(np.zeros(10, np.float32), 4, 1.0, 1.0)
    assert list(ids) == [9, 8, 7, 6] and np.allclose(probs, 0.25)
    # two-point distribution: p = sigmoid(difference / temperature)
    lg = np.full(16, -50.0, np.float32)
    lg[3], lg[11] = 1.0, 0.0
    ids, probs = automodel.sample_candidates(lg, 2, 1.0, 0.5)
    assert list(ids) == [3, 11] and abs(probs[0] - 1 / (1 + np.exp(-2.0))) < 1e-6
    # top-p: with probabilities .5 .25 .125 ... the running sum passes 0.8 at the 3rd candidate
    # (index 2), which is not > 2, so 2 remain; it passes 0.9 at index 3, so 3 remain
    lg = (-np.arange(12) * np.log(2.0)).astype(np.float32)
    assert len(automodel.sample_candidates(lg, 12, 0.8, 1.0)[0]) == 2
    assert len(automodel.sample_candidates(lg, 12, 0.9, 1.0)[0]) == 3
    # the draw is the inverse CDF: u just under / over a boundary
    ids, probs = np.asarray([7, 5, 9], np.int32), np.asarray([0.5, 0.25, 0.25], np.float32)
    assert automodel.sample_pick(ids, probs, 0.0) == 7 and automodel.sample_pick(ids, probs, 0.5) == 7
    assert automodel.sample_pick(ids, probs, 0.500001) == 5 and automodel.sample_pick(ids, probs, 0.76) == 9
    assert automodel.sample_pick(ids, probs, 1.0) == 9


def test_python_face_rejects_what_the_reference_rejects(tmp_path):
    from xfastertransformer_amd import automodel
    with pytest.raises(Exception, match="don't support fp64"):
        automodel.AutoModel(str(tmp_path), "fp64")
    with pytest.raises(Exception, match="KV cache data type"):
        automodel.AutoModel(str(tmp_path), "int8", "fp32")
    with pytest.raises(Exception, match="of this build don't support the type fp8_e4m3"):
        automodel.AutoModel(str(tmp_path), "fp8_e4m3")
    with pytest.raises(FileNotFoundError):
        automodel.AutoModel(str(tmp_path), "int8")
    with pytest.raises(FileNotFoundError):  # the mixed first-token / next-token types are served
        automodel.AutoModel(str(tmp_path), "bf16_int8")


def _run(code):
    return subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)


def test_loader_messages_for_unusable_directories(tmp_path):
    """The C++ constructor prints the reference's message and exits before touching the device."""
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.ini").write_text("[chatglm]\nvocab_size = 10\n")
    r = _run(f"from xfastertransformer_amd import automodel as a; a.AutoModel({str(d)!r}, 'int8')")
    assert r.returncode == 255 and "Unsupported data type or KV cache data type: chatglm-int8-fp16" in r.stdout
    (d / "config.ini").write_text("; empty\n")
    r = _run(f"from xfastertransformer_amd import automodel as a; a.AutoModel({str(d)!r}, 'int8')")
    assert r.returncode == 255 and "Could not load model config.ini." in r.stdout


def test_fixture_writer_round_trips_its_element_types(tmp_path):
    import make_llama_fixture as fx
    cfg = dict(fx.TINY, layers=1, vocab=64, inter=128)
    for wt, dt in (("fp32", np.float32), ("fp16", np.float16), ("bf16", np.uint16)):
        held = fx.write_model_dir(str(tmp_path / wt), cfg, 1, wt)
        raw = np.fromfile(tmp_path / wt / "model.lm_head.weight.bin", dt)
        back = raw.astype(np.float32) if wt != "bf16" else (raw.astype(np.uint32) << 16).view(np.float32)
        assert np.array_equal(back.reshape(64, 256), held["lm_head"])
    held = fx.write_model_dir(str(tmp_path / "q4"), cfg, 1, "fp32", "uint4")
    raw = np.fromfile(tmp_path / "q4" / "model.layers.0.mlp.down_proj.qweight.0.bin", np.uint8).reshape(128, 128)
    q = held["layers"][0]["down"]["q"]
    assert np.array_equal(raw & 15, q[:, 0::2]) and np.array_equal(raw >> 4, q[:, 1::2])
