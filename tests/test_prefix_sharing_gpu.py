"""Prefix sharing (Model::setPrefix / unsetPrefix, src/models/models.cpp:930-946; CommonDecoder::setPrefix,
prefixForward and the step-0 branch of forward, src/models/common_decoder.h:337-350, 440-443, 695-768): the prefix runs
once as one sequence, every later input carries it in front and only runs what follows it, over cache rows that start
as copies of the prefix's positions.

Pinned against the same library without the prefix.  FP16 cache: the keys and values a sequence attends over are bit
for bit those of the whole prompt pass (a cache row is computed token by token, whatever the batch and the chunk), so
prompt logits and generated ids must be equal, for a prefix of whole 32-token blocks and for a ragged one (copy of a
partly filled last block).  INT8 cache: a prompt pass from position 0 attends over the unquantised keys and values of
the pass, a pass over a prefix over the prefix's INT8 codes (as in the reference, whose first pass takes its flash-style
route and whose pass over a past reads the cache), so the logits agree to the size of that quantisation only."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))


@pytest.fixture(scope="module")
def am():
    from xfastertransformer_amd import automodel
    return automodel


@pytest.mark.parametrize("kv", ["fp16", "int8"])
@pytest.mark.parametrize("prefix_len", [64, 41])
def test_generation_over_a_shared_prefix_equals_generation_from_the_whole_prompt(am, tmp_path, kv, prefix_len):
    import make_llama_fixture as fx
    held = fx.write_model_dir(str(tmp_path / "model"), None, 21)
    V = held["cfg"]["vocab"]
    rng = np.random.default_rng(prefix_len)
    B, tail, max_len = 3, 9, prefix_len + 9 + 14
    prefix = rng.integers(0, V, (1, prefix_len)).astype(np.int32)
    ids = np.concatenate([np.repeat(prefix, B, 0), rng.integers(0, V, (B, tail)).astype(np.int32)], 1)
    model = am.AutoModel.from_pretrained(str(tmp_path / "model"), dtype="int8", kv_cache_dtype=kv)
    whole = model.generate(ids, max_length=max_len)
    model.input(ids)
    whole_logits = model.logits().copy()

    model.prefix_sharing(prefix)
    shared = model.generate(ids, max_length=max_len)
    model.input(ids)
    shared_logits = model.logits().copy()
    err = float(np.abs(shared_logits - whole_logits).max())
    print(f"kv={kv} prefix={prefix_len}: prompt logits with / without the shared prefix differ by {err:.3e}", flush=True)
    if kv == "fp16":
        assert err == 0.0 and np.array_equal(shared, whole)
    else:
        assert err < 3e-2 and np.array_equal(shared[:, :prefix_len + tail], whole[:, :prefix_len + tail])

    # a second input over the same prefix (the prefix is not run again), other tails and another batch size
    ids2 = np.concatenate([np.repeat(prefix, 2, 0), rng.integers(0, V, (2, tail + 3)).astype(np.int32)], 1)
    shared2 = model.generate(ids2, max_length=max_len + 3)
    model.disable_prefix_sharing()
    whole2 = model.generate(ids2, max_length=max_len + 3)
    if kv == "fp16":
        assert np.array_equal(shared2, whole2)
    assert shared2.shape == whole2.shape and np.array_equal(shared2[:, :ids2.shape[1]], ids2)
    model.free()
