"""The benchmark's CPU baseline (oracle/xft_cpu_baseline.c, the fast restatement that is timed beside
the GPU) computes the same decode step as the bit-faithful oracle: logits of a small model agree, and
so do the greedy ids, over a few teacher-forced steps."""
import ctypes as C

import numpy as np

import bench
from oracle import pyoracle as orc


def test_cpu_baseline_decode_step_matches_oracle():
    lib, _ = bench._build_cpu_baseline_lib()
    cfg = dict(layers=2, hidden=256, inter=384, q_heads=4, kv_heads=2, head=64, vocab=50)
    B, max_seq = 2, 16
    rng = np.random.default_rng(7)
    for kind in (orc.W_INT8, orc.W_UINT4):
        shapes = [(cfg["hidden"], (cfg["q_heads"] + 2 * cfg["kv_heads"]) * cfg["head"]), (cfg["q_heads"] * cfg["head"], cfg["hidden"]),
                  (cfg["hidden"], 2 * cfg["inter"]), (cfg["inter"], cfg["hidden"])]
        ln = rng.uniform(0.8, 1.2, cfg["hidden"]).astype(np.float32)
        layers, arrays = [], [[], [], [], []]
        for _ in range(cfg["layers"]):
            ws = [orc.quantize(kind, (rng.standard_normal(s) * 0.05).astype(np.float32)) for s in shapes]
            layers.append(orc.LlamaLayerOracle(cfg["hidden"], cfg["inter"], cfg["q_heads"], cfg["kv_heads"], cfg["head"], *ws, ln, ln,
                                               batch=B, max_seq=max_seq))
            for i, w in enumerate(ws):
                arrays[i].append((w.q, w.scale, w.zero if kind == orc.W_UINT4 else None))
        emb = orc.to_fp16(rng.standard_normal((cfg["vocab"], cfg["hidden"])) * 0.5)
        lm = orc.round_bf16(rng.standard_normal((cfg["hidden"], cfg["vocab"])) * 0.05)
        ref = orc.LlamaModelOracle(layers, emb, ln, lm)
        kc = np.zeros((cfg["layers"], B, cfg["kv_heads"], max_seq, cfg["head"]), np.uint16)
        vc = np.zeros_like(kc)
        m, keep = bench.cpu_model(lib, cfg, kind, arrays, ln, ln, ln, emb, orc.to_bf16(lm), kc, vc, B, max_seq)
        n = int(lib.cpu_scratch_floats(C.byref(m)))
        scratch = np.zeros(n, np.float32)
        ids = rng.integers(0, cfg["vocab"], B).astype(np.int32)
        for pos in range(4):
            elogits, enext = ref.step(ids.reshape(B, 1), B, 1, pos)
            got = ids.copy()
            lib.cpu_decode_step(C.byref(m), got.ctypes.data_as(C.c_void_p), pos, scratch.ctypes.data_as(C.c_void_p))
            # the logits of the last sequence are still in the scratch area (its tail, before 64 spare floats)
            logits = scratch[n - 64 - cfg["vocab"]:n - 64]
            assert np.abs(logits - elogits[B - 1]).max() < 2e-3 * max(1.0, np.abs(elogits).max())
            for b in range(B):
                assert elogits[b, got[b]] >= elogits[b].max() - 1e-3
            ids = enext.astype(np.int32)
