#!/usr/bin/env python3
"""Decode-throughput benchmark of the MI355X decoder-layer hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--weights int8|uint4]

Workload (BASELINE.json configs[3]): a 32-layer Llama-2-7B-shape model with random weights
(vocab 32000, hidden 4096, intermediate 11008, 32 heads), weight-only INT8 (or UINT4)
per-channel codes against bf16 activations, FP16 KV cache, a 512-token prompt, then greedy
decode.  One "step" is one decode step of the whole batch (one graph replay); the value is
decoded tokens per second with every weight and the KV cache resident in HBM.

One JSON line goes to stdout.  Besides the driver's fields it carries
  roofline     the dominant kernel (the M<=32 weight-only GEMM) timed live with HIP events
               on the launch stream, in algorithmic bytes per launch
  cpu_baseline this repository's CPU restatement of the reference's arithmetic (the oracle),
               timed on the host cores on a bounded sample of the same workload
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

CFG = dict(layers=32, hidden=4096, inter=11008, q_heads=32, kv_heads=32, head=128, vocab=32000)


def synth_codes(rng, kind, K, N):
    """Codes distributed like N(0, 0.02^2) weights quantised per output channel."""
    if kind == 0:
        q = np.clip(np.rint(rng.standard_normal((K, N), dtype=np.float32) * (127.0 / 4.2)), -127, 127).astype(np.int8)
        scale = np.full(N, 0.02 * 4.2 / 127.0, np.float32)
        return q, scale, None
    u = np.clip(np.rint(rng.standard_normal((K, N), dtype=np.float32) * (15.0 / 8.4) + 7.5), 0, 15).astype(np.uint8)
    q = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    scale = np.full(N, 0.02 * 8.4 / 15.0, np.float32)
    zero = np.full(N, -0.02 * 4.2, np.float32)
    return q, scale, zero


def build_model(xh, kind, batch, max_seq, prompt):
    c = CFG
    rng = np.random.default_rng(3)
    qkv_cols = (c["q_heads"] + 2 * c["kv_heads"]) * c["head"]
    shapes = [(c["hidden"], qkv_cols), (c["q_heads"] * c["head"], c["hidden"]), (c["hidden"], 2 * c["inter"]),
              (c["inter"], c["hidden"])]
    host = [synth_codes(rng, kind, K, N) for K, N in shapes]
    model = xh.Model(c["layers"], c["hidden"], c["inter"], c["q_heads"], c["kv_heads"], c["head"], vocab=c["vocab"],
                     max_batch=batch, max_seq=max_seq, max_tokens=batch * prompt, kv_dtype=xh.FP16)
    ones = np.ones(c["hidden"], np.float32)
    layer_weights = []
    for l in range(c["layers"]):
        ws = [xh.Weight(kind, K, N, q, s, z, flags=xh.WF_GATEUP if i == 2 else xh.WF_NONE)
              for i, ((K, N), (q, s, z)) in enumerate(zip(shapes, host))]
        model.set_layer(l, *ws, ones, ones)
        layer_weights.append(ws)
    emb = (rng.standard_normal((c["vocab"], c["hidden"]), dtype=np.float32) * 0.02).astype(np.float16).view(np.uint16)
    lm = xh.f32_to_bf16_bits(rng.standard_normal((c["hidden"], c["vocab"]), dtype=np.float32) * 0.02)
    lmw = xh.Weight(xh.W_BF16, c["hidden"], c["vocab"], lm)
    model.set_head(emb, ones, lmw)
    return model, layer_weights, lmw, host, shapes


def time_gemm_kernel(xh, layer_weights, which, M, iters):
    """Average duration of one launch of the weight-only GEMM over the distinct per-layer weights
    `which` (indices into a layer's [qkv, o, gateup, down]), HIP events on the launch stream."""
    c = CFG
    K_max = max(c["hidden"], c["inter"])
    A = xh.DeviceBuffer.from_numpy(xh.f32_to_bf16_bits(np.random.default_rng(1).standard_normal((M, K_max)).astype(np.float32)))
    out = xh.DeviceBuffer(M * 2 * c["inter"] * 4)

    def launch(w, i):
        if i == 2:
            xh.gemm_gateup_silu(w, A.ptr, M, w.K, out.ptr, w.N // 2, xh.BF16)
        else:
            xh.gemm(w, A.ptr, M, w.K, out.ptr, w.N, xh.BF16)

    for ws in layer_weights:
        for i in which:
            launch(ws[i], i)
    xh.synchronize()
    t = xh.Timer()
    n = 0
    t.start()
    for _ in range(iters):
        for ws in layer_weights:
            for i in which:
                launch(ws[i], i)
                n += 1
    ms = t.stop()
    byts = sum(layer_weights[0][i].bytes() + 2 * M * layer_weights[0][i].K
               + 2 * M * (layer_weights[0][i].N // (2 if i == 2 else 1)) for i in which) / len(which)
    return ms * 1e3 / n, byts


def cpu_baseline(kind, host, shapes, batch):
    """The oracle's decode step of one layer (GEMMs + norm + SwiGLU; attention over a short
    context is negligible next to 202 MB of weights), extrapolated to 32 layers + lm_head."""
    from oracle import pyoracle as orc
    c = CFG
    ws = [orc.QWeight(kind, K, N, q, s, z) for (K, N), (q, s, z) in zip(shapes, host)]
    rng = np.random.default_rng(5)
    x = rng.standard_normal((batch, c["hidden"])).astype(np.float32)
    ones = np.ones(c["hidden"], np.float32)

    def layer_step():
        xn = orc.rmsnorm(x, ones)
        qkv = orc.qgemm(ws[0], xn)
        att = qkv[:, :c["hidden"]].copy()
        x1 = orc.qgemm(ws[1], att, orc.EPI_RESIDENTIAL, res=x)
        h = orc.silu_sum(orc.qgemm(ws[2], orc.rmsnorm(x1, ones)))
        return orc.qgemm(ws[3], h, orc.EPI_RESIDENTIAL, res=x1)

    layer_step()
    t0 = time.time()
    n = 0
    while time.time() - t0 < 12.0 and n < 50:
        layer_step()
        n += 1
    per_layer = (time.time() - t0) / n
    # lm_head: fp32 GEMM of the same byte count per row as one more 131 M-element matrix
    step = per_layer * (c["layers"] + c["hidden"] * c["vocab"] / 202375168.0)
    return dict(value=round(batch / step, 3), unit="tok/s", cores=orc.num_threads(), kind="port",
                sample=f"{n} decode steps of 1 of 32 layers (INT8/UINT4 weight-only GEMMs, RMSNorm, SwiGLU), "
                       f"extrapolated x32 + lm_head; attention over the cache not timed")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=512)
    ap.add_argument("--weights", choices=["int8", "uint4"], default="int8")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fusion", action="store_true", help="run RMSNorm / RoPE + cache append as their own kernels instead of inside the decode GEMVs")
    ap.add_argument("--persistent", action="store_true", help="run each decode step as the single persistent kernel (experimental)")
    ap.add_argument("--eager", action="store_true", help="launch decode kernels one by one instead of replaying the captured graph (for per-kernel profiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no collectives are part of it)", file=sys.stderr)
        sys.exit(2)

    from xfastertransformer_amd import capi as xh
    xh.init(0)
    kind = 0 if args.weights == "int8" else 1
    B = args.batch
    max_seq = args.prompt + args.warmup + args.steps + 1
    model, layer_weights, lmw, host, shapes = build_model(xh, kind, B, max_seq, args.prompt)

    if args.eager:
        model.use_graph(False)
    if args.no_fusion:
        model.use_fusion(False)
    if args.persistent:
        model.use_persistent(True)
    rng = np.random.default_rng(3)
    ids = rng.integers(0, CFG["vocab"], (B, args.prompt)).astype(np.int32)
    t0 = time.time()
    model.prefill(ids)
    xh.synchronize()
    ttft_ms = (time.time() - t0) * 1e3

    if args.warmup > 0:
        model.decode_untracked(args.warmup)
    xh.synchronize()
    t0 = time.time()
    model.decode_untracked(args.steps)  # launches `steps` graph replays, then synchronises
    xh.synchronize()
    dt = time.time() - t0
    ms_per_step = dt * 1e3 / args.steps
    tok_s = B * args.steps / dt

    # algorithmic HBM bytes of one decode step at the mean context of the timed region
    wbytes = sum(w.bytes() for w in layer_weights[0]) * CFG["layers"] + lmw.bytes()
    ctx = args.prompt + args.warmup + args.steps / 2.0
    kv_bytes = CFG["layers"] * 2 * B * ctx * CFG["kv_heads"] * CFG["head"] * 2
    step_bytes = wbytes + kv_bytes

    # dominant kernel: the M<=32 weight-only GEMM; the two instantiations the layer uses
    narrow_us, narrow_bytes = time_gemm_kernel(xh, layer_weights, (0, 1, 3), B, 4)
    wide_us, wide_bytes = time_gemm_kernel(xh, layer_weights, (2,), B, 4)
    dom = dict(name="qgemm_skinny_kernel (qkv, out-proj, down)", us=narrow_us, bytes=narrow_bytes, launches=3)
    alt = dict(name="qgemm_skinny_kernel (gate/up + SwiGLU)", us=wide_us, bytes=wide_bytes, launches=1)
    if alt["us"] * alt["launches"] > dom["us"] * dom["launches"]:
        dom, alt = alt, dom
    achieved = dom["bytes"] / dom["us"] / 1e3

    result = {
        "metric": "decode tok/s (7B-shape, INT8/INT4 wts, bs1/32); qGEMM % HBM roofline",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 activations x %s weights, fp32 accumulate" % args.weights,
        "data": "synthetic",
        "config": {"workload": "configs[3]: 32-layer Llama-2-7B-shape, %s weight-only, FP16 KV, batch %d, "
                               "%d-token prompt, greedy decode" % (args.weights.upper(), B, args.prompt),
                   "batch": B, "prompt": args.prompt, "weights": args.weights},
        "ttft_ms": round(ttft_ms, 2),
        "step_hbm_bytes": int(step_bytes),
        "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": {"bound": "hbm", "kernel": dom["name"], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "avg_launch_us": round(dom["us"], 3), "bytes_per_launch": int(dom["bytes"])},
        "other_kernels": [{"kernel": alt["name"], "avg_launch_us": round(alt["us"], 3),
                           "bytes_per_launch": int(alt["bytes"]),
                           "frac": round(alt["bytes"] / alt["us"] / 1e3 / HBM_PEAK_GBS, 4)}],
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(kind, host, shapes, B)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
