#!/usr/bin/env python3
"""Decode-throughput benchmark of the MI355X decoder-layer hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--weights int8|uint4] [--kv fp16|int8]
                    [--eager | --no-fusion | --persistent]        (variants of the decode step)
                    [--pmc-workload | --pmc-summary FETCH_CSV WRITE_CSV]   (hardware-counter traffic)

Workload (configs[3] of the benchmark definition): a 32-layer Llama-2-7B-shape model with random weights
(vocab 32000, hidden 4096, intermediate 11008, 32 heads), weight-only INT8 (or UINT4)
per-channel codes against bf16 activations, FP16 KV cache, a 512-token prompt, then greedy
decode.  One "step" is one decode step of the whole batch (one graph replay); the value is
decoded tokens per second with every weight and the KV cache resident in HBM.

One JSON line goes to stdout.  Besides the driver's fields it carries
  roofline     the dominant kernel of the step (one of the three forms of the M<=32 weight-only
               GEMV) timed live with HIP events on the launch stream, in algorithmic bytes per
               launch; traffic = counter-measured HBM bytes per launch (profiles/)
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


def build_model(xh, kind, batch, max_seq, prompt, kv_int8=False):
    c = CFG
    rng = np.random.default_rng(3)
    qkv_cols = (c["q_heads"] + 2 * c["kv_heads"]) * c["head"]
    shapes = [(c["hidden"], qkv_cols), (c["q_heads"] * c["head"], c["hidden"]), (c["hidden"], 2 * c["inter"]),
              (c["inter"], c["hidden"])]
    host = [synth_codes(rng, kind, K, N) for K, N in shapes]
    model = xh.Model(c["layers"], c["hidden"], c["inter"], c["q_heads"], c["kv_heads"], c["head"], vocab=c["vocab"],
                     max_batch=batch, max_seq=max_seq, max_tokens=batch * prompt, kv_dtype=xh.INT8 if kv_int8 else xh.FP16)
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


class GemvHarness:
    """Launches the decode GEMVs exactly as the decode step does, one kernel at a time:
    index 0 QKV (RMSNorm prologue, RoPE + cache-append epilogue), 1 out-projection, 2 gate/up
    (RMSNorm prologue, SwiGLU), 3 down projection."""

    def __init__(self, xh, M):
        c = CFG
        self.xh, self.M = xh, M
        rng = np.random.default_rng(1)
        k_max = max(c["hidden"], c["inter"])
        self.A = xh.DeviceBuffer.from_numpy(xh.f32_to_bf16_bits(rng.standard_normal((M, k_max)).astype(np.float32)))
        self.x = xh.DeviceBuffer.from_numpy(rng.standard_normal((M, c["hidden"])).astype(np.float32))
        self.g = xh.DeviceBuffer.from_numpy(np.ones(c["hidden"], np.float32))
        self.out = xh.DeviceBuffer(M * 2 * c["inter"] * 4)
        self.cache = xh.KVCache(xh.FP16, M, c["kv_heads"], 64, c["head"])
        self.tables = xh.RopeTables(c["head"], 64)
        self.fused = M <= 4

    def launch(self, w, i):
        xh, c, M = self.xh, CFG, self.M
        if i == 0 and self.fused:
            xh.gemm_qkv_rmsnorm_rope(w, self.cache, self.x.ptr, M, c["hidden"], self.g.ptr, 1e-6, self.out.ptr,
                                     c["q_heads"] * c["head"], c["q_heads"], self.tables, 7)
        elif i == 2 and self.fused:
            xh.gemm_gateup_silu_rmsnorm(w, self.x.ptr, M, c["hidden"], self.g.ptr, 1e-6, self.out.ptr, w.N // 2, xh.BF16)
        elif i == 2:
            xh.gemm_gateup_silu(w, self.A.ptr, M, w.K, self.out.ptr, w.N // 2, xh.BF16)
        elif i in (1, 3):
            # out-projection / down projection: fp32 result + fp32 residual, as in the layer
            xh.gemm(w, self.A.ptr, M, w.K, self.out.ptr, w.N, xh.F32, epi=xh.EPI_RESIDENTIAL, res=self.x.ptr, ldres=c["hidden"],
                    res_dtype=xh.F32)
        else:
            xh.gemm(w, self.A.ptr, M, w.K, self.out.ptr, w.N, xh.BF16)


def time_gemm_kernel(xh, layer_weights, which, M, iters):
    """Average duration of one launch of the weight-only GEMV over the distinct per-layer weights
    `which` (indices into a layer's [qkv, o, gateup, down]), HIP events on the launch stream, and
    its algorithmic bytes (the packed weight, the activation rows in, the result rows out)."""
    h = GemvHarness(xh, M)
    for ws in layer_weights:
        for i in which:
            h.launch(ws[i], i)
    xh.synchronize()
    t = xh.Timer()
    n = 0
    t.start()
    for _ in range(iters):
        for ws in layer_weights:
            for i in which:
                h.launch(ws[i], i)
                n += 1
    ms = t.stop()
    in_bytes = lambda i, w: (4 if (h.fused and i in (0, 2)) else 2) * M * w.K
    # result rows: bf16, except the fp32 result + fp32 residual of out-proj / down
    out_bytes = lambda i, w: (8 * M * w.N) if i in (1, 3) else 2 * M * (w.N // (2 if i == 2 else 1))
    byts = sum(layer_weights[0][i].bytes() + in_bytes(i, layer_weights[0][i]) + out_bytes(i, layer_weights[0][i])
               for i in which) / len(which)
    return ms * 1e3 / n, byts


PMC_COPY_BYTES = 256 << 20


def pmc_workload(xh, layer_weights, M):
    """What `rocprofv3 --pmc FETCH_SIZE` (and, in a second run, WRITE_SIZE) is pointed at: 8 launches
    of the library's plain copy kernel over PMC_COPY_BYTES (known traffic: that many bytes read and
    as many written), then one launch of the decode GEMV over every layer's weights (distinct
    memory each time, so nothing is served from a cache)."""
    src = xh.DeviceBuffer(PMC_COPY_BYTES)
    dst = xh.DeviceBuffer(PMC_COPY_BYTES)
    src.zero()
    xh.synchronize()
    for _ in range(8):
        xh.copy_kernel(dst.ptr, src.ptr, PMC_COPY_BYTES)
    xh.synchronize()
    for which in ((0,), (1, 3), (2,)):
        time_gemm_kernel(xh, layer_weights, which, M, 1)
    xh.synchronize()


TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "qgemm_skinny_int8_bs1_hbm_traffic.txt")


def pmc_summary(fetch_csv, write_csv):
    """Turns the two counter CSVs of `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv --
    python3 bench.py --pmc-workload` into the summary kept under profiles/ (runs on the CPU)."""
    import csv

    def per_kernel(path, counter):
        acc = {}
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] != counter:
                    continue
                name = r["Kernel_Name"]
                if "stream_copy_kernel" in name:
                    key = "copy"
                elif "qgemm_skinny_kernel<" in name:
                    # <KIND, NT, MT, U, NEED_SUM, KTAIL, NORM, ROPE>
                    targs = name.split("qgemm_skinny_kernel<")[1].split(">")[0].replace(" ", "").split(",")
                    key = "qkv" if targs[7] in ("true", "1") else ("wide" if targs[1] == "2" else "narrow")
                else:
                    continue
                acc.setdefault(key, []).append(float(r["Counter_Value"]))
        return {k: (sum(v) / len(v), len(v)) for k, v in acc.items()}

    fetch, write = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    copy_kib = PMC_COPY_BYTES / 1024.0
    sf, sw = copy_kib / fetch["copy"][0], copy_kib / write["copy"][0]
    print("HBM traffic per launch of the M=1 INT8 weight-only GEMV (qgemm_skinny_kernel), from hardware counters")
    print("commands (each its own run, as the counter blocks cannot be split over passes):")
    print("  rocprofv3 --pmc FETCH_SIZE --output-format csv -d <outdir>/pmc_fetch -- python3 bench.py --pmc-workload")
    print("  rocprofv3 --pmc WRITE_SIZE --output-format csv -d <outdir>/pmc_write -- python3 bench.py --pmc-workload")
    print("  python bench.py --pmc-summary <fetch counter_collection.csv> <write counter_collection.csv>")
    print("calibration: the library's plain copy kernel over %d KiB read %.1f (FETCH_SIZE) and wrote %.1f (WRITE_SIZE) counter units"
          % (copy_kib, fetch["copy"][0], write["copy"][0]))
    print("scale factors (KiB per counter unit): FETCH_SIZE %.4f  WRITE_SIZE %.4f" % (sf, sw))
    for key, label in (("qkv", "norm + qkv + RoPE / cache append (2 column tiles per wave)"),
                       ("narrow", "out-proj / down (1 column tile per wave), mean over the two shapes"),
                       ("wide", "norm + gate/up + SwiGLU (2 column tiles per wave)")):
        fb, wb = fetch[key][0] * sf * 1024.0, write[key][0] * sw * 1024.0
        print("%s: %d launches, fetch %.0f B + write %.0f B" % (label, fetch[key][1], fb, wb))
        print("traffic_bytes %s=%d" % (key, round(fb + wb)))


def measured_traffic(key):
    """HBM bytes per launch recorded by the last counter run (see pmc_summary), or None."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                if line.startswith("traffic_bytes %s=" % key):
                    return int(line.split("=")[1])
    except OSError:
        pass
    return None


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
    ap.add_argument("--kv", choices=["fp16", "int8"], default="fp16", help="KV cache format")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fusion", action="store_true", help="run RMSNorm / RoPE + cache append as their own kernels instead of inside the decode GEMVs")
    ap.add_argument("--persistent", action="store_true", help="run each decode step as the single persistent kernel (experimental)")
    ap.add_argument("--pmc-workload", action="store_true", help="counter workload for rocprofv3 --pmc: a plain copy kernel of known size, then every distinct decode GEMV of the model once; prints no result line")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), help="summarise the two counter CSVs of the --pmc-workload runs (CPU only)")
    ap.add_argument("--eager", action="store_true", help="launch decode kernels one by one instead of replaying the captured graph (for per-kernel profiling)")
    args = ap.parse_args()
    if args.pmc_summary:
        pmc_summary(*args.pmc_summary)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no collectives are part of it)", file=sys.stderr)
        sys.exit(2)

    from xfastertransformer_amd import capi as xh
    xh.init(0)
    kind = 0 if args.weights == "int8" else 1
    B = args.batch
    max_seq = args.prompt + args.warmup + args.steps + 1
    model, layer_weights, lmw, host, shapes = build_model(xh, kind, B, max_seq, args.prompt, args.kv == "int8")

    if args.pmc_workload:
        pmc_workload(xh, layer_weights, B)
        return
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
    # the same prompt again: the first call also pays for loading every prefill kernel's code
    t0 = time.time()
    model.prefill(ids)
    xh.synchronize()
    ttft_warm_ms = (time.time() - t0) * 1e3

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
    kv_elem = (1 + 4.0 / CFG["head"]) if args.kv == "int8" else 2  # INT8 code + one fp32 scale per (token, head)
    kv_bytes = CFG["layers"] * 2 * B * ctx * CFG["kv_heads"] * CFG["head"] * kv_elem
    step_bytes = wbytes + kv_bytes

    # dominant kernel: the M<=32 weight-only GEMV, in the three forms the decode step launches it
    groups = []
    fused = B <= 4  # beyond 4 rows the norm and the rotation run as kernels of their own
    for key, name, which in (("qkv", "qgemm_skinny_kernel (norm + qkv + RoPE/cache append)" if fused else "qgemm_skinny_kernel (qkv)", (0,)),
                             ("narrow", "qgemm_skinny_kernel (out-proj, down)", (1, 3)),
                             ("wide", "qgemm_skinny_kernel (norm + gate/up + SwiGLU)" if fused else "qgemm_skinny_kernel (gate/up + SwiGLU)", (2,))):
        us, byts = time_gemm_kernel(xh, layer_weights, which, B, 4)
        groups.append(dict(name=name, us=us, bytes=byts, launches=len(which), key=key))
    groups.sort(key=lambda g: -g["us"] * g["launches"])
    dom, others = groups[0], groups[1:]
    achieved = dom["bytes"] / dom["us"] / 1e3
    # counter-measured HBM bytes per launch exist for the configuration the counters were run on
    traffic = measured_traffic(dom["key"]) if (args.weights == "int8" and B == 1) else None

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
        "config": {"workload": "configs[3]: 32-layer Llama-2-7B-shape, %s weight-only, %s KV, batch %d, "
                               "%d-token prompt, greedy decode" % (args.weights.upper(), args.kv.upper(), B, args.prompt),
                   "batch": B, "prompt": args.prompt, "weights": args.weights, "kv": args.kv},
        "ttft_ms": round(ttft_ms, 2),
        "ttft_warm_ms": round(ttft_warm_ms, 2),
        "step_hbm_bytes": int(step_bytes),
        "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": {"bound": "hbm", "kernel": dom["name"], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "avg_launch_us": round(dom["us"], 3), "bytes_per_launch": int(dom["bytes"])},
        "other_kernels": [{"kernel": g["name"], "launches_per_layer": g["launches"], "avg_launch_us": round(g["us"], 3),
                           "bytes_per_launch": int(g["bytes"]),
                           "frac": round(g["bytes"] / g["us"] / 1e3 / HBM_PEAK_GBS, 4)} for g in others],
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(kind, host, shapes, B)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
