#!/usr/bin/env python3
"""Decode-throughput benchmark of the MI355X decoder-layer hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--weights int8|uint4] [--kv fp16|int8]
                    [--eager | --no-fusion]                       (variants of the decode step)
                    [--no-extras] [--no-cpu-baseline]
                    [--prefill-gemm | --attention | --moe | --stream-floor]   (one of the extra measurements alone, one JSON line)
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
  cpu_baseline this repository's CPU restatement of the reference's data flow
               (oracle/xft_cpu_baseline.c, compiled on this machine with -O3 -march=native -fopenmp),
               timed on the host cores on a bounded sample of the same workload
  extra        the other points the metric names, measured in the same run: decode at batch 32 and
               with UINT4 weights, the weight-only GEMM sweep at 2048 rows against the bf16 MFMA
               peak, the GQA attention sweep, and the sparse-MLP layer
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
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, published
MFMA_INT8_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA, published

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


def stream_floor(xh, sizes_mb=(16.8, 45.1, 50.4, 90.2), buffers=32, iters=4):
    """The library's read-only kernel over `buffers` distinct device buffers of each size (the byte counts of
    one decode layer's four packed INT8 weights), launched back to back and timed with HIP events: what
    streaming that many bytes costs on this machine with nothing behind the loads, launch ramp and tail
    included.  The weight-streaming GEMVs are held against these, not against bytes / 8 TB/s."""
    out = []
    for mb in sizes_mb:
        nbytes = int(mb * 1e6) // 4096 * 4096
        bufs = [xh.DeviceBuffer(nbytes) for _ in range(buffers)]
        for b in bufs:
            b.zero()
        for b in bufs:
            xh.read_kernel(b.ptr, nbytes)
        xh.synchronize()
        t = xh.Timer()
        t.start()
        for _ in range(iters):
            for b in bufs:
                xh.read_kernel(b.ptr, nbytes)
        ms = t.stop()
        us = ms * 1e3 / (iters * buffers)
        out.append({"bytes": nbytes, "avg_launch_us": round(us, 2), "gbs": round(nbytes / us / 1e3, 1),
                    "frac_of_hbm_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
        for b in bufs:
            b.free()
    return out


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


def traffic_from_counters(fetch_csv, write_csv):
    """HBM bytes per launch of the three decode GEMV forms ({'qkv' | 'narrow' | 'wide': bytes}) from the counter CSVs of two
    `rocprofv3 --pmc FETCH_SIZE | WRITE_SIZE -- python3 bench.py --pmc-workload` runs, each counter scaled by what it reads
    for the plain copy kernel of known size in the same run."""
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
                    targs = name.split("qgemm_skinny_kernel<")[1].split(">")[0].replace(" ", "").split(",")
                    key = "qkv" if targs[7] in ("true", "1") else ("wide" if targs[1] == "2" else "narrow")
                else:
                    continue
                acc.setdefault(key, []).append(float(r["Counter_Value"]))
        return {k: sum(v) / len(v) for k, v in acc.items()}

    fetch, write = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    copy_kib = PMC_COPY_BYTES / 1024.0
    sf, sw = copy_kib / fetch["copy"], copy_kib / write["copy"]
    return {k: int(round((fetch[k] * sf + write[k] * sw) * 1024.0)) for k in ("qkv", "narrow", "wide")}


def live_traffic(timeout_s=100):
    """Runs the two counter passes as child processes of this run (rocprofv3 with this file's --pmc-workload after `--`,
    one counter a pass, each under a time limit and in a process group of its own) and returns traffic_from_counters() of
    them, or None when the profiler is missing, a pass fails or runs out of time.  Called before this process touches
    the GPU."""
    import glob
    import shutil
    import signal
    import subprocess
    import tempfile
    if shutil.which("rocprofv3") is None:
        return None
    me = os.path.abspath(__file__)
    out = tempfile.mkdtemp(prefix="xft_pmc_", dir="/tmp")
    env = dict(os.environ, TMPDIR="/tmp")
    csvs = []
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            d = os.path.join(out, counter)
            cmd = ["rocprofv3", "--pmc", counter, "--output-format", "csv", "-d", d, "--", sys.executable, me, "--pmc-workload"]
            pr = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, start_new_session=True)
            try:
                rc = pr.wait(timeout=timeout_s)
            except subprocess.TimeoutExpired:
                os.killpg(pr.pid, signal.SIGKILL)
                pr.wait()
                return None
            found = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
            if rc != 0 or not found:
                return None
            csvs.append(found[0])
        return traffic_from_counters(csvs[0], csvs[1])
    except Exception:
        return None
    finally:
        shutil.rmtree(out, ignore_errors=True)


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


def _cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown CPU"


def _build_cpu_baseline_lib():
    """oracle/xft_cpu_baseline.c compiled for THIS machine's vector ISA (gcc -O3 -march=native -fopenmp)
    into a temporary directory; the generic build kept next to the oracle is the fallback."""
    import ctypes
    import subprocess
    import tempfile
    src = os.path.join(ROOT, "oracle", "xft_cpu_baseline.c")
    out = os.path.join(tempfile.mkdtemp(prefix="xft_cpu_baseline_"), "libxft_cpu_baseline.so")
    flags = "-O3 -march=native -fopenmp"
    try:
        subprocess.check_call(["gcc"] + flags.split() + ["-fPIC", "-shared", "-fno-math-errno", "-std=gnu11", src, "-o", out, "-lm"],
                              stderr=subprocess.DEVNULL)
        return ctypes.CDLL(out), flags
    except (OSError, subprocess.CalledProcessError):
        return ctypes.CDLL(os.path.join(ROOT, "oracle", "libxft_cpu_baseline.so")), "-O3 -mavx2 -mfma -mf16c -fopenmp (prebuilt)"


def cpu_model(lib, cfg, kind, layer_arrays, ln1, ln2, final_norm, emb_fp16, lm_bf16, kcache, vcache, batch, max_seq):
    """The cpu_model struct of oracle/xft_cpu_baseline.c.  layer_arrays[i] (i = qkv, o, gate/up, down) is
    a list over layers of (codes, scale, zero-or-None) numpy arrays; returns (struct, objects to keep alive)."""
    import ctypes as C
    L = cfg["layers"]

    class CpuModel(C.Structure):
        _fields_ = [("kind", C.c_int), ("layers", C.c_int), ("hidden", C.c_int), ("inter", C.c_int), ("heads", C.c_int),
                    ("kv_heads", C.c_int), ("head", C.c_int), ("vocab", C.c_int), ("max_seq", C.c_int),
                    ("wq", C.POINTER(C.c_void_p) * 4), ("ws", C.POINTER(C.c_void_p) * 4), ("wz", C.POINTER(C.c_void_p) * 4),
                    ("ln1", C.c_void_p), ("ln2", C.c_void_p), ("final_norm", C.c_void_p), ("embedding", C.c_void_p),
                    ("lm_head", C.c_void_p), ("kcache", C.c_void_p), ("vcache", C.c_void_p), ("batch", C.c_int)]

    keep = [layer_arrays, ln1, ln2, final_norm, emb_fp16, lm_bf16, kcache, vcache]
    ptr = lambda a: a.ctypes.data_as(C.c_void_p)

    def table(arrs):
        t = (C.c_void_p * L)(*[a.ctypes.data for a in arrs])
        keep.append(t)
        return C.cast(t, C.POINTER(C.c_void_p))

    m = CpuModel()
    m.kind, m.layers, m.hidden, m.inter = kind, L, cfg["hidden"], cfg["inter"]
    m.heads, m.kv_heads, m.head, m.vocab = cfg["q_heads"], cfg["kv_heads"], cfg["head"], cfg["vocab"]
    m.max_seq, m.batch = max_seq, batch
    for i, per_layer in enumerate(layer_arrays):
        m.wq[i] = table([w[0] for w in per_layer])
        m.ws[i] = table([w[1] for w in per_layer])
        m.wz[i] = table([w[2] for w in per_layer]) if per_layer[0][2] is not None else None
    m.ln1, m.ln2, m.final_norm = ptr(ln1), ptr(ln2), ptr(final_norm)
    m.embedding, m.lm_head, m.kcache, m.vcache = ptr(emb_fp16), ptr(lm_bf16), ptr(kcache), ptr(vcache)
    lib.cpu_num_threads.restype = C.c_int
    lib.cpu_scratch_floats.restype = C.c_int64
    return m, keep


def cpu_baseline(kind, host, shapes, batch, prompt, budget_s=15.0):
    """Greedy decode steps of the whole 32-layer model on the host cores (every layer its own copy of
    the weights, FP16 cache filled up to the prompt length), as many as fit the time budget."""
    import ctypes as C
    lib, flags = _build_cpu_baseline_lib()
    c = CFG
    L = c["layers"]
    steps_max = 24
    max_seq = prompt + steps_max + 2
    # distinct memory per layer: nothing stays in a cache from one layer to the next
    layer_arrays = [[(q.copy(), sc, z) for _ in range(L)] for (q, sc, z) in host]
    rng = np.random.default_rng(5)
    ones = np.ones(c["hidden"], np.float32)
    emb = (rng.standard_normal((c["vocab"], c["hidden"]), dtype=np.float32) * 0.02).astype(np.float16).view(np.uint16)
    lm = ((rng.standard_normal((c["hidden"], c["vocab"]), dtype=np.float32) * 0.02).view(np.uint32) >> 16).astype(np.uint16)
    cache_shape = (L, batch, c["kv_heads"], max_seq, c["head"])
    kc = rng.standard_normal(cache_shape, dtype=np.float32).astype(np.float16).view(np.uint16)
    vc = rng.standard_normal(cache_shape, dtype=np.float32).astype(np.float16).view(np.uint16)
    m, keep = cpu_model(lib, c, kind, layer_arrays, ones, ones, ones, emb, lm, kc, vc, batch, max_seq)
    scratch = np.zeros(int(lib.cpu_scratch_floats(C.byref(m))), np.float32)
    ids = rng.integers(0, c["vocab"], batch).astype(np.int32)
    ptr = lambda a: a.ctypes.data_as(C.c_void_p)
    times = []
    t_start = time.time()
    for t in range(steps_max + 2):
        t0 = time.time()
        lib.cpu_decode_step(C.byref(m), ptr(ids), prompt + t, ptr(scratch))
        if t >= 2:  # two warm-up steps
            times.append(time.time() - t0)
        if time.time() - t_start > budget_s and len(times) >= 3:
            break
    med = float(np.median(times))
    return dict(value=round(batch / med, 3), unit="tok/s", cores=int(lib.cpu_num_threads()), kind="port",
                sample="xFT-semantics CPU restatement (not the xDNN binary): %d greedy decode steps (median, after 2 warm-up steps) "
                       "of the full 32-layer model at context %d, batch %d, every layer its own weights; gcc %s on %s"
                       % (len(times), prompt, batch, flags, _cpu_model_name()))


# ---------------------------------------------------------------------------- extra measurements
def decode_run(xh, kind, B, prompt, steps, warmup, kv_int8=False):
    """tok/s of greedy decode for one (weights, batch) point, with its share of the HBM roofline."""
    max_seq = prompt + warmup + steps + 1
    model, layer_weights, lmw, _, _ = build_model(xh, kind, B, max_seq, prompt, kv_int8)
    ids = np.random.default_rng(3).integers(0, CFG["vocab"], (B, prompt)).astype(np.int32)
    model.prefill(ids)
    model.decode_untracked(warmup)
    xh.synchronize()
    t0 = time.time()
    model.decode_untracked(steps)
    xh.synchronize()
    dt = time.time() - t0
    wbytes = sum(w.bytes() for w in layer_weights[0]) * CFG["layers"] + lmw.bytes()
    ctx = prompt + warmup + steps / 2.0
    kv_elem = (1 + 4.0 / CFG["head"]) if kv_int8 else 2
    step_bytes = wbytes + CFG["layers"] * 2 * B * ctx * CFG["kv_heads"] * CFG["head"] * kv_elem
    ms = dt * 1e3 / steps
    out = dict(weights="int8" if kind == 0 else "uint4", batch=B, kv="int8" if kv_int8 else "fp16", tok_s=round(B * steps / dt, 1),
               ms_per_step=round(ms, 4), step_hbm_bytes=int(step_bytes),
               step_hbm_frac=round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4))
    model.free()
    for ws in layer_weights:
        for w in ws:
            w.free()
    lmw.free()
    return out


def prefill_gemm_sweep(xh, M=2048, nweights=8, iters=3):
    """The weight-only GEMM sweep at M rows (bf16 in, bf16 out): every (N, K) x kind of the sweep
    launched back to back over `nweights` distinct weights (more than the 256 MB the Infinity Cache
    holds for every case but 4096 x 4096 UINT4/NF4, which get twice as many), HIP events on the
    launch stream; TFLOP/s = 2 M N K / time, against the published dense bf16 MFMA peak."""
    rng = np.random.default_rng(1)
    res = []
    for (N, K) in ((4096, 4096), (11008, 4096), (4096, 11008)):
        A = xh.DeviceBuffer.from_numpy(xh.f32_to_bf16_bits(rng.standard_normal((M, K), dtype=np.float32)))
        Cd = xh.DeviceBuffer(M * N * 2)
        for kind, name in ((xh.W_INT8, "int8"), (xh.W_UINT4, "uint4"), (xh.W_NF4, "nf4"), (xh.W_W8A8, "w8a8")):
            q, sc, z = synth_codes(rng, 0 if kind in (xh.W_INT8, xh.W_W8A8) else 1, K, N)
            if kind == xh.W_NF4:
                z = None
            nw = nweights * (2 if (kind in (xh.W_UINT4, xh.W_NF4) and N * K <= 4096 * 4096) else 1)
            ws = [xh.Weight(kind, K, N, q, sc, z) for _ in range(nw)]
            for w in ws:
                xh.gemm(w, A.ptr, M, K, Cd.ptr, N, xh.BF16)
            xh.synchronize()
            t = xh.Timer()
            t.start()
            for _ in range(iters):
                for w in ws:
                    xh.gemm(w, A.ptr, M, K, Cd.ptr, N, xh.BF16)
            us = t.stop() * 1e3 / (iters * nw)
            tf = 2.0 * M * N * K / us / 1e6
            if kind == xh.W_W8A8:  # per-row activation quantisation + int8 MFMA GEMM, against the int8 peak
                res.append(dict(kind=name, M=M, N=N, K=K, avg_launch_us=round(us, 2), tops=round(tf, 1),
                                frac_of_int8_mfma_peak=round(tf / MFMA_INT8_PEAK_TOPS, 4)))
            else:
                res.append(dict(kind=name, M=M, N=N, K=K, avg_launch_us=round(us, 2), tflops=round(tf, 1),
                                frac_of_bf16_mfma_peak=round(tf / MFMA_BF16_PEAK_TFLOPS, 4)))
            for w in ws:
                w.free()
    return res


def gemm_few_rows_sweep(xh, Ms=(1, 8, 32), iters=4):
    """The few-row cells of the weight-only GEMM sweep (bf16 in, bf16 out, plain epilogue): every (N, K) x kind at M rows
    over enough distinct weights to exceed the Infinity Cache, HIP events on the launch stream; these launches are bound
    by the weight bytes, so the figure is GB/s over packed weight + activation rows + result rows against the HBM peak."""
    rng = np.random.default_rng(1)
    res = []
    for (N, K) in ((4096, 4096), (11008, 4096), (4096, 11008)):
        for kind, name in ((xh.W_INT8, "int8"), (xh.W_UINT4, "uint4"), (xh.W_NF4, "nf4")):
            q, sc, z = synth_codes(rng, 0 if kind == xh.W_INT8 else 1, K, N)
            if kind == xh.W_NF4:
                z = None
            nw = 24 if kind == xh.W_INT8 else 40
            ws = [xh.Weight(kind, K, N, q, sc, z) for _ in range(nw)]
            for M in Ms:
                A = xh.DeviceBuffer.from_numpy(xh.f32_to_bf16_bits(rng.standard_normal((M, K), dtype=np.float32)))
                Cd = xh.DeviceBuffer(M * N * 2)
                for w in ws:
                    xh.gemm(w, A.ptr, M, K, Cd.ptr, N, xh.BF16)
                xh.synchronize()
                t = xh.Timer()
                t.start()
                for _ in range(iters):
                    for w in ws:
                        xh.gemm(w, A.ptr, M, K, Cd.ptr, N, xh.BF16)
                us = t.stop() * 1e3 / (iters * nw)
                byts = ws[0].bytes() + 2 * M * K + 2 * M * N
                res.append(dict(kind=name, M=M, N=N, K=K, avg_launch_us=round(us, 2), gbs=round(byts / us / 1e3, 1),
                                frac_of_hbm_peak=round(byts / us / 1e3 / HBM_PEAK_GBS, 4)))
                A.free()
                Cd.free()
            for w in ws:
                w.free()
    return res


def attention_sweep(xh, iters=10):
    """GQA attention, 32 query / 8 KV heads, head size 128: decode at batch 1 / 16 / 64 and context
    1024 / 4096 / 16384 over FP16 and INT8 caches (achieved GB/s against B ctx 8 128 2 e bytes, e = 2
    or 1 + 4/128) and the causal prefill of 4 x 2048 tokens (TFLOP/s on the causal-halved flops)."""
    qh, kvh, D = 32, 8, 128
    scale = 1.0 / np.sqrt(D)
    out = []
    for int8 in (0, 1):
        for B in (1, 16, 64):
            cache = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, kvh, 16384, D)
            q = xh.DeviceBuffer(B * qh * D * 2)
            q.zero()
            o = xh.DeviceBuffer(B * qh * D * 2)
            for ctx in (1024, 4096, 16384):
                for _ in range(2):
                    xh.attention(cache, q.ptr, qh * D, o.ptr, qh * D, xh.BF16, B, 1, qh, scale, ctx - 1)
                xh.synchronize()
                t = xh.Timer()
                t.start()
                for _ in range(iters):
                    xh.attention(cache, q.ptr, qh * D, o.ptr, qh * D, xh.BF16, B, 1, qh, scale, ctx - 1)
                us = t.stop() * 1e3 / iters
                byts = B * ctx * kvh * D * 2 * ((1 + 4.0 / D) if int8 else 2) + B * qh * D * 2 * 2
                out.append(dict(phase="decode", kv="int8" if int8 else "fp16", batch=B, ctx=ctx, avg_launch_us=round(us, 2),
                                gbs=round(byts / us / 1e3, 1), frac_of_hbm_peak=round(byts / us / 1e3 / HBM_PEAK_GBS, 4)))
            cache.free()
    B, S = 4, 2048
    stride = (qh + 2 * kvh) * D
    # N(0, 1) rows (bf16): the running maxima move as they do on real activations (all-zero rows never rescale)
    qkv = xh.DeviceBuffer.from_numpy(xh.f32_to_bf16_bits(np.random.default_rng(5).standard_normal((B * S, stride), dtype=np.float32)))
    o = xh.DeviceBuffer(B * S * qh * D * 2)
    flops = 4.0 * B * qh * S * S * D / 2
    for int8 in (0, 1):
        cache = xh.KVCache(xh.INT8 if int8 else xh.FP16, B, kvh, S, D)
        xh.rope_kvstore(cache, qkv.ptr, xh.BF16, stride, B, S, qh, None, 0)
        xh.attention(cache, qkv.ptr, stride, o.ptr, qh * D, xh.BF16, B, S, qh, scale, 0)
        xh.synchronize()
        t = xh.Timer()
        t.start()
        for _ in range(3):
            xh.attention(cache, qkv.ptr, stride, o.ptr, qh * D, xh.BF16, B, S, qh, scale, 0)
        us = t.stop() * 1e3 / 3
        out.append(dict(phase="prefill", kv="int8" if int8 else "fp16", batch=B, seq=S, avg_launch_us=round(us, 1),
                        tflops=round(flops / us / 1e6, 1), frac_of_bf16_mfma_peak=round(flops / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)))
        cache.free()
    return out


def moe_layer(xh, iters=5):
    """Mixtral-8x7B-shape sparse MLP: hidden 4096, FFN 14336, 8 experts, top-2, INT8 per-channel expert
    weights, 256 tokens with N(0,1) router logits.  1.409 GB of expert weights and 180.4 GFLOP per pass."""
    H, I, E, T = 4096, 14336, 8, 256
    rng = np.random.default_rng(4)
    moe = xh.MoE(H, I, E, T, np.zeros((H, E), np.float32), np.ones(H, np.float32))
    gq, gs, _ = synth_codes(rng, 0, H, 2 * I)
    dq, ds, _ = synth_codes(rng, 0, I, H)
    for e in range(E):
        moe.set_expert(e, xh.Weight(xh.W_INT8, H, 2 * I, gq, gs, None, flags=xh.WF_GATEUP), xh.Weight(xh.W_INT8, I, H, dq, ds, None))
    x = xh.DeviceBuffer.from_numpy(rng.standard_normal((T, H), dtype=np.float32))
    y = xh.DeviceBuffer(T * H * 4)
    lg = xh.DeviceBuffer.from_numpy(rng.standard_normal((T, E), dtype=np.float32))
    moe.forward(x.ptr, y.ptr, T, True, lg.ptr)
    xh.synchronize()
    t0 = time.time()
    for _ in range(iters):
        moe.forward(x.ptr, y.ptr, T, True, lg.ptr)
    xh.synchronize()
    us = (time.time() - t0) * 1e6 / iters
    t0 = time.time()
    for _ in range(4 * iters):
        moe.forward(x.ptr, y.ptr, T, True, lg.ptr, want_routing=False)
    xh.synchronize()
    us_queued = (time.time() - t0) * 1e6 / (4 * iters)
    # one token (a decode step): two of the eight experts work, 352 MB of their weights
    moe.forward(x.ptr, y.ptr, 1, True, lg.ptr, want_routing=False)
    xh.synchronize()
    t0 = time.time()
    for _ in range(20 * iters):
        moe.forward(x.ptr, y.ptr, 1, True, lg.ptr, want_routing=False)
    xh.synchronize()
    us_one = (time.time() - t0) * 1e6 / (20 * iters)
    wbytes, flops = 8 * (4096 * 28672 + 14336 * 4096), 512 * 3 * 2 * 4096 * 14336
    moe.free()
    return dict(tokens=T, experts=E, us_per_layer=round(us, 1), us_per_layer_no_wait=round(us_queued, 1),
                weight_gbs=round(wbytes / us_queued / 1e3, 1), frac_of_hbm_peak=round(wbytes / us_queued / 1e3 / HBM_PEAK_GBS, 4),
                tflops=round(flops / us_queued / 1e6, 1), us_per_layer_one_token=round(us_one, 1),
                one_token_weight_gbs=round(wbytes / 4 / us_one / 1e3, 1),
                note="us_per_layer: wall time of xfthip_moe_forward with the routing copied back to the host (one wait a call); "
                     "us_per_layer_no_wait (the rates are quoted on it): calls that return no routing, queued back to back (nothing waits: the row "
                     "counts stay on the device)")


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
    ap.add_argument("--pmc-workload", action="store_true", help="counter workload for rocprofv3 --pmc: a plain copy kernel of known size, then every distinct decode GEMV of the model once; prints no result line")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"), help="summarise the two counter CSVs of the --pmc-workload runs (CPU only)")
    ap.add_argument("--eager", action="store_true", help="launch decode kernels one by one instead of replaying the captured graph (for per-kernel profiling)")
    ap.add_argument("--no-extras", action="store_true", help="skip the extra measurements (batch 32 / UINT4 decode, GEMM sweep, attention sweep, sparse MLP)")
    ap.add_argument("--prefill-gemm", action="store_true", help="only the weight-only GEMM sweep: M = 256, 2048 against the MFMA peak, M = 1, 8, 32 against the HBM peak (one JSON line)")
    ap.add_argument("--attention", action="store_true", help="only the GQA attention sweep (one JSON line)")
    ap.add_argument("--moe", action="store_true", help="only the sparse-MLP layer (one JSON line)")
    ap.add_argument("--no-live-traffic", action="store_true", help="do not run the two rocprofv3 counter passes for roofline.traffic (the recorded figure under profiles/ is reported instead)")
    ap.add_argument("--stream-floor", action="store_true", help="only the read-only streaming floor at the decode GEMVs' byte counts (one JSON line)")
    args = ap.parse_args()
    if args.pmc_summary:
        pmc_summary(*args.pmc_summary)
        return
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no collectives are part of it)", file=sys.stderr)
        sys.exit(2)

    # HBM counters of the dominant kernel, measured by two profiler passes over child runs of this file: only in the
    # full default run (the headline configuration), and first, while this process has not touched the GPU
    single = args.prefill_gemm or args.attention or args.moe or args.stream_floor or args.pmc_workload or args.eager or args.no_extras
    live = None
    if not single and not args.no_live_traffic and args.weights == "int8" and args.batch == 1 and args.kv == "fp16":
        live = live_traffic()

    from xfastertransformer_amd import capi as xh
    xh.init(0)
    if args.prefill_gemm:
        print(json.dumps({"prefill_gemm": [r for M in (256, 2048) for r in prefill_gemm_sweep(xh, M)], "peak_tflops": MFMA_BF16_PEAK_TFLOPS,
                          "gemm_few_rows": gemm_few_rows_sweep(xh), "hbm_peak_gbs": HBM_PEAK_GBS}))
        return
    if args.attention:
        print(json.dumps({"attention": attention_sweep(xh), "hbm_peak_gbs": HBM_PEAK_GBS, "peak_tflops": MFMA_BF16_PEAK_TFLOPS}))
        return
    if args.moe:
        print(json.dumps({"moe": moe_layer(xh)}))
        return
    if args.stream_floor:
        print(json.dumps({"stream_floor": stream_floor(xh), "hbm_peak_gbs": HBM_PEAK_GBS}))
        return
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
    traffic_source = "recorded counter run, profiles/qgemm_skinny_int8_bs1_hbm_traffic.txt (not measured in this run)"
    if live is not None:
        traffic = live[dom["key"]]
        traffic_source = ("two rocprofv3 --pmc passes (FETCH_SIZE, WRITE_SIZE) over child runs of `bench.py --pmc-workload` started by "
                          "this run, each scaled by the same counter over the library's 256 MiB copy kernel")

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
        "data": "synthetic: integer codes drawn as N(0, 0.02) weights quantise to, one layer's codes uploaded as 32 distinct device weights",
        "config": {"workload": "configs[3]: 32-layer Llama-2-7B-shape, %s weight-only, %s KV, batch %d, "
                               "%d-token prompt, greedy decode" % (args.weights.upper(), args.kv.upper(), B, args.prompt),
                   "batch": B, "prompt": args.prompt, "weights": args.weights, "kv": args.kv},
        "ttft_ms": round(ttft_ms, 2),
        "ttft_warm_ms": round(ttft_warm_ms, 2),
        "step_hbm_bytes": int(step_bytes),
        "step_hbm_frac": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": {"bound": "hbm", "kernel": dom["name"], "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                     "traffic_source": traffic_source,
                     "avg_launch_us": round(dom["us"], 3), "bytes_per_launch": int(dom["bytes"])},
        "other_kernels": [{"kernel": g["name"], "launches_per_layer": g["launches"], "avg_launch_us": round(g["us"], 3),
                           "bytes_per_launch": int(g["bytes"]),
                           "frac": round(g["bytes"] / g["us"] / 1e3 / HBM_PEAK_GBS, 4)} for g in others],
    }
    if not args.no_extras:
        # free the main model before the other points of the metric are built
        model.free()
        for ws in layer_weights:
            for w in ws:
                w.free()
        lmw.free()
        extra = {"decode": []}
        for k2, b2 in ((0, 32), (1, 1), (1, 32)):
            if (k2, b2) != (kind, B):
                extra["decode"].append(decode_run(xh, k2, b2, args.prompt, 64, 8))
        # the INT8 KV cache at the batch where the cache is most of the step's bytes
        extra["decode"].append(decode_run(xh, 0, 32, args.prompt, 64, 8, kv_int8=True))
        extra["prefill_gemm"] = prefill_gemm_sweep(xh, 2048)
        extra["gemm_few_rows"] = gemm_few_rows_sweep(xh)
        extra["attention"] = attention_sweep(xh)
        extra["moe"] = moe_layer(xh)
        # what the bytes of a decode layer's four GEMVs cost as a pure read (out-proj, down, QKV, gate/up)
        extra["stream_floor"] = stream_floor(xh)
        result["extra"] = extra
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(kind, host, shapes, B, args.prompt)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
