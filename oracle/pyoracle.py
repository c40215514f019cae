"""ctypes binding of the CPU oracle (oracle/liboracle.so) and, when present, of the
reference's own in-tree kernels (oracle/_ref/libxft_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the CPU-baseline
leg of the benchmark.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_REF = os.path.join(_HERE, "_ref", "libxft_ref.so")

W_INT8, W_UINT4, W_NF4, W_W8A8, W_BF16 = 0, 1, 2, 3, 4
EPI_NONE, EPI_BIAS, EPI_SILU, EPI_GELU, EPI_RESMUL, EPI_RESIDENTIAL, EPI_RESEXT, EPI_BIAS_RELU = range(8)


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is mounted)."""
    if force or not os.path.exists(_LIB):
        subprocess.check_call(["make", "-C", _HERE, "-s", "all"])


def _load():
    if not os.path.exists(_LIB):
        build()
    return C.CDLL(_LIB)


lib = _load()


def host_has_avx512():
    try:
        with open("/proc/cpuinfo") as f:
            flags = f.read()
        return all(x in flags for x in ("avx512f", "avx512bw", "avx512vl", "avx512_bf16"))
    except OSError:
        return False


def load_ref():
    """The reference's in-tree kernels, or None (library absent / host lacks AVX-512)."""
    if not os.path.exists(_REF) or not host_has_avx512():
        return None
    return C.CDLL(_REF)


def p(a):
    """Raw pointer of a C-contiguous numpy array (None -> NULL)."""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


lib.orc_f32_to_bf16.restype = C.c_uint16
lib.orc_f32_to_bf16.argtypes = [C.c_float]
lib.orc_f32_to_bf16_hw.restype = C.c_uint16
lib.orc_f32_to_bf16_hw.argtypes = [C.c_float]
lib.orc_f32_to_fp16.restype = C.c_uint16
lib.orc_f32_to_fp16.argtypes = [C.c_float]
lib.orc_vexp.restype = C.c_float
lib.orc_vexp.argtypes = [C.c_float]
lib.orc_nf4_codebook.restype = C.POINTER(C.c_float)
lib.orc_num_threads.restype = C.c_int


# --------------------------------------------------------------------------- conversions
def to_bf16(x):
    x = f32(x)
    out = np.empty(x.shape, np.uint16)
    lib.orc_f32_to_bf16_array(p(x), p(out), C.c_int64(x.size))
    return out


def from_bf16(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, np.float32)
    lib.orc_bf16_to_f32_array(p(b), p(out), C.c_int64(b.size))
    return out


def round_bf16(x):
    return from_bf16(to_bf16(x))


def to_fp16(x):
    x = f32(x)
    out = np.empty(x.shape, np.uint16)
    lib.orc_f32_to_fp16_array(p(x), p(out), C.c_int64(x.size))
    return out


def from_fp16(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.orc_fp16_to_f32_array(p(h), p(out), C.c_int64(h.size))
    return out


def vexp(x):
    x = f32(x)
    out = np.empty_like(x)
    lib.orc_vexp_array(p(x), p(out), C.c_int64(x.size))
    return out


def nf4_codebook():
    return np.array([lib.orc_nf4_codebook()[i] for i in range(16)], np.float32)


# --------------------------------------------------------------------------- weights
class QWeight:
    """A quantised [K,N] weight in the reference's pre-pack convention:
    int8 [K,N]; uint4/nf4 [K,N/2] bytes with column n in the low nibble for even n."""

    def __init__(self, kind, K, N, q, scale, zero=None):
        self.kind, self.K, self.N = kind, K, N
        self.q, self.scale, self.zero = q, scale, zero
        self.colsum = None


def quantize(kind, W):
    W = f32(W)
    K, N = W.shape
    scale = np.empty(N, np.float32)
    if kind in (W_INT8, W_W8A8):
        q = np.empty((K, N), np.int8)
        zero = np.zeros(N, np.float32)
        lib.orc_quantize_int8_sym(p(W), K, N, p(q), p(scale), p(zero))
        w = QWeight(kind, K, N, q, scale, zero)
        if kind == W_W8A8:
            w.colsum = np.empty(N, np.float32)
            lib.orc_w8a8_colsum(p(q), K, N, p(w.colsum))
        return w
    q = np.empty((K, N // 2), np.uint8)
    if kind == W_UINT4:
        zero = np.empty(N, np.float32)
        lib.orc_quantize_uint4_asym(p(W), K, N, p(q), p(scale), p(zero))
        return QWeight(kind, K, N, q, scale, zero)
    if kind == W_NF4:
        lib.orc_quantize_nf4(p(W), K, N, p(q), p(scale))
        return QWeight(kind, K, N, q, scale, None)
    raise ValueError(kind)


def dequant(w):
    out = np.empty((w.K, w.N), np.float32)
    lib.orc_dequant(w.kind, p(w.q), p(w.scale), p(w.zero), w.K, w.N, p(out))
    return out


def dequant_bf16(w):
    out = np.empty((w.K, w.N), np.uint16)
    lib.orc_dequant_bf16(w.kind, p(w.q), p(w.scale), p(w.zero), w.K, w.N, p(out))
    return out


def qgemm(w, A, epi=EPI_NONE, bias=None, res=None, gamma=1.0, f64=False):
    A = f32(A)
    M, K = A.shape
    assert K == w.K
    Cm = np.empty((M, w.N), np.float32)
    if f64:
        lib.orc_qgemm_f64(w.kind, M, w.N, K, p(A), K, p(w.q), p(w.scale), p(w.zero), p(Cm), w.N)
        return Cm
    bias = None if bias is None else f32(bias)
    res = None if res is None else f32(res)
    ldres = 0 if res is None else res.shape[1]
    if w.kind == W_W8A8:
        rc = lib.orc_w8a8_gemm(M, w.N, K, p(A), K, p(w.q), p(w.scale), p(w.zero), p(w.colsum), p(Cm), w.N, epi,
                               p(bias), p(res), ldres, C.c_float(gamma))
        assert rc == 0
        return Cm
    lib.orc_qgemm(w.kind, M, w.N, K, p(A), K, p(w.q), p(w.scale), p(w.zero), p(Cm), w.N, epi, p(bias), p(res),
                  ldres, C.c_float(gamma))
    return Cm


def gemm_f32(A, W, epi=EPI_NONE, bias=None, res=None, gamma=1.0):
    A, W = f32(A), f32(W)
    M, K = A.shape
    N = W.shape[1]
    Cm = np.empty((M, N), np.float32)
    bias = None if bias is None else f32(bias)
    res = None if res is None else f32(res)
    ldres = 0 if res is None else res.shape[1]
    lib.orc_gemm_f32(M, N, K, p(A), K, p(W), N, p(Cm), N, epi, p(bias), p(res), ldres, C.c_float(gamma))
    return Cm


_DEQ_CACHE = {}


def blas_gemm(w, A, epi=EPI_NONE, bias=None, res=None, gamma=1.0):
    """A . deq(w) with numpy's sgemm on the weight dequantised once per QWeight object (kept until
    clear_blas_cache()); epilogues NONE / BIAS / RESIDENTIAL / RESEXT as apply_epilogue has them."""
    A = f32(A)
    Wd = None
    if not isinstance(w, QWeight):
        Wd = f32(w)
    elif A.shape[0] > 8 or w.kind not in (W_INT8, W_UINT4):
        key = id(w)
        if key not in _DEQ_CACHE:
            _DEQ_CACHE[key] = (w, dequant(w))
        Wd = _DEQ_CACHE[key][1]
    if A.shape[0] <= 8 and isinstance(w, QWeight) and w.kind in (W_INT8, W_UINT4):
        # few rows: stream the integer codes once (a quarter or an eighth of the fp32 bytes)
        out = np.empty((A.shape[0], w.N), np.float32)
        rc = lib.orc_qgemm_skinny(w.kind, A.shape[0], w.N, w.K, p(A), w.K, p(w.q), p(w.scale), p(w.zero), p(out), w.N)
        assert rc == 0
    elif A.shape[0] <= 8:
        # one threaded sgemv per row (the skinny sgemm of the BLAS behind numpy runs on one core)
        out = np.stack([a @ Wd for a in A])
    else:
        out = A @ Wd
    if epi == EPI_BIAS:
        out += f32(bias)
    elif epi in (EPI_RESIDENTIAL, EPI_RESEXT):
        if bias is not None:
            out += f32(bias)
        out += f32(res) if epi == EPI_RESIDENTIAL else np.float32(gamma) * f32(res)
    elif epi != EPI_NONE:
        raise ValueError("blas_gemm: epilogue %d not offered" % epi)
    return out


def clear_blas_cache():
    _DEQ_CACHE.clear()


def w8a8_quantize_rows(A):
    A = f32(A)
    M, K = A.shape
    qa = np.empty((M, K), np.int8)
    s, z, sm = (np.empty(M, np.float32) for _ in range(3))
    lib.orc_w8a8_quantize_rows(M, K, p(A), K, p(qa), K, p(s), p(z), p(sm))
    return qa, s, z, sm


# --------------------------------------------------------------------------- norm / rope
def rmsnorm(x, weight, eps=1e-6):
    x = f32(x)
    out = np.empty_like(x)
    rows, cols = x.shape
    lib.orc_rmsnorm(p(out), p(x), p(f32(weight)), rows, cols, -1, -1, C.c_float(eps))
    return out


def layernorm(x, gamma, beta, eps=1e-5):
    x = f32(x)
    out = np.empty_like(x)
    rows, cols = x.shape
    lib.orc_layernorm(p(out), p(x), p(f32(gamma)), p(f32(beta)), rows, cols, -1, -1, C.c_float(eps))
    return out


def rope_tables(dim, max_pos, base=10000, scaling=1.0):
    half = (dim + 1) // 2
    cos = np.empty((max_pos, half), np.float32)
    sin = np.empty((max_pos, half), np.float32)
    lib.orc_rope_tables(dim, max_pos, int(base), C.c_float(scaling), p(cos), p(sin))
    return cos, sin


def rope_apply(q, k, q_stride, k_stride, cos, sin, qk_shape, pos):
    """In place on fp32 q/k (flat arrays); qk_shape = (batch, seq, qHeads, headSize, kvHeads)."""
    lib.orc_rope_apply(p(q), p(k), q_stride, k_stride, p(cos), p(sin), cos.shape[1], p(i32(qk_shape)),
                       p(i32(pos)))


def rope_apply_tokens(q, k, cos, sin, q_stride, k_stride, dim, tokens, q_heads, k_heads, pos):
    lib.orc_rope_apply_tokens(p(q), p(k), p(cos), p(sin), q_stride, k_stride, dim, tokens, q_heads, k_heads,
                              p(i32(pos)))


# --------------------------------------------------------------------------- KV cache
class KVCache:
    """One layer's K or V cache, [B][H][maxSeq][D] (+ scales [B][H][maxSeq] when INT8)."""

    def __init__(self, int8, B, H, max_seq, D):
        self.int8, self.B, self.H, self.S, self.D = int(int8), B, H, max_seq, D
        self.data = np.zeros((B, H, max_seq, D), np.int8 if int8 else np.uint16)
        self.scales = np.zeros((B, H, max_seq), np.float32)

    def store(self, b, past, rows, kv_stride=None):
        """rows: fp32 [n, H*D] (or wider with kv_stride)."""
        rows = f32(rows)
        n = rows.shape[0]
        lib.orc_kv_store(self.int8, self.B, self.H, self.S, self.D, p(self.data), p(self.scales), b, past, n,
                         p(rows), kv_stride or rows.shape[1])

    def as_f32(self):
        if self.int8:
            return self.data.astype(np.float32) * self.scales[..., None]
        return from_fp16(self.data)


def kv_quantize_row(x):
    x = f32(x)
    q = np.empty(x.shape, np.int8)
    s = np.zeros(1, np.float32)
    lib.orc_kv_quantize_row(p(q), p(s), p(x), x.size)
    return q, s[0]


# --------------------------------------------------------------------------- attention
def cross_attn_by_head(q, k, v, q_heads, kv_heads, D, in_lens, past_lens, scale, kc, vc):
    """q: fp32 [tokens, q_heads*D]; k, v: fp32 [tokens, kv_heads*D]. Stores new rows, returns output."""
    q, k, v = f32(q), f32(k), f32(v)
    out = np.zeros_like(q)
    B = len(in_lens)
    lib.orc_cross_attn_by_head(p(out), p(q), p(k), p(v), q_heads, kv_heads, D, q.shape[1], q.shape[1], k.shape[1],
                               B, p(i32(in_lens)), p(i32(past_lens)), C.c_float(scale), kc.int8, kc.B, kc.S,
                               p(kc.data), p(kc.scales), p(vc.data), p(vc.scales))
    return out


def cross_attn_sharded_head(q, present, q_heads, kv_heads, D, scale, splits, kc, vc):
    q = f32(q)
    out = np.zeros_like(q)
    B = q.shape[0]
    lib.orc_cross_attn_sharded_head(p(out), p(q), present, q_heads, kv_heads, D, q.shape[1], q.shape[1], B,
                                    C.c_float(scale), splits, kc.int8, kc.B, kc.S, p(kc.data), p(kc.scales),
                                    p(vc.data), p(vc.scales))
    return out


def flash_prefill(q, k_bf16, v_bf16, q_heads, kv_heads, D, in_lens, past_lens, scale, kv_stride=None):
    """q fp32 [tokens, q_heads*D]; k_bf16/v_bf16: uint16 views with row stride kv_stride."""
    q = f32(q)
    out = np.zeros_like(q)
    lib.orc_flash_prefill(p(out), p(q), p(k_bf16), p(v_bf16), q_heads, kv_heads, D, q.shape[1], q.shape[1],
                          kv_stride or k_bf16.shape[1], len(in_lens), p(i32(in_lens)), p(i32(past_lens)),
                          C.c_float(scale))
    return out


def attention_ref_f64(q, K, V, q_heads, kv_heads, D, in_lens, past_lens, scale):
    """K, V fp32 [B, kvH, S, D]."""
    q, K, V = f32(q), f32(K), f32(V)
    out = np.zeros_like(q)
    lib.orc_attention_ref_f64(p(out), p(q), p(K), p(V), q_heads, kv_heads, D, q.shape[1], q.shape[1], len(in_lens),
                              p(i32(in_lens)), p(i32(past_lens)), K.shape[2], C.c_float(scale))
    return out


def softmax_scaled(x, scale):
    x = f32(x).copy()
    lib.orc_softmax_scaled(p(x), C.c_float(scale), x.size)
    return x


# --------------------------------------------------------------------------- misc
def silu_sum(x):
    x = f32(x)
    M, N2 = x.shape
    out = np.empty((M, N2 // 2), np.float32)
    lib.orc_silu_sum(p(x), N2, p(out), N2 // 2, M, N2 // 2)
    return out


def moe_top2(logits):
    logits = f32(logits)
    M, N = logits.shape
    sel = np.empty((M, 2), np.int32)
    w = np.empty((M, 2), np.float32)
    lib.orc_moe_top2(p(logits), M, N, p(sel), p(w))
    return sel, w


def argmax(logits):
    logits = f32(logits)
    B, V = logits.shape
    ids = np.empty(B, np.int32)
    lib.orc_argmax(p(logits), B, V, p(ids))
    return ids


def num_threads():
    return lib.orc_num_threads()


# --------------------------------------------------------------------------- decoder layer / model
class LlamaLayerOracle:
    """One Llama-family decoder layer as the reference runs it for quantised weights
    (src/layers/decoder_layer.h:101-170, attention.h:267-496, mlp_llama.h:197-290):
    fp32 activations end to end; prefill attention through the flash-style path (Q/K/V
    narrowed to bf16, attention.h:1121-1188), decode attention over the FP16/INT8 cache.

    rounding="bf16" instead narrows activations to bf16 where the GPU pipeline does
    (normalised input, qkv, rotated q, attention output, SwiGLU output), which isolates
    kernel error from the declared precision of the activation format."""

    def __init__(self, hidden, inter, q_heads, kv_heads, head, wqkv, wo, wgateup, wdown, ln1, ln2, kv_int8=0,
                 batch=1, max_seq=256, eps=1e-6, rope_base=10000, max_pos=2048, rounding="fp32", gemm="oracle",
                 prefill_attention="flash", ln1_beta=None, ln2_beta=None, moe=None):
        self.hidden, self.inter, self.qh, self.kvh, self.D = hidden, inter, q_heads, kv_heads, head
        # moe = (router fp32 [hidden, experts], [(gateup, down) per expert]): the layer of MixtralLLM
        # (src/models/mixtral.h:25-54), whose MLP half is MixtralMLP; wgateup / wdown are then unused
        self.moe = moe
        # shifts given: the layer built over LayerNorm instead of RmsNorm (NormType::LN, decoder_layer.cpp:179-181)
        self.ln1_beta = None if ln1_beta is None else f32(ln1_beta)
        self.ln2_beta = None if ln2_beta is None else f32(ln2_beta)
        self.wqkv, self.wo, self.wgateup, self.wdown = wqkv, wo, wgateup, wdown
        self.ln1, self.ln2, self.eps = f32(ln1), f32(ln2), eps
        self.kc = KVCache(kv_int8, batch, kv_heads, max_seq, head)
        self.vc = KVCache(kv_int8, batch, kv_heads, max_seq, head)
        self.cos, self.sin = rope_tables(head, max_pos, rope_base)
        self.rounding = rounding
        # gemm="blas": C = A . deq(W) through the BLAS sgemm behind numpy on the weight dequantised
        # once (orc_dequant), for shapes where the scalar orc_qgemm would take minutes; same closed
        # form, fp32 accumulation in another order (tests/test_oracle_pins.py compares the two)
        self.gemm = gemm
        # prefill_attention="cache": a prefill from position 0 also takes the route the reference
        # takes when a past exists (crossAttnByHead: rows go to the FP16/INT8 cache first, fp32 scores
        # and probabilities over the cache) instead of the flash-style path, which narrows K, V and
        # the probabilities to bf16.  This is the precision the GPU attention kernel works at.
        self.prefill_attention = prefill_attention

    def _r(self, x):
        return round_bf16(x) if self.rounding == "bf16" else x

    def _mm(self, w, a, **kw):
        if self.gemm == "blas":
            return blas_gemm(w, a, **kw)
        if isinstance(w, QWeight):
            return qgemm(w, a, **kw)
        return gemm_f32(a, w, **kw)

    def forward(self, x, B, S, past):
        x = f32(x)
        T = B * S
        qcols, kvcols = self.qh * self.D, self.kvh * self.D
        xn = self._r(rmsnorm(x, self.ln1, self.eps) if self.ln1_beta is None else layernorm(x, self.ln1, self.ln1_beta, self.eps))
        qkv = self._r(self._mm(self.wqkv, xn))
        stride = qkv.shape[1]
        flat = qkv.reshape(-1)
        lib.orc_rope_apply(C.c_void_p(flat.ctypes.data), C.c_void_p(flat.ctypes.data + qcols * 4), stride, stride,
                           p(self.cos), p(self.sin), self.D // 2, p(i32([B, S, self.qh, self.D, self.kvh])),
                           p(i32(np.arange(past, past + S))))
        q = np.ascontiguousarray(qkv[:, :qcols])
        k = np.ascontiguousarray(qkv[:, qcols:qcols + kvcols])
        v = np.ascontiguousarray(qkv[:, qcols + kvcols:])
        q = self._r(q)
        scale = 1.0 / np.sqrt(self.D)
        if past == 0 and S > 1 and self.prefill_attention == "flash":
            att = flash_prefill(q, to_bf16(k), to_bf16(v), self.qh, self.kvh, self.D, [S] * B, [0] * B, scale)
            for b in range(B):
                self.kc.store(b, 0, k[b * S:(b + 1) * S])
                self.vc.store(b, 0, v[b * S:(b + 1) * S])
        else:
            att = cross_attn_by_head(q, k, v, self.qh, self.kvh, self.D, [S] * B, [past] * B, scale, self.kc, self.vc)
        att = self._r(att)
        x1 = self._mm(self.wo, att, epi=EPI_RESIDENTIAL, res=x)
        if self.moe is not None:
            return mixtral_mlp(x1, self.ln2, self.moe[0], self.moe[1], rounding=self.rounding)[0]
        xn2 = self._r(rmsnorm(x1, self.ln2, 1e-6) if self.ln2_beta is None else layernorm(x1, self.ln2, self.ln2_beta, 1e-6))
        h = self._r(silu_sum(self._mm(self.wgateup, xn2)))
        return self._mm(self.wdown, h, epi=EPI_RESIDENTIAL, res=x1)


class LlamaModelOracle:
    """Embedding (FP16 table) -> layers -> last-token final RMSNorm -> lm_head -> greedy argmax
    (src/models/common_decoder.h:315-589, src/searchers/sampling.cpp:22-131)."""

    def __init__(self, layers, embedding_fp16, final_norm, lm_head_f32, eps=1e-6):
        self.layers, self.emb, self.fn, self.lm, self.eps = layers, embedding_fp16, f32(final_norm), lm_head_f32, eps
        self.rounding = layers[0].rounding
        self.gemm = layers[0].gemm

    def step(self, ids, B, S, past):
        x = from_fp16(self.emb[np.asarray(ids).reshape(-1)])
        for L in self.layers:
            x = L.forward(x, B, S, past)
        last = x.reshape(B, S, -1)[:, -1, :]
        xn = rmsnorm(last, self.fn, self.eps)
        if self.rounding == "bf16":
            xn = round_bf16(xn)
        logits = f32(xn) @ f32(self.lm) if self.gemm == "blas" else gemm_f32(xn, self.lm)
        return logits, argmax(logits)


def mixtral_mlp(x, ln, router, experts, logits_override=None, do_norm=True, rounding="fp32"):
    """MixtralMLP::forward (src/layers/mlp_mixtral.h:85-187).  experts: list of (gateup QWeight,
    down QWeight) with gateup = cat(gate, up) [hidden, 2*inter].  Returns (out, sel, weights)."""
    x = f32(x)
    r = (lambda a: round_bf16(a)) if rounding == "bf16" else (lambda a: a)
    xn = r(rmsnorm(x, ln, 1e-6) if do_norm else x)
    logits = gemm_f32(xn, router) if logits_override is None else f32(logits_override)
    sel, w = moe_top2(logits)
    out = x.copy()
    for e, (gu, dn) in enumerate(experts):
        rows, slot = np.nonzero(sel == e)
        if rows.size == 0:
            continue
        order = np.argsort(rows, kind="stable")
        rows, slot = rows[order], slot[order]
        xe = np.ascontiguousarray(xn[rows])
        mm = lambda w, a: qgemm(w, a) if isinstance(w, QWeight) else gemm_f32(a, w)  # (plain fp32 / bf16-valued experts)
        h = r(silu_sum(mm(gu, xe)))
        eo = mm(dn, h)
        idx = i32(rows)
        wt = f32(w[rows, slot])
        lib.orc_scatter_add(p(out), out.shape[1], p(f32(eo)), out.shape[1], p(idx), p(wt), rows.size)
    return out, sel, w


# ---- attention over a block-paged BF16 cache (xft::invokeAttention) ------------------------------
# The reference's crossAttention (src/kernels/attention_kernels.cpp:24-112) per (sequence, head):
# store the new key / value rows at slot_mapping[b], scores = q . K^T over context + 1 tokens through
# the block table (fp32, xDNN small_sgemm_bf16bf16f32_b: closed source, textbook GEMM assumed),
# small_softmax_f32(scores, scale, n) = softmax(scale * scores) in fp32, out = P . V in fp32
# narrowed to bf16.  PARITY UNPINNED against the reference (no test of it there, xDNN kernels not in
# the tree); pinned against float64 brute force in tests/test_oracle_pins.py.  Sequence b uses row b
# of query / key / value and KV head hq // (q_heads // kv_heads): see include/layers_attention.h for
# how that differs from the reference's text.
def paged_attention_decode(q, k, v, kcache, vcache, block_tables, context_lens, slot_mapping, scale):
    """q [B, qH, D], k / v [B, kvH, D] fp32 holding bf16 values; kcache / vcache
    [blocks, block_size, kvH, D] fp32 holding bf16 values, updated in place.  Returns bf16-rounded
    fp32 [B, qH, D]."""
    B, qH, D = q.shape
    kvH = k.shape[1]
    bs = kcache.shape[1]
    kflat, vflat = kcache.reshape(-1, kvH, D), vcache.reshape(-1, kvH, D)
    out = np.zeros((B, qH, D), np.float32)
    for b in range(B):
        kflat[slot_mapping[b]] = k[b]
        vflat[slot_mapping[b]] = v[b]
    for b in range(B):
        n = int(context_lens[b]) + 1
        slots = [int(block_tables[b][t // bs]) * bs + t % bs for t in range(n)]
        for h in range(qH):
            kh = h // (qH // kvH)
            K, V = f32(kflat[slots, kh]), f32(vflat[slots, kh])
            s = (K @ f32(q[b, h])).astype(np.float32) * np.float32(scale)
            e = np.exp(s - s.max()).astype(np.float32)
            p = e / e.sum(dtype=np.float32)
            out[b, h] = round_bf16((p @ V).astype(np.float32))
    return out


def paged_attention_prefill(q, k, v, token_lens, kcache, vcache, slot_mapping, scale):
    """Causal self-attention per sequence over its own tokens (xft::selfAttention as invokeAttention
    calls it, attention_kernels.cpp:141-151: bf16 inputs, fp32 softmax) and every token's key / value
    row stored at its slot.  q [T, qH, D], k / v [T, kvH, D].  Returns bf16-rounded fp32 [T, qH, D]."""
    T, qH, D = q.shape
    kvH = k.shape[1]
    kflat, vflat = kcache.reshape(-1, kvH, D), vcache.reshape(-1, kvH, D)
    for t in range(T):
        kflat[slot_mapping[t]] = k[t]
        vflat[slot_mapping[t]] = v[t]
    out = np.zeros((T, qH, D), np.float32)
    first = 0
    for L in token_lens:
        for h in range(qH):
            kh = h // (qH // kvH)
            Q, K, V = f32(q[first:first + L, h]), f32(k[first:first + L, kh]), f32(v[first:first + L, kh])
            s = (Q @ K.T).astype(np.float32) * np.float32(scale)
            s = np.where(np.tril(np.ones((L, L), bool)), s, -np.inf)
            e = np.exp(s - s.max(1, keepdims=True)).astype(np.float32)
            p = e / e.sum(1, keepdims=True, dtype=np.float32)
            out[first:first + L, h] = round_bf16((p @ V).astype(np.float32))
        first += L
    return out


# ---- beam search (src/searchers/beam_search.cpp) ----------------------------------------------------
# Plain-Python restatement of BeamSearch::searchTopK / beam_search, BeamSearchScorer::process / finalize
# and BeamHypotheses.  Pinned in tests/test_oracle_pins.py by brute force: with enough beams to keep every
# prefix alive the best hypothesis must be the best of all vocab ** steps continuations.  The reference's
# log-softmax uses a vectorised polynomial exp (bert_util.h); float32 numpy exp / log here: scores agree to
# rounding, which can only matter at exact near-ties.
class BeamSearchOracle:
    def __init__(self, prompts, num_beams, max_len, eos, pad, vocab, keep=1, len_penalty=1.0, early=False):
        prompts = np.asarray(prompts, np.int64)
        self.batch, self.seq_len = prompts.shape
        self.nb, self.keep, self.max_len, self.eos, self.pad, self.vocab = num_beams, keep, max_len, eos, pad, vocab
        self.len_penalty, self.early = float(len_penalty), bool(early)
        self.k = 2 * num_beams  # :284 kVal
        self.rows = [list(prompts[b]) for b in range(self.batch) for _ in range(num_beams)]  # :285-291
        self.scores = np.full(self.batch * num_beams, -1e9, np.float32)  # :296-300
        self.scores[::num_beams] = 0.0
        self.tokens = [0] * (self.batch * num_beams)
        self.indices = [0] * (self.batch * num_beams)
        self.hyps = [[] for _ in range(self.batch)]  # (score, ids)
        self.worst = [1e9] * self.batch
        self.done = [False] * self.batch
        self.steps = 0

    def _add(self, b, ids, sum_logprobs):  # BeamHypotheses::add :89-104
        score = np.float32(sum_logprobs) / np.float32(float(len(ids)) ** self.len_penalty)
        if len(self.hyps[b]) < self.nb or score > self.worst[b]:
            self.hyps[b].append((float(score), list(ids)))
            if len(self.hyps[b]) > self.nb:
                self.hyps[b].sort(key=lambda h: h[0])
                self.hyps[b].pop(0)
                self.worst[b] = self.hyps[b][0][0]
            else:
                self.worst[b] = min(float(score), self.worst[b])

    def _hyps_done(self, b, best_sum, cur_len):  # :106-116
        if len(self.hyps[b]) < self.nb:
            return False
        if self.early:
            return True
        return self.worst[b] >= float(np.float32(best_sum) / np.float32(float(cur_len) ** self.len_penalty))

    def step(self, logits):
        """logits [batch * num_beams, vocab] of the rows' next token.  Returns (tokens, source rows)."""
        lg = f32(logits).reshape(self.batch * self.nb, self.vocab)
        mx = lg.max(axis=1, keepdims=True)
        logp = lg - (mx + np.log(np.exp(lg - mx, dtype=np.float32).sum(axis=1, keepdims=True, dtype=np.float32)))  # :27-66
        cur_len = len(self.rows[0])
        next_scores, next_tokens, next_indices = [], [], []
        for b in range(self.batch):
            el = []
            for j in range(self.nb):
                row = b * self.nb + j
                # the kVal largest under std::greater<pair<float, int>>: value, then the larger index (:470-481)
                order = sorted(range(self.vocab), key=lambda t: (-float(logp[row, t]), -t))[:self.k]
                el += [(np.float32(logp[row, t] + self.scores[row]), t, j) for t in order]
            el.sort(key=lambda e: (-float(e[0]), e[2]))  # tupleCompare :69-77 (stable where it leaves the order open)
            uniq = []
            for e in el:  # std::unique with uniqueCompare :79-81: adjacent equal (score, token)
                if uniq and uniq[-1][0] == e[0] and uniq[-1][1] == e[1]:
                    continue
                uniq.append(e)
            uniq += el[len(uniq):]  # what std::unique leaves behind its new end is read as it lies; pad the same way
            for e in uniq[:self.k]:
                next_scores.append(e[0]), next_tokens.append(e[1]), next_indices.append(e[2])
        new_scores = np.zeros(self.batch * self.nb, np.float32)
        new_tokens = [self.pad] * (self.batch * self.nb)
        new_indices = [0] * (self.batch * self.nb)
        for b in range(self.batch):  # BeamSearchScorer::process :137-193
            if self.done[b]:
                continue
            beam = 0
            for rank in range(self.k):
                tok, sc = next_tokens[b * self.k + rank], next_scores[b * self.k + rank]
                row = b * self.nb + next_indices[b * self.k + rank]
                if self.eos != -1 and tok == self.eos:
                    if rank >= self.nb:
                        continue
                    self._add(b, self.rows[row], sc)
                else:
                    new_scores[b * self.nb + beam], new_tokens[b * self.nb + beam], new_indices[b * self.nb + beam] = sc, tok, row
                    beam += 1
                    if beam == self.nb:
                        break
            assert beam == self.nb, "At most tokens can be equal to `eosTokenId`"
            # :187-190 reads nextScores with a stride of numBeams although a user sequence owns kVal entries
            best = max(float(x) for x in next_scores[b * self.nb:(b + 1) * self.nb])
            self.done[b] = self.done[b] or self._hyps_done(b, best, cur_len)
        self.scores, self.tokens, self.indices = new_scores, new_tokens, new_indices
        self.rows = [list(self.rows[self.indices[i]]) + [self.tokens[i]] for i in range(self.batch * self.nb)]  # :553-563
        self.steps += 1
        return list(self.tokens), list(self.indices)

    def is_done(self):  # :330-332
        return self.steps != 0 and (all(self.done) or len(self.rows[0]) >= self.max_len)

    def finalize(self):  # BeamSearchScorer::finalize :195-263
        for b in range(self.batch):
            if self.done[b]:
                continue
            for j in range(self.nb):
                self._add(b, self.rows[b * self.nb + j], self.scores[b * self.nb + j])
        best = []
        for b in range(self.batch):
            hs = sorted(self.hyps[b], key=lambda h: h[0])
            for _ in range(self.keep):
                best.append(hs.pop()[1])
        out_len = min(max(len(h) for h in best) + 1, self.max_len)
        out = np.full((len(best), out_len), self.pad, np.int32)
        for i, h in enumerate(best):
            if len(h) < self.max_len:
                out[i, :len(h)] = h
                out[i, len(h)] = self.eos
            else:
                out[i, :] = h[:self.max_len]
        return out
