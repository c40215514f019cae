"""ctypes binding of include/xft_hip.h plus small numpy <-> device helpers."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libxft_hip.so")

F32, BF16, FP16, INT8 = 0, 1, 2, 3
W_INT8, W_UINT4, W_NF4, W_W8A8, W_BF16 = 0, 1, 2, 3, 4
EPI_NONE, EPI_BIAS, EPI_SILU, EPI_GELU, EPI_RESMUL, EPI_RESIDENTIAL, EPI_RESEXT = range(7)
WF_NONE, WF_GATEUP = 0, 1

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `python -m xfastertransformer_amd.build` "
        "(there is no CPU fallback)")

lib = C.CDLL(LIB_PATH)
lib.xfthip_last_error.restype = C.c_char_p
lib.xfthip_weight_bytes.restype = C.c_size_t
lib.xfthip_weight_bytes.argtypes = [C.c_void_p]


class XftHipError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        raise XftHipError(lib.xfthip_last_error().decode())


_initialised = False


def init(device=0):
    global _initialised
    if not _initialised:
        check(lib.xfthip_init(device))
        _initialised = True


def device_info():
    name = C.create_string_buffer(256)
    cus = C.c_int()
    mem = C.c_size_t()
    check(lib.xfthip_device_info(name, 256, C.byref(cus), C.byref(mem)))
    return name.value.decode(), cus.value, mem.value


def copy_kernel(dst_ptr, src_ptr, nbytes, stream=None):
    check(lib.xfthip_copy_kernel(dst_ptr, src_ptr, C.c_size_t(nbytes), stream))


def read_kernel(src_ptr, nbytes, blocks=0, stream=None):
    """Read-only stream over nbytes (results discarded): the floor of a weight-streaming launch."""
    check(lib.xfthip_read_kernel(src_ptr, C.c_size_t(nbytes), int(blocks), stream))


def synchronize():
    check(lib.xfthip_device_synchronize())


class Stream:
    """A stream of default priority; pass `.h` wherever a call takes a stream."""

    def __init__(self):
        self.h = C.c_void_p()
        check(lib.xfthip_stream_create(C.byref(self.h)))

    def synchronize(self):
        check(lib.xfthip_stream_synchronize(self.h))

    def free(self):
        if self.h is not None:
            lib.xfthip_stream_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Graph:
    """Records the calls made on `stream` inside the `with` block and replays them with launch()."""

    def __init__(self, stream):
        self.stream, self.h = stream, None

    def __enter__(self):
        check(lib.xfthip_graph_begin(self.stream.h))
        return self

    def __exit__(self, exc_type, exc, tb):
        g = C.c_void_p()
        rc = lib.xfthip_graph_end(self.stream.h, C.byref(g))
        if exc_type is None:
            check(rc)
            self.h = g
        return False

    def launch(self, stream=None):
        check(lib.xfthip_graph_launch(self.h, (stream or self.stream).h))

    def free(self):
        if self.h is not None:
            lib.xfthip_graph_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _hp(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class DeviceBuffer:
    """A device allocation owned through the C-ABI."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        ptr = C.c_void_p()
        check(lib.xfthip_malloc(C.byref(ptr), C.c_size_t(self.nbytes)))
        self.ptr = ptr

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        check(lib.xfthip_memcpy_h2d(buf.ptr, _hp(a), C.c_size_t(a.nbytes), None))
        return buf

    def upload(self, a, offset=0):
        a = np.ascontiguousarray(a)
        assert offset + a.nbytes <= self.nbytes
        check(lib.xfthip_memcpy_h2d(C.c_void_p(self.ptr.value + offset), _hp(a), C.c_size_t(a.nbytes), None))

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        check(lib.xfthip_memcpy_d2h(_hp(out), self.ptr, C.c_size_t(out.nbytes), None))
        return out

    def zero(self):
        check(lib.xfthip_memset(self.ptr, 0, C.c_size_t(self.nbytes), None))
        synchronize()

    def at(self, byte_offset):
        return C.c_void_p(self.ptr.value + int(byte_offset))

    def free(self):
        if self.ptr is not None and self.ptr.value:
            lib.xfthip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def f32_to_bf16_bits(x):
    """Round-to-nearest-even narrowing of fp32 to bf16 bit patterns (normals)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    sub = (u & 0x7F800000) == 0
    r[sub] = (u[sub] >> 16).astype(np.uint16) & 0x8000
    return r


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


class Weight:
    """Handle of a packed quantised weight (xfthip_weight_create)."""

    def __init__(self, kind, K, N, q, scale=None, zero=None, flags=WF_NONE):
        self.kind, self.K, self.N, self.flags = kind, K, N, flags
        q = np.ascontiguousarray(q)
        scale = None if scale is None else np.ascontiguousarray(scale, np.float32)
        zero = None if zero is None else np.ascontiguousarray(zero, np.float32)
        h = C.c_void_p()
        check(lib.xfthip_weight_create(kind, K, N, _hp(q), _hp(scale), _hp(zero), flags, C.byref(h)))
        self.h = h

    def unpack(self):
        if self.kind in (W_UINT4, W_NF4):
            out = np.empty((self.K, self.N // 2), np.uint8)
        elif self.kind == W_BF16:
            out = np.empty((self.K, self.N), np.uint16)
        else:
            out = np.empty((self.K, self.N), np.int8)
        check(lib.xfthip_weight_unpack(self.h, _hp(out)))
        return out

    def dequant(self, out_dtype=F32):
        buf = DeviceBuffer(self.K * self.N * (4 if out_dtype == F32 else 2))
        check(lib.xfthip_weight_dequant(self.h, buf.ptr, out_dtype, None))
        synchronize()
        return buf.to_numpy(np.float32 if out_dtype == F32 else np.uint16, (self.K, self.N))

    def bytes(self):
        return lib.xfthip_weight_bytes(self.h)

    def free(self):
        if self.h is not None:
            lib.xfthip_weight_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def quantize_weight(kind, W):
    W = np.ascontiguousarray(W, np.float32)
    K, N = W.shape
    scale = np.empty(N, np.float32)
    zero = np.zeros(N, np.float32)
    q = np.empty((K, N), np.int8) if kind in (W_INT8, W_W8A8) else np.empty((K, N // 2), np.uint8)
    check(lib.xfthip_quantize_weight(kind, K, N, _hp(W), _hp(q), _hp(scale), _hp(zero)))
    return q, scale, (None if kind == W_NF4 else zero)


def gemm(w, A_dev, M, lda, C_dev, ldc, c_dtype=BF16, epi=EPI_NONE, bias=None, res=None, ldres=0, res_dtype=F32,
         gamma=1.0, stream=None):
    check(lib.xfthip_gemm(w.h, M, A_dev, lda, C_dev, ldc, c_dtype, epi, bias, res, ldres, res_dtype,
                          C.c_float(gamma), stream))


def gemm_gateup_silu(w, A_dev, M, lda, out_dev, ldo, out_dtype=BF16, stream=None):
    check(lib.xfthip_gemm_gateup_silu(w.h, M, A_dev, lda, out_dev, ldo, out_dtype, stream))


class Timer:
    """HIP-event timer on a given stream (None = default stream)."""

    def __init__(self):
        self.a, self.b = C.c_void_p(), C.c_void_p()
        check(lib.xfthip_event_create(C.byref(self.a)))
        check(lib.xfthip_event_create(C.byref(self.b)))

    def start(self, stream=None):
        check(lib.xfthip_event_record(self.a, stream))

    def stop(self, stream=None):
        check(lib.xfthip_event_record(self.b, stream))
        check(lib.xfthip_event_synchronize(self.b))
        ms = C.c_float()
        check(lib.xfthip_event_elapsed_ms(self.a, self.b, C.byref(ms)))
        return ms.value


# ---------------------------------------------------------------------------- norm / rope / KV / attention
def rmsnorm(out_dev, out_dtype, in_dev, in_dtype, weight_dev, rows, cols, i_stride=-1, o_stride=-1, eps=1e-6,
            stream=None):
    check(lib.xfthip_rmsnorm(out_dev, out_dtype, in_dev, in_dtype, weight_dev, rows, cols, i_stride, o_stride,
                             C.c_float(eps), stream))


class RopeTables:
    def __init__(self, dim, max_pos, base=10000, scaling=1.0):
        self.dim, self.max_pos = dim, max_pos
        self.cos, self.sin = C.c_void_p(), C.c_void_p()
        check(lib.xfthip_rope_tables_create(dim, max_pos, int(base), C.c_float(scaling), C.byref(self.cos),
                                            C.byref(self.sin)))

    def to_numpy(self):
        half = (self.dim + 1) // 2
        c = np.empty((self.max_pos, half), np.float32)
        s = np.empty((self.max_pos, half), np.float32)
        check(lib.xfthip_memcpy_d2h(_hp(c), self.cos, C.c_size_t(c.nbytes), None))
        check(lib.xfthip_memcpy_d2h(_hp(s), self.sin, C.c_size_t(s.nbytes), None))
        return c, s

    def free(self):
        if self.cos is not None:
            lib.xfthip_free(self.cos)
            lib.xfthip_free(self.sin)
            self.cos = self.sin = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def rotary_embedding(dtype, positions_dev, q_dev, k_dev, tables, dim, q_stride, k_stride, tokens, heads, head_size,
                     kv_heads, stream=None):
    check(lib.xfthip_rotary_embedding(dtype, positions_dev, q_dev, k_dev, tables.cos, tables.sin, dim, q_stride,
                                      k_stride, tokens, heads, head_size, kv_heads, stream))


class KVCache:
    def __init__(self, dtype, batch, kv_heads, max_seq, head_size):
        self.dtype, self.B, self.H, self.S, self.D = dtype, batch, kv_heads, max_seq, head_size
        h = C.c_void_p()
        check(lib.xfthip_kvcache_create(dtype, batch, kv_heads, max_seq, head_size, C.byref(h)))
        self.h = h

    def _np_dtype(self):
        return np.int8 if self.dtype == INT8 else np.uint16

    def export(self, which, sbhd=False):
        """Reference layouts: data [B][H][maxSeq][D] (fp16 bits / int8), or [maxSeq][B][H][D] with sbhd; scales [B][H][maxSeq]."""
        n = self.B * self.H * self.S
        data = DeviceBuffer(n * self.D * (1 if self.dtype == INT8 else 2))
        scales = DeviceBuffer(n * 4)
        scales.zero()
        fn = lib.xfthip_kvcache_export_sbhd if sbhd else lib.xfthip_kvcache_export
        check(fn(self.h, which, data.ptr, scales.ptr, None))
        synchronize()
        shape = (self.S, self.B, self.H, self.D) if sbhd else (self.B, self.H, self.S, self.D)
        return (data.to_numpy(self._np_dtype(), shape), scales.to_numpy(np.float32, (self.B, self.H, self.S)))

    def load(self, which, data, scales=None, sbhd=False):
        data = np.ascontiguousarray(data, self._np_dtype())
        assert data.shape == ((self.S, self.B, self.H, self.D) if sbhd else (self.B, self.H, self.S, self.D))
        d = DeviceBuffer.from_numpy(data)
        s = None
        if self.dtype == INT8:
            s = DeviceBuffer.from_numpy(np.ascontiguousarray(scales, np.float32))
        fn = lib.xfthip_kvcache_import_sbhd if sbhd else lib.xfthip_kvcache_import
        check(fn(self.h, which, d.ptr, None if s is None else s.ptr, None))
        synchronize()

    def reorder(self, dst_rows, src_rows, pos0, pos1, stream=None):
        """Row dst_rows[i] becomes a copy of row src_rows[i] over positions [pos0, pos1) (32-token blocks)."""
        d = np.ascontiguousarray(dst_rows, np.int32)
        s_ = np.ascontiguousarray(src_rows, np.int32)
        assert d.size == s_.size
        check(lib.xfthip_kvcache_reorder(self.h, _hp(d), _hp(s_), int(d.size), int(pos0), int(pos1), stream))

    def free(self):
        if self.h is not None:
            lib.xfthip_kvcache_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def gemm_gateup_silu_rmsnorm(w, x_dev, M, ldx, norm_w_dev, eps, out_dev, ldo, out_dtype, stream=None):
    check(lib.xfthip_gemm_gateup_silu_rmsnorm(w.h, M, x_dev, ldx, norm_w_dev, C.c_float(eps), out_dev, ldo, out_dtype, stream))


def gemm_qkv_rmsnorm_rope(w, cache, x_dev, M, ldx, norm_w_dev, eps, q_dev, ldq, q_heads, tables, position, pos_dev=None,
                          stream=None):
    check(lib.xfthip_gemm_qkv_rmsnorm_rope(w.h, cache.h, M, x_dev, ldx, norm_w_dev, C.c_float(eps), q_dev, ldq, q_heads,
                                           tables.cos, tables.sin, position, pos_dev, stream))


def rope_kvstore(cache, qkv_dev, dtype, stride, B, S, q_heads, tables, past, past_dev=None, stream=None):
    cos = None if tables is None else tables.cos
    sin = None if tables is None else tables.sin
    check(lib.xfthip_rope_kvstore(cache.h, qkv_dev, dtype, stride, B, S, q_heads, cos, sin, past, past_dev, stream))


def attention(cache, q_dev, q_stride, out_dev, o_stride, out_dtype, B, S, q_heads, scale, past, past_dev=None,
              stream=None):
    check(lib.xfthip_attention(cache.h, q_dev, q_stride, out_dev, o_stride, out_dtype, B, S, q_heads,
                               C.c_float(scale), past, past_dev, stream))


def attention_static(cache, q_dev, q_stride, out_dev, o_stride, out_dtype, B, S, q_heads, scale, past, past_dev=None,
                     stream=None):
    """xfthip_attention through the statically allocated split workspace (allocates nothing)."""
    check(lib.xfthip_attention_static(cache.h, q_dev, q_stride, out_dev, o_stride, out_dtype, B, S, q_heads,
                                      C.c_float(scale), past, past_dev, stream))


# ---------------------------------------------------------------------------- model driver
class ModelConfig(C.Structure):
    _fields_ = [("layers", C.c_int), ("hidden", C.c_int), ("intermediate", C.c_int), ("q_heads", C.c_int),
                ("kv_heads", C.c_int), ("head_size", C.c_int), ("vocab", C.c_int), ("max_batch", C.c_int),
                ("max_seq", C.c_int), ("max_tokens", C.c_int), ("max_pos_embed", C.c_int), ("rope_base", C.c_int),
                ("kv_dtype", C.c_int), ("rms_eps", C.c_float)]


class Model:
    def __init__(self, layers, hidden, intermediate, q_heads, kv_heads, head_size=128, vocab=0, max_batch=1,
                 max_seq=256, max_tokens=None, max_pos_embed=2048, rope_base=10000, kv_dtype=FP16, rms_eps=1e-6):
        self.cfg = ModelConfig(layers, hidden, intermediate, q_heads, kv_heads, head_size, vocab, max_batch, max_seq,
                               max_tokens or max_batch * max_seq, max(max_pos_embed, max_seq), rope_base, kv_dtype,
                               rms_eps)
        h = C.c_void_p()
        check(lib.xfthip_model_create(C.byref(self.cfg), C.byref(h)))
        self.h = h
        self._keep = []

    def set_layer(self, idx, qkv, o, gateup, down, ln1, ln2, qkv_bias=None, o_bias=None):
        self._keep += [qkv, o, gateup, down]
        f = lambda a: None if a is None else np.ascontiguousarray(a, np.float32)
        ln1, ln2, qkv_bias, o_bias = f(ln1), f(ln2), f(qkv_bias), f(o_bias)
        check(lib.xfthip_model_set_layer(self.h, idx, qkv.h, o.h, gateup.h, down.h, _hp(ln1), _hp(ln2), _hp(qkv_bias),
                                         _hp(o_bias)))

    def set_sparse_layer(self, idx, qkv, o, moe, ln1, qkv_bias=None, o_bias=None):
        """Layer idx = attention half + a sparse MLP (capi.MoE created with its own norm weight)."""
        self._keep += [qkv, o, moe]
        f = lambda a: None if a is None else np.ascontiguousarray(a, np.float32)
        ln1, qkv_bias, o_bias = f(ln1), f(qkv_bias), f(o_bias)
        check(lib.xfthip_model_set_attention(self.h, idx, qkv.h, o.h, _hp(ln1), _hp(qkv_bias), _hp(o_bias)))
        check(lib.xfthip_model_set_moe(self.h, idx, moe.h))

    def set_first_token_weights(self, idx, qkv, o, gateup, down):
        """A second weight set of layer idx for the prompt pass only (None x 4 drops it)."""
        ws = [qkv, o, gateup, down]
        self._keep += [w for w in ws if w is not None]
        check(lib.xfthip_model_set_first_token_weights(self.h, idx, *[None if w is None else w.h for w in ws]))

    def set_head(self, embedding_fp16, final_norm, lm_head):
        self._keep.append(lm_head)
        e = np.ascontiguousarray(embedding_fp16, np.uint16)
        fn = np.ascontiguousarray(final_norm, np.float32)
        check(lib.xfthip_model_set_head(self.h, _hp(e), _hp(fn), lm_head.h))

    def set_prefix(self, ids, stream=None):
        ids = np.ascontiguousarray(ids, np.int32).reshape(-1)
        check(lib.xfthip_model_set_prefix(self.h, _hp(ids), len(ids), stream))

    def prefill_after_prefix(self, ids, want_logits=False, stream=None):
        """ids [B, S]: what follows the shared prefix in each sequence."""
        ids = np.ascontiguousarray(ids, np.int32)
        B, S = ids.shape
        logits = np.empty((B, self.cfg.vocab), np.float32) if want_logits else None
        check(lib.xfthip_model_prefill_after_prefix(self.h, _hp(ids), B, S, _hp(logits), stream))
        return self.last_ids(B), logits

    def layer_forward(self, idx, x_in_dev, x_out_dev, B, S, past, stride=None, stream=None):
        stride = stride or self.cfg.hidden
        check(lib.xfthip_model_layer_forward(self.h, idx, x_in_dev, stride, x_out_dev, stride, B, S, past, stream))

    def prefill(self, ids, want_logits=False, stream=None):
        ids = np.ascontiguousarray(ids, np.int32)
        B, S = ids.shape
        logits = np.empty((B, self.cfg.vocab), np.float32) if want_logits else None
        check(lib.xfthip_model_prefill(self.h, _hp(ids), B, S, _hp(logits), stream))
        return self.last_ids(B), logits

    def decode(self, steps, B, stream=None):
        out = np.empty((steps, B), np.int32)
        check(lib.xfthip_model_decode(self.h, steps, _hp(out), stream))
        return out

    def decode_untracked(self, steps, stream=None):
        check(lib.xfthip_model_decode(self.h, steps, None, stream))

    def use_graph(self, enable):
        check(lib.xfthip_model_use_graph(self.h, int(bool(enable))))

    def use_fusion(self, enable):
        check(lib.xfthip_model_use_fusion(self.h, int(bool(enable))))

    def decode_mode(self):
        return int(lib.xfthip_model_decode_mode(self.h))

    def seq_prefill(self, row, ids, want_logits=False, stream=None):
        ids = np.ascontiguousarray(ids, np.int32).ravel()
        logits = np.empty(self.cfg.vocab, np.float32) if want_logits else None
        check(lib.xfthip_model_seq_prefill(self.h, int(row), _hp(ids), len(ids), _hp(logits), stream))
        return logits

    def seq_decode(self, rows, stream=None):
        rows = np.ascontiguousarray(rows, np.int32)
        out = np.empty(len(rows), np.int32)
        check(lib.xfthip_model_seq_decode(self.h, _hp(rows), len(rows), _hp(out), stream))
        return out

    def seq_logits(self, row):
        out = np.empty(self.cfg.vocab, np.float32)
        check(lib.xfthip_model_seq_logits(self.h, int(row), _hp(out)))
        return out

    def seq_set_next_id(self, row, tok):
        check(lib.xfthip_model_seq_set_next_id(self.h, int(row), int(tok)))

    def seq_release(self, row):
        check(lib.xfthip_model_seq_release(self.h, int(row)))

    def seq_reorder(self, dst_rows, src_rows, pos0, pos1, stream=None):
        """Cache row dst_rows[i] becomes a copy of row src_rows[i] over positions [pos0, pos1)."""
        d = np.ascontiguousarray(dst_rows, np.int32)
        s_ = np.ascontiguousarray(src_rows, np.int32)
        assert d.size == s_.size
        check(lib.xfthip_model_seq_reorder(self.h, _hp(d), _hp(s_), int(d.size), int(pos0), int(pos1), stream))

    def set_next_ids(self, ids, stream=None):
        ids = np.ascontiguousarray(ids, np.int32)
        check(lib.xfthip_model_set_next_ids(self.h, _hp(ids), stream))

    def last_ids(self, B):
        ids = np.empty(B, np.int32)
        pos = C.c_int()
        check(lib.xfthip_model_last_ids(self.h, _hp(ids), C.byref(pos)))
        return ids

    def logits(self, B):
        ptr = C.c_void_p()
        check(lib.xfthip_model_logits(self.h, C.byref(ptr)))
        out = np.empty((B, self.cfg.vocab), np.float32)
        check(lib.xfthip_memcpy_d2h(_hp(out), ptr, C.c_size_t(out.nbytes), None))
        return out

    def free(self):
        if self.h is not None:
            lib.xfthip_model_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def paged_attention_decode(out_dev, q_dev, k_dev, v_dev, q_heads, kv_heads, head, q_stride, kv_stride, o_stride, scale, batch,
                           kcache_dev, vcache_dev, block_num, block_size, tables_dev, table_stride, ctx_dev, slots_dev, max_context,
                           stream=None):
    check(lib.xfthip_paged_attention_decode(out_dev, q_dev, k_dev, v_dev, q_heads, kv_heads, head, q_stride, kv_stride, o_stride,
                                            C.c_float(scale), batch, kcache_dev, vcache_dev, block_num, block_size, tables_dev,
                                            table_stride, ctx_dev, slots_dev, max_context, stream))


def paged_attention_prefill(out_dev, q_dev, k_dev, v_dev, q_heads, kv_heads, head, q_stride, kv_stride, o_stride, scale, token_lens,
                            kcache_dev, vcache_dev, block_num, block_size, slots_dev, stream=None):
    lens = np.ascontiguousarray(token_lens, np.int32)
    check(lib.xfthip_paged_attention_prefill(out_dev, q_dev, k_dev, v_dev, q_heads, kv_heads, head, q_stride, kv_stride, o_stride,
                                             C.c_float(scale), len(lens), _hp(lens), kcache_dev, vcache_dev, block_num, block_size,
                                             slots_dev, stream))


def argmax(logits_dev, rows, cols, stream=None):
    """First-maximum argmax of fp32 logits [rows, cols] in device memory; returns host int32 [rows]."""
    ids = DeviceBuffer(rows * 4)
    check(lib.xfthip_argmax(logits_dev, rows, cols, ids.ptr, stream))
    synchronize()
    return ids.to_numpy(np.int32, (rows,))


# ---------------------------------------------------------------------------- W8A8
def w8a8_quantize_rows(A_dev, a_dtype, M, K, lda, stream=None):
    """Returns device buffers (qa [M, ldq], scale, zero, sum) and ldq."""
    ldq = (K + 15) // 16 * 16
    qa = DeviceBuffer(M * ldq)
    s, z, sm = DeviceBuffer(M * 4), DeviceBuffer(M * 4), DeviceBuffer(M * 4)
    check(lib.xfthip_w8a8_quantize_rows(A_dev, a_dtype, M, K, lda, qa.ptr, ldq, s.ptr, z.ptr, sm.ptr, stream))
    return qa, s, z, sm, ldq


def gemm_w8a8(w, M, qa, ldq, s, z, sm, C_dev, ldc, c_dtype=F32, epi=EPI_NONE, bias=None, res=None, ldres=0,
              res_dtype=F32, gamma=1.0, stream=None):
    check(lib.xfthip_gemm_w8a8(w.h, M, qa.ptr, ldq, s.ptr, z.ptr, sm.ptr, C_dev, ldc, c_dtype, epi, bias, res, ldres,
                               res_dtype, C.c_float(gamma), stream))


# ---------------------------------------------------------------------------- Mixtral MoE
class MoE:
    def __init__(self, hidden, inter, experts, max_tokens, router, ln=None, beside=None):
        """beside: another MoE of the same shape whose per-call buffers this one works in (layers of one model)."""
        self.hidden, self.inter, self.E = hidden, inter, experts
        router = np.ascontiguousarray(router, np.float32)
        ln = None if ln is None else np.ascontiguousarray(ln, np.float32)
        h = C.c_void_p()
        if beside is None:
            check(lib.xfthip_moe_create(hidden, inter, experts, max_tokens, _hp(router), _hp(ln), C.byref(h)))
        else:
            check(lib.xfthip_moe_create_beside(beside.h, _hp(router), _hp(ln), C.byref(h)))
        self.h = h
        self._keep = [beside]

    def set_expert(self, e, gateup, down):
        self._keep += [gateup, down]
        check(lib.xfthip_moe_set_expert(self.h, e, gateup.h, down.h))

    def forward(self, x_in_dev, x_out_dev, tokens, do_norm=True, logits_override_dev=None, stream=None, want_routing=True):
        """Returns the chosen experts and their weights (which costs a wait for the stream); with
        want_routing=False nothing is copied back, the call only enqueues work and may be captured into a graph."""
        if not want_routing:
            check(lib.xfthip_moe_forward(self.h, x_in_dev, self.hidden, x_out_dev, self.hidden, tokens, int(do_norm),
                                         logits_override_dev, None, None, stream))
            return None, None
        sel = np.empty((tokens, 2), np.int32)
        w = np.empty((tokens, 2), np.float32)
        check(lib.xfthip_moe_forward(self.h, x_in_dev, self.hidden, x_out_dev, self.hidden, tokens, int(do_norm),
                                     logits_override_dev, _hp(sel), _hp(w), stream))
        return sel, w

    def free(self):
        if self.h is not None:
            lib.xfthip_moe_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def moe_top2(logits_dev, M, E, stream=None):
    sel, w = DeviceBuffer(M * 8), DeviceBuffer(M * 8)
    check(lib.xfthip_moe_top2(logits_dev, M, E, sel.ptr, w.ptr, stream))
    synchronize()
    return sel.to_numpy(np.int32, (M, 2)), w.to_numpy(np.float32, (M, 2))
