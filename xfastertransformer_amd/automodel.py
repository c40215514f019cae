"""Python face of xft::AutoModel: the generation API of the reference's
src/xfastertransformer/automodel.py (from_pretrained / config / input / forward / generate / is_done /
finalize with the same argument names and defaults), bound with ctypes to the C entry points of
libxft_layers.so instead of a Torch custom class.  Token ids go in and come out as torch tensors
when torch tensors are given, numpy arrays otherwise.  There is no CPU path: without the built
libraries the import of this package fails."""
import ctypes as C
import os

import numpy as np

from . import capi  # loads libxft_hip.so (RTLD_GLOBAL) or raises

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libxft_layers.so")
if not os.path.exists(_LIB_PATH):
    raise ImportError(f"{_LIB_PATH} is not built; run `python -m xfastertransformer_amd.build`")
_lib = C.CDLL(_LIB_PATH)
_lib.xft_automodel_create.restype = C.c_void_p
_lib.xft_automodel_create.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p]
_lib.xft_automodel_destroy.argtypes = [C.c_void_p]
_lib.xft_automodel_destroy.restype = None
_lib.xft_automodel_config.restype = None
_lib.xft_automodel_config.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, C.c_int, C.c_int,
                                      C.c_float, C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_int]
_lib.xft_automodel_input.restype = None
_lib.xft_automodel_input.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int]
_lib.xft_automodel_generate.argtypes = [C.c_void_p, C.c_void_p]
_lib.xft_automodel_is_done.argtypes = [C.c_void_p]
_lib.xft_automodel_finalize.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
_lib.xft_automodel_forward.argtypes = [C.c_void_p, C.c_void_p]
_lib.xft_automodel_vocab_size.argtypes = [C.c_void_p]
_lib.xft_automodel_max_seq_len.argtypes = [C.c_void_p]
_lib.xft_automodel_set_input.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                         C.c_float, C.c_void_p]
_lib.xft_automodel_free_seqs.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
_lib.xft_automodel_set_prefix.restype = None
_lib.xft_automodel_set_prefix.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
_lib.xft_sample_candidates.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_void_p]
_lib.xft_sample_pick.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_float]
_lib.xft_beam_create.restype = C.c_void_p
_lib.xft_beam_create.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, C.c_int, C.c_int]
_lib.xft_beam_step.restype = None
_lib.xft_beam_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
_lib.xft_beam_is_done.argtypes = [C.c_void_p]
_lib.xft_beam_finalize.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
_lib.xft_beam_destroy.restype = None
_lib.xft_beam_destroy.argtypes = [C.c_void_p]

# the types this build serves out of the reference's list (automodel.py:21-39)
_DTYPES = ["fp16", "bf16", "int8", "w8a8", "int4", "nf4", "bf16_fp16", "bf16_int8", "bf16_w8a8", "bf16_int4", "bf16_nf4", "w8a8_int8",
           "w8a8_int4", "w8a8_nf4"]
_REFERENCE_DTYPES = _DTYPES + ["fp8_e4m3"]
_KV_DTYPES = ["fp16", "int8"]


def _is_torch(x):
    return type(x).__module__.startswith("torch")


def _ids_array(input_ids):
    if _is_torch(input_ids):
        input_ids = input_ids.detach().cpu().numpy()
    a = np.ascontiguousarray(np.asarray(input_ids), dtype=np.int32)
    if a.ndim == 1:
        a = a[None, :]
    if a.ndim != 2 or a.size == 0:
        raise ValueError("input_ids must be [batch, seq_len]")
    return a


def sample_candidates(logits, top_k=50, top_p=1.0, temperature=1.0):
    """The candidate ids and probabilities the sampler draws from for one row of logits."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    k = max(2, min(int(top_k), logits.size))
    ids = np.zeros(k, np.int32)
    probs = np.zeros(k, np.float32)
    n = _lib.xft_sample_candidates(logits.ctypes.data, logits.size, int(top_k), float(top_p), float(temperature),
                                   ids.ctypes.data, probs.ctypes.data)
    return ids[:n], probs[:n]


def sample_pick(ids, probs, u):
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    probs = np.ascontiguousarray(probs, dtype=np.float32)
    return int(_lib.xft_sample_pick(ids.ctypes.data, probs.ctypes.data, len(ids), float(u)))


class BeamSearcher:
    """The beam searcher's host half on its own: feed it the logits of every beam row, read the token and the
    source row it chose for each (what Model.generate does between two device steps)."""

    def __init__(self, prompts, num_beams, max_length, eos_token_id, pad_token_id, vocab_size, num_return_sequences=1,
                 length_penalty=1.0, early_stopping=False):
        a = _ids_array(prompts)
        self.rows, self.vocab, self.keep, self.max_length = a.shape[0] * num_beams, vocab_size, num_return_sequences, max_length
        self.batch = a.shape[0]
        self._h = _lib.xft_beam_create(a.ctypes.data, a.shape[0], a.shape[1], int(num_beams), int(num_return_sequences), int(max_length),
                                       float(length_penalty), int(bool(early_stopping)), int(eos_token_id), int(pad_token_id),
                                       int(vocab_size))

    def step(self, logits):
        lg = np.array(logits, dtype=np.float32, order="C").reshape(self.rows, self.vocab)
        tokens, indices, scores = np.zeros(self.rows, np.int32), np.zeros(self.rows, np.int32), np.zeros(self.rows, np.float32)
        _lib.xft_beam_step(self._h, lg.ctypes.data, tokens.ctypes.data, indices.ctypes.data, scores.ctypes.data)
        return tokens.tolist(), indices.tolist(), scores

    def is_done(self):
        return bool(_lib.xft_beam_is_done(self._h))

    def finalize(self):
        cap = self.batch * self.keep * (self.max_length + 1)
        out = np.zeros(cap, np.int32)
        n = _lib.xft_beam_finalize(self._h, out.ctypes.data, cap)
        return out[:n].reshape(self.batch * self.keep, -1)

    def __del__(self):
        try:
            if self._h:
                _lib.xft_beam_destroy(self._h)
                self._h = None
        except Exception:
            pass


class AutoModel:
    def __init__(self, path, dtype: str = "fp16", kv_cache_dtype: str = "fp16"):
        if dtype not in _REFERENCE_DTYPES:
            raise Exception(f"{self.__class__.__name__} don't support {dtype}.")
        if dtype not in _DTYPES:
            raise Exception(f"{self.__class__.__name__} of this build don't support the type {dtype}.")
        if kv_cache_dtype not in _KV_DTYPES:
            raise Exception(f"{self.__class__.__name__} don't support KV cache data type: {kv_cache_dtype}.")
        if not os.path.exists(os.path.join(path, "config.ini")):
            raise FileNotFoundError(os.path.join(path, "config.ini"))
        self._h = _lib.xft_automodel_create(os.fsencode(path), dtype.encode(), kv_cache_dtype.encode())
        self._torch_out = False
        self._batch = 0
        self._beams, self._keep = 1, 1

    @classmethod
    def from_pretrained(cls, path, dtype: str = "fp16", kv_cache_dtype: str = "fp16"):
        return cls(path, dtype, kv_cache_dtype)

    @property
    def rank(self):
        return 0

    @property
    def vocab_size(self):
        return int(_lib.xft_automodel_vocab_size(self._h))

    @property
    def max_seq_len(self):
        return int(_lib.xft_automodel_max_seq_len(self._h))

    def config(self, max_length=20, num_beams=1, num_return_sequences=1, length_penalty=1.0, early_stopping=False,
               eos_token_id=-1, pad_token_id=-1, do_sample=False, temperature=1.0, top_k=50, top_p=1.0,
               repetition_penalty=1.0, stop_words_ids=None, **kwargs):
        self._beams, self._keep = int(num_beams), int(num_return_sequences)
        words = [list(w) for w in (stop_words_ids or [])]
        lens = np.asarray([len(w) for w in words], np.int32)
        flat = np.asarray([t for w in words for t in w], np.int32)
        _lib.xft_automodel_config(self._h, int(max_length), int(num_beams), int(num_return_sequences), float(length_penalty),
                                  int(bool(early_stopping)), int(eos_token_id), int(pad_token_id), int(bool(do_sample)),
                                  float(temperature), int(top_k), float(top_p), float(repetition_penalty),
                                  lens.ctypes.data if len(words) else None, flat.ctypes.data if len(words) else None, len(words))

    def input(self, input_ids=None):
        self._torch_out = _is_torch(input_ids)
        a = _ids_array(input_ids)
        self._batch = a.shape[0]
        _lib.xft_automodel_input(self._h, a.ctypes.data, a.shape[0], a.shape[1])

    def set_input_cb(self, input_ids=None, seq_ids=None, max_length=20, eos_token_id=-1, pad_token_id=-1, repetition_penalty=1.0):
        """Continuous batching (automodel.py:41-69 of the reference): prompts of any lengths become new
        sequences when seq_ids is None, else seq_ids names the live sequences the next forward_cb() steps.
        Returns the sequence ids."""
        if seq_ids is None:
            prompts = [list(map(int, (p.tolist() if hasattr(p, "tolist") else p))) for p in input_ids]
            given = np.zeros(0, np.int32)
        else:
            given = np.ascontiguousarray(seq_ids.tolist() if hasattr(seq_ids, "tolist") else seq_ids, np.int32)
            prompts = [[0]] * len(given)
        lens = np.asarray([len(p) for p in prompts], np.int32)
        flat = np.asarray([t for p in prompts for t in p], np.int32)
        out = np.zeros(len(prompts), np.int32)
        n = _lib.xft_automodel_set_input(self._h, lens.ctypes.data, flat.ctypes.data, len(prompts), given.ctypes.data if len(given) else None,
                                         len(given), int(max_length), int(eos_token_id), int(pad_token_id), float(repetition_penalty),
                                         out.ctypes.data)
        self._batch = n
        self._beams = 1
        self._torch_out = False
        return out[:n].tolist()

    def forward_cb(self):
        """One step of the sequences chosen by set_input_cb: their next tokens, in that order."""
        return self.forward().ravel().tolist()

    def prefix_sharing(self, input_ids=None, truncate_tail=0):
        """The reference's AutoModel.prefix_sharing (automodel.py:180-184): input_ids [1, n] is run once; inputs that
        follow carry it in front and only run what comes after it."""
        ids = np.asarray(input_ids.tolist() if hasattr(input_ids, "tolist") else input_ids, np.int32)
        if truncate_tail > 0:
            ids = ids[..., :-truncate_tail]
        ids = np.ascontiguousarray(ids.reshape(-1), np.int32)
        _lib.xft_automodel_set_prefix(self._h, ids.ctypes.data, len(ids))

    def disable_prefix_sharing(self):
        _lib.xft_automodel_set_prefix(self._h, None, 0)

    def free_seqs(self, seq_ids):
        ids = np.ascontiguousarray(seq_ids.tolist() if hasattr(seq_ids, "tolist") else seq_ids, np.int32)
        return bool(_lib.xft_automodel_free_seqs(self._h, ids.ctypes.data, len(ids)))

    def _wrap(self, a):
        if self._torch_out:
            import torch
            return torch.from_numpy(a.astype(np.int64))
        return a

    def forward(self):
        """One generation step: the next token of every sequence (of every beam row under beam search), [rows, 1]."""
        out = np.zeros(self._batch * self._beams, np.int32)
        n = _lib.xft_automodel_generate(self._h, out.ctypes.data)
        return self._wrap(out[:n, None])

    def logits(self):
        """fp32 [batch, vocab] logits of the prompt's next token (Model::forward(false))."""
        out = np.zeros((self._batch, self.vocab_size), np.float32)
        _lib.xft_automodel_forward(self._h, out.ctypes.data)
        return out

    def is_done(self):
        return bool(_lib.xft_automodel_is_done(self._h))

    def finalize(self):
        n = _lib.xft_automodel_finalize(self._h, None, 0)
        out = np.zeros(n, np.int32)
        _lib.xft_automodel_finalize(self._h, out.ctypes.data, n)
        rows = self._batch * (self._keep if self._beams > 1 else 1)
        if rows <= 0 or n % rows != 0:
            return self._wrap(out)  # sequences of different lengths, back to back
        return self._wrap(out.reshape(rows, -1))

    def generate(self, input_ids=None, max_length=20, num_beams=1, num_return_sequences=1, length_penalty=1.0,
                 early_stopping=False, eos_token_id=-1, pad_token_id=-1, do_sample=False, temperature=1.0, top_k=50,
                 top_p=1.0, repetition_penalty=1.0, stop_words_ids=None, streamer=None, **kwargs):
        if streamer is not None:
            if input_ids is not None and _ids_array(input_ids).shape[0] != 1:
                raise ValueError("`streamer` cannot be used with batch size != 1 (yet!).")
            if input_ids is not None:
                streamer.put(input_ids.cpu() if _is_torch(input_ids) else input_ids)
        self.config(max_length, num_beams, num_return_sequences, length_penalty, early_stopping, eos_token_id, pad_token_id,
                    do_sample, temperature, top_k, top_p, repetition_penalty, stop_words_ids)
        self.input(input_ids)
        while not self.is_done():
            next_tokens = self.forward()
            if streamer is not None and input_ids is not None:
                streamer.put(next_tokens.cpu() if _is_torch(next_tokens) else next_tokens)
        if streamer is not None:
            streamer.end()
        return self.finalize()

    def free(self):
        if getattr(self, "_h", None):
            _lib.xft_automodel_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass
