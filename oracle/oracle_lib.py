"""ctypes view of liboracle.so — TEST INFRASTRUCTURE ONLY.

The oracle is the CPU restatement of the reference's token loop (oracle.c).
Only tests, the smoke check and the benchmark's cpu_baseline leg may import
this module; the product path never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile oracle.c with gcc (no GPU, no reference sources needed)."""
    src = os.path.join(_HERE, "oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class OrDims(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads",
                                         "vocab_size", "seq_len", "group_size", "max_seq")]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.or_weights_bytes.restype = C.c_size_t
        L.or_weights_bytes.argtypes = [C.POINTER(OrDims)]
        L.or_model_view.restype = C.c_void_p
        L.or_model_view.argtypes = [C.c_void_p, C.c_size_t, C.POINTER(OrDims)]
        L.or_model_free.argtypes = [C.c_void_p]
        L.or_state_new.restype = C.c_void_p
        L.or_state_new.argtypes = [C.c_void_p]
        L.or_state_free.argtypes = [C.c_void_p]
        L.or_state_key_cache.restype = C.POINTER(C.c_float)
        L.or_state_key_cache.argtypes = [C.c_void_p]
        L.or_state_value_cache.restype = C.POINTER(C.c_float)
        L.or_state_value_cache.argtypes = [C.c_void_p]
        L.or_transformer.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int,
                                     C.c_void_p]
        L.or_generate_greedy.restype = C.c_int
        L.or_generate_greedy.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                         C.c_int, C.c_void_p, C.c_void_p]
        L.or_qmatvec.argtypes = [C.c_void_p] * 4 + [C.c_int] * 4 + [C.c_void_p] * 2
        L.or_dense_matvec.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.or_rmsnorm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_int]
        L.or_softmax.argtypes = [C.c_void_p, C.c_int]
        L.or_silu_gate.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.or_rope.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 4
        L.or_rope_table_row.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.or_attention.argtypes = [C.c_void_p] * 5 + [C.c_int] * 4
        L.or_argmax.restype = C.c_int
        L.or_argmax.argtypes = [C.c_void_p, C.c_int]
        L.or_accum.argtypes = [C.c_void_p, C.c_void_p, C.c_int]
        L.or_str_lookup.restype = C.c_int
        L.or_str_lookup.argtypes = [C.c_char_p, C.c_int, C.c_void_p, C.c_void_p, C.c_int]
        L.or_bpe_encode.restype = C.c_int
        L.or_bpe_encode.argtypes = [C.c_char_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        L.or_num_threads.restype = C.c_int
        L.or_set_num_threads.argtypes = [C.c_int]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def num_threads() -> int:
    return lib().or_num_threads()


def set_num_threads(n: int) -> None:
    lib().or_set_num_threads(n)


def qmatvec(qweight, qzeros, scales, g_index, group_size: int, x) -> np.ndarray:
    """QLinear::matvec<B> (src/gptq.rs:94-176) on `.bin`-layout arrays; x is [IN] or [B][IN]."""
    qweight, qzeros, scales, g_index = _i32(qweight), _i32(qzeros), _f32(scales), _i32(g_index)
    x = _f32(x)
    one = x.ndim == 1
    xb = x.reshape(1, -1) if one else x
    n_out, n_in = qweight.shape[0], qweight.shape[1] * 8
    assert xb.shape[1] == n_in and g_index.shape[0] == n_in
    y = np.empty((xb.shape[0], n_out), np.float32)
    lib().or_qmatvec(_p(qweight), _p(qzeros), _p(scales), _p(g_index), n_in, n_out, group_size,
                     xb.shape[0], _p(xb), _p(y))
    return y[0] if one else y


def dense_matvec(w, x) -> np.ndarray:
    w, x = _f32(w), _f32(x)
    one = x.ndim == 1
    xb = x.reshape(1, -1) if one else x
    y = np.empty((xb.shape[0], w.shape[0]), np.float32)
    lib().or_dense_matvec(_p(w), w.shape[1], w.shape[0], xb.shape[0], _p(xb), _p(y))
    return y[0] if one else y


def rmsnorm(x, weight, eps: float) -> np.ndarray:
    x, weight = _f32(x), _f32(weight)
    o = np.empty_like(x)
    lib().or_rmsnorm(_p(o), _p(x), _p(weight), eps, x.shape[0])
    return o


def softmax(x) -> np.ndarray:
    x = _f32(x).copy()
    lib().or_softmax(_p(x), x.shape[0])
    return x


def silu_gate(s, s2) -> np.ndarray:
    s, s2 = _f32(s).copy(), _f32(s2)
    lib().or_silu_gate(_p(s), _p(s2), s.shape[0])
    return s


def rope(q, k, pos: int, n_heads: int, n_kv_heads: int, head_size: int):
    q, k = _f32(q).copy(), _f32(k).copy()
    lib().or_rope(_p(q), _p(k), pos, n_heads, n_kv_heads, head_size)
    return q, k


def rope_table_row(pos: int, head_size: int):
    c = np.empty(head_size // 2, np.float32)
    s = np.empty(head_size // 2, np.float32)
    lib().or_rope_table_row(pos, head_size, _p(c), _p(s))
    return c, s


def attention(queries, value_cache, key_cache, pos, n_heads: int, n_kv_heads: int,
              head_size: int) -> np.ndarray:
    """queries [B][DIM]; caches [T][KVH][HS] of one layer; pos [B]."""
    q, vc, kc, pos = _f32(queries), _f32(value_cache), _f32(key_cache), _i32(pos)
    out = np.empty_like(q)
    lib().or_attention(_p(out), _p(q), _p(vc), _p(kc), _p(pos), q.shape[0], n_heads, n_kv_heads,
                       head_size)
    return out


def argmax(v) -> int:
    v = _f32(v)
    return lib().or_argmax(_p(v), v.shape[0])


def read_tokenizer_file(path: str, vocab_size: int):
    """Tokenizer::load (src/tokenizer.rs:22-37): i32 max_token_length, then vocab_size x {f32 score, i32 len,
    bytes}.  Returns (list of bytes, float32 scores, max_token_length)."""
    import struct
    data = open(path, "rb").read()
    (max_len,) = struct.unpack_from("<i", data, 0)
    off, vocab, scores = 4, [], np.empty(vocab_size, np.float32)
    for i in range(vocab_size):
        sc, ln = struct.unpack_from("<fi", data, off)
        off += 8
        vocab.append(data[off:off + ln])
        off += ln
        scores[i] = sc
    return vocab, scores, max_len


class Tokenizer:
    """Tokenizer (src/tokenizer.rs:13-108) over a vocabulary given as a list of byte strings and scores."""

    def __init__(self, vocab, scores):
        self.vocab = [bytes(v) for v in vocab]
        self.scores = _f32(scores)
        assert len(self.vocab) == self.scores.shape[0]
        self._bytes = np.frombuffer(b"".join(self.vocab) + b"\0", np.uint8).copy()
        self._off = np.zeros(len(self.vocab) + 1, np.int32)
        np.cumsum([len(v) for v in self.vocab], out=self._off[1:])

    @classmethod
    def from_file(cls, path: str, vocab_size: int = 32000):
        vocab, scores, _ = read_tokenizer_file(path, vocab_size)
        return cls(vocab, scores)

    def str_lookup(self, s) -> int:
        """util::str_lookup (src/util.rs:29-37); -1 for None."""
        b = s.encode("utf-8") if isinstance(s, str) else bytes(s)
        return lib().or_str_lookup(b, len(b), _p(self._bytes), _p(self._off), len(self.vocab))

    def bpe_encode(self, text) -> list:
        """Tokenizer::bpe_encode (src/tokenizer.rs:46-108)."""
        b = text.encode("utf-8") if isinstance(text, str) else bytes(text)
        out = np.empty(max(len(b), 1), np.int32)
        n = lib().or_bpe_encode(b, len(b), _p(self._bytes), _p(self._off), _p(self.scores), len(self.vocab),
                                _p(out), out.shape[0])
        if n == -1:
            raise ValueError("a character of the text is not in the vocabulary")
        if n < 0:
            raise ValueError("empty text")
        return out[:n].tolist()


class Model:
    """A weights image viewed through the oracle (TWeights + RunState)."""

    def __init__(self, weights_image: np.ndarray, dims, max_seq: int | None = None):
        self.image = weights_image  # keep alive: the model only points into it
        self.dims = dims
        self.max_seq = int(max_seq or dims.seq_len)
        self.od = OrDims(dims.dim, dims.hidden_dim, dims.n_layers, dims.n_heads, dims.n_kv_heads,
                         dims.vocab_size, dims.seq_len, dims.group_size, self.max_seq)
        addr = weights_image.ctypes.data if isinstance(weights_image, np.ndarray) else weights_image[0]
        nbytes = weights_image.nbytes if isinstance(weights_image, np.ndarray) else weights_image[1]
        self.h = lib().or_model_view(C.c_void_p(addr), nbytes, C.byref(self.od))
        if not self.h:
            raise ValueError("weights image size %d != struct size %d" %
                             (nbytes, lib().or_weights_bytes(C.byref(self.od))))
        self.state = None

    def new_state(self):
        if self.state:
            lib().or_state_free(self.state)
        self.state = lib().or_state_new(self.h)
        if not self.state:
            raise MemoryError("oracle KV cache")
        return self.state

    def kv_cache(self):
        d = self.dims
        shape = (d.n_layers, self.max_seq, d.n_kv_heads, d.head_size)
        n = int(np.prod(shape))
        k = np.ctypeslib.as_array(lib().or_state_key_cache(self.state), shape=(n,)).reshape(shape)
        v = np.ctypeslib.as_array(lib().or_state_value_cache(self.state), shape=(n,)).reshape(shape)
        return k, v

    def transformer(self, tokens, pos) -> np.ndarray | None:
        """transformer<B> (src/models.rs:178-298); logits only for B == 1."""
        if self.state is None:
            self.new_state()
        tokens, pos = _i32(tokens), _i32(pos)
        B = tokens.shape[0]
        logits = np.empty(self.dims.vocab_size, np.float32) if B == 1 else None
        lib().or_transformer(self.h, self.state, _p(tokens), _p(pos), B,
                             _p(logits) if B == 1 else None)
        return logits

    def generate_greedy(self, prompt_ids, steps: int, use_prefill: bool = True,
                        return_logits: bool = False):
        """generate() at temperature 0 on ids (src/inference.rs:49-193), fresh state."""
        prompt = _i32(prompt_ids)
        out = np.empty(max(steps, 1), np.int32)
        logits = np.empty(self.dims.vocab_size, np.float32)
        self.new_state()
        n = lib().or_generate_greedy(self.h, self.state, _p(prompt), prompt.shape[0], steps,
                                     1 if use_prefill else 0, _p(out), _p(logits))
        return (out[:n].copy(), logits) if return_logits else out[:n].copy()

    def close(self):
        if self.state:
            lib().or_state_free(self.state)
            self.state = None
        if self.h:
            lib().or_model_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
