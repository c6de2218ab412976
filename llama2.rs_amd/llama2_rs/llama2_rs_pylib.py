"""The names the reference's pyO3 module exports (src/lib.rs:111-131,
python/llama2_rs/llama2_rs_pylib.pyi), over the C ABI of libllama2_hip.so.

    model = llama2_rs.LlamaModel("llama2_7b.bin", False)
    tokenizer = llama2_rs.Tokenizer("tokenizer.bin")
    random = llama2_rs.Random()
    ms, tokens = llama2_rs.generate(model, tokenizer, "Hello", 50, random, 0.0)

The reference fixes the model size at compile time through cargo features; a
`.bin` file carries no group size, so here the preset is inferred from the
header and the file size, or given through LLAMA2_RS_FEATURES (e.g.
"70B,group_64,quantized").
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Tuple

from . import checkpoint as ck
from . import ops
from ._lib import Config, check, lib

VOCAB_SIZE = 32000  # src/constants.rs:13,26,37


def _preset_for(path: str) -> ck.Dims:
    feats = os.environ.get("LLAMA2_RS_FEATURES", "")
    names = [f.strip() for f in feats.split(",") if f.strip()]
    size = next((n for n in names if n in ck.PRESETS), None)
    group = next((int(n.split("_")[1]) for n in names if n.startswith("group_")), None)
    hdr = ck.read_header(path)
    nbytes = os.path.getsize(path)
    candidates = []
    for name, base in ck.PRESETS.items():
        if size and name != size:
            continue
        # with features named and no `quantized` among them the build is the dense one (build.rs:16-38)
        dense_only = bool(names) and "quantized" not in names and group is None
        for g in ([0] if dense_only else [group] if group else [128, 64, 32, 0]):
            d = ck.preset(name, g)
            if (d.dim, d.hidden_dim, d.n_layers, d.n_heads) == (hdr["dim"], hdr["hidden_dim"], hdr["n_layers"],
                                                                hdr["n_heads"]) and ck.checkpoint_bytes(d) == nbytes:
                candidates.append(d)
    if not candidates:
        raise ValueError(f"{path}: header {hdr} and size {nbytes} match no 7B/13B/70B preset (group_32/64/128 or without quantisation)"
                         + (f" allowed by LLAMA2_RS_FEATURES={feats}" if feats else ""))
    return candidates[0]


class LlamaModel:
    """LlamaModel(checkpoint, debug=False)  (src/lib.rs:113-119, from_file :45-63)."""

    def __init__(self, checkpoint: str, debug: bool = False, dims: ck.Dims | None = None, max_seq: int = 0):
        d = dims or _preset_for(checkpoint)
        self._m = ops.Model(checkpoint, d, max_seq=max_seq)
        self.dims = d
        if debug:
            print(f"Configuration: {self.config!r}")

    @property
    def config(self) -> Config:
        return self._m.config

    def prefill(self) -> bool:
        return self._m.prefill()

    def close(self):
        self._m.close()


class Tokenizer:
    """Tokenizer(filename)  (src/tokenizer.rs:111-123)."""

    def __init__(self, filename: str, vocab_size: int = VOCAB_SIZE):
        self.h = C.c_void_p()
        check(lib().l2_tokenizer_open(filename.encode(), vocab_size, C.byref(self.h)))
        self.vocab_size = vocab_size

    def bpe_encode(self, text: str) -> List[int]:
        n = C.c_int()
        raw = text.encode("utf-8")
        check(lib().l2_tokenizer_encode(self.h, raw, None, 0, C.byref(n)))
        ids = (C.c_int32 * max(n.value, 1))()
        check(lib().l2_tokenizer_encode(self.h, raw, ids, n.value, C.byref(n)))
        return list(ids[:n.value])

    def token(self, i: int) -> Tuple[str, float]:
        s, n, sc = C.c_char_p(), C.c_int(), C.c_float()
        check(lib().l2_tokenizer_token(self.h, i, C.byref(s), C.byref(n), C.byref(sc)))
        return C.string_at(s, n.value).decode("utf-8"), sc.value

    def __del__(self):
        try:
            if self.h:
                lib().l2_tokenizer_free(self.h)
                self.h = C.c_void_p()
        except Exception:
            pass


class Random:
    """Random()  (src/util.rs:87-92): seeded from the clock; Random(seed) pins it."""

    def __init__(self, seed: int | None = None):
        self.h = C.c_void_p()
        check(lib().l2_random_new(0 if seed is None else seed, 1 if seed is None else 0, C.byref(self.h)))

    def random(self) -> float:
        return lib().l2_random_f32(self.h)

    def __del__(self):
        try:
            if self.h:
                lib().l2_random_free(self.h)
                self.h = C.c_void_p()
        except Exception:
            pass


def generate(model: LlamaModel, tokenizer: Tokenizer, prompt: str, steps: int, random: Random,
             temperature: float = 0.0, print_tokens: bool = False) -> Tuple[int, List[str]]:
    """generate(...) -> (milliseconds, token strings)  (src/inference.rs:47-57)."""
    cap = max(steps, 1) * 64 + 64
    buf = C.create_string_buffer(cap)
    n, ms = C.c_int(), C.c_int64()
    check(lib().l2_generate(model._m.h, model._m.state, tokenizer.h, prompt.encode("utf-8"), steps, random.h,
                            temperature, 1 if print_tokens else 0, buf, cap, C.byref(n), C.byref(ms)))
    out, off = [], 0
    raw = buf.raw
    for _ in range(n.value):
        end = raw.index(b"\0", off)
        out.append(raw[off:end].decode("utf-8", "replace"))
        off = end + 1
    return ms.value, out
