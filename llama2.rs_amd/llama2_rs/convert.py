"""AutoGPTQ Llama-2 checkpoint (a local directory of safetensors) -> llama2.rs `.bin`.

The reference's exporter (export.py:25-122) loads the model through `auto_gptq` from a Hub name; this
restates what it writes from the tensors themselves, so that a GPTQ checkpoint already on disk can be
converted with numpy + safetensors only.  Nothing is fetched.

    python -m llama2_rs.convert <model_dir> <out.bin> [--max-vocab-size 32000] [--max-seq-len 2048]

Layout written (export.py:76-119, src/gptq.rs:36-66): 7 x i32 header, f32 rms_eps, token embedding,
[L] attention norms, [L] q, k, v, o projections, [L] ffn norms, [L] gate (w1), down (w2), up (w3)
projections, final norm, the two deprecated RoPE tables, classifier.  Each projection is
`qweight i32[OUT][IN/8]` (input rows re-sorted by the stable argsort of g_idx and re-packed),
`qzeros i32[OUT/8][GROUPS]`, `scales f32[OUT][GROUPS]`, `g_index i32[IN]` (that argsort): the transform
of export.py:50-67, `checkpoint.export_transform`.
"""
from __future__ import annotations

import argparse
import glob
import json
import os
import sys
from typing import Dict

import numpy as np

from . import checkpoint as ck


class _Tensors:
    """Name -> numpy array over every *.safetensors file of a directory, opened lazily."""

    def __init__(self, model_dir: str):
        from safetensors import safe_open  # no pickle: the loader reads raw tensors only
        self._open = safe_open
        self._where: Dict[str, str] = {}
        files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"{model_dir}: no *.safetensors file")
        for f in files:
            with safe_open(f, framework="np") as h:
                for k in h.keys():
                    self._where[k] = f

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def get(self, name: str) -> np.ndarray:
        if name not in self._where:
            raise KeyError(f"tensor {name!r} is not in the checkpoint")
        with self._open(self._where[name], framework="np") as h:
            return h.get_tensor(name)


def _read_json(path: str) -> dict:
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def convert(model_dir: str, out_path: str, max_vocab_size: int = 32000, max_seq_len: int = 2048,
            log=print) -> ck.Dims:
    """Write `out_path`; returns the dims of what was written (group size from quantize_config.json)."""
    cfg = _read_json(os.path.join(model_dir, "config.json"))
    qcfg_path = os.path.join(model_dir, "quantize_config.json")
    qcfg = _read_json(qcfg_path) if os.path.exists(qcfg_path) else cfg.get("quantization_config", {})
    if int(qcfg.get("bits", 4)) != 4:
        raise ValueError(f"{model_dir}: {qcfg.get('bits')}-bit weights; the .bin format holds 4-bit only")
    group = int(qcfg.get("group_size", 128))
    if group not in (32, 64, 128):
        raise ValueError(f"group_size {group}: the reference builds for 32, 64 or 128 (src/constants.rs:44-56)")
    T = _Tensors(model_dir)
    n_layers = int(cfg["num_hidden_layers"])
    n_heads = int(cfg["num_attention_heads"])
    n_kv = int(cfg.get("num_key_value_heads") or n_heads)
    dim = int(cfg["hidden_size"])
    hidden = int(cfg["intermediate_size"])
    vocab = min(int(cfg["vocab_size"]), max_vocab_size)          # export.py:79-81
    d = ck.Dims(dim=dim, hidden_dim=hidden, n_layers=n_layers, n_heads=n_heads, n_kv_heads=n_kv,
                vocab_size=vocab, seq_len=max_seq_len, group_size=group)
    eps = float(cfg.get("rms_norm_eps", 1e-5))

    written = 0
    with open(out_path, "wb") as f:
        def put(a: np.ndarray, dtype) -> None:
            nonlocal written
            b = np.ascontiguousarray(a, dtype=dtype)
            f.write(memoryview(b).cast("B"))
            written += b.nbytes

        def dense(name: str, rows: int | None = None) -> None:
            w = T.get(name)
            put(w[:rows] if rows is not None else w, np.float32)

        def qlinear(prefix: str, n_in: int, n_out: int) -> None:
            qweight, qzeros = T.get(prefix + ".qweight"), T.get(prefix + ".qzeros")
            scales, g_idx = T.get(prefix + ".scales"), T.get(prefix + ".g_idx")
            groups = ck.groups_of(n_in, group)
            want = {"qweight": (n_in // 8, n_out), "qzeros": (groups, n_out // 8), "scales": (groups, n_out),
                    "g_idx": (n_in,)}
            for nm, a in (("qweight", qweight), ("qzeros", qzeros), ("scales", scales), ("g_idx", g_idx)):
                if tuple(a.shape) != want[nm]:
                    raise ValueError(f"{prefix}.{nm}: shape {tuple(a.shape)}, expected {want[nm]}")
            qw, qz, sc, gi = ck.export_transform(qweight.astype(np.int32, copy=False), qzeros, scales, g_idx)
            put(qw, np.int32), put(qz, np.int32), put(sc, np.float32), put(gi, np.int32)

        f.write(ck.header_bytes(d))
        put(np.array([eps]), np.float32)                                              # export.py:94
        dense("model.embed_tokens.weight", vocab)
        L = "model.layers.{}."
        kv_dim = d.kv_dim
        for i in range(n_layers): dense(L.format(i) + "input_layernorm.weight")
        for name, n_out in (("q_proj", dim), ("k_proj", kv_dim), ("v_proj", kv_dim), ("o_proj", dim)):
            for i in range(n_layers):
                qlinear(L.format(i) + "self_attn." + name, dim, n_out)
            log(f"wrote {name} x {n_layers}")
        for i in range(n_layers): dense(L.format(i) + "post_attention_layernorm.weight")
        for name, n_in, n_out in (("gate_proj", dim, hidden), ("down_proj", hidden, dim), ("up_proj", dim, hidden)):
            for i in range(n_layers):
                qlinear(L.format(i) + "mlp." + name, n_in, n_out)
            log(f"wrote {name} x {n_layers}")
        dense("model.norm.weight")
        # the deprecated tables (export.py:14-21,113-115); unused at run time (src/models.rs:193-197)
        hs = d.head_size
        freqs = 1.0 / (10000.0 ** (np.arange(0, hs, 2)[: hs // 2].astype(np.float32) / hs))
        ang = np.outer(np.arange(max_seq_len, dtype=np.float32), freqs).astype(np.float32)
        put(np.cos(ang), np.float32), put(np.sin(ang), np.float32)
        dense("lm_head.weight", vocab)
    if written != ck.weights_bytes(d):
        raise RuntimeError(f"wrote {written} bytes after the header, the struct for these dims is {ck.weights_bytes(d)}")
    log(f"wrote {out_path}: {ck.HEADER_BYTES + written} bytes, dims {d}")
    return d


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("model_dir")
    ap.add_argument("output_path")
    ap.add_argument("--max-vocab-size", type=int, default=32000)
    ap.add_argument("--max-seq-len", type=int, default=2048)
    a = ap.parse_args(argv)
    convert(a.model_dir, a.output_path, a.max_vocab_size, a.max_seq_len)
    return 0


if __name__ == "__main__":
    sys.exit(main())
