"""The llama2.rs `.bin` checkpoint format: sizes, writer, and the act-order transform.

Host-side only (numpy).  Restates, without auto_gptq or torch, what the
reference's exporter does to each AutoGPTQ tensor before it is written
(export.py:50-67) and the order the tensors are written in (export.py:82-119),
which is the field order of the memory-mapped struct (src/gptq.rs:34-84).

Layout after the 28-byte header (little endian, no padding):
  f32 rms_eps | f32[V][DIM] tok_emb | f32[L][DIM] rms_att |
  QLinear[L] wq | wk | wv | wo | f32[L][DIM] rms_ffn |
  QLinear[L] w1 (gate) | w2 (down) | w3 (up) | f32[DIM] rms_final |
  f32[seq_len][HS/2] freq_cos | freq_sin | f32[V][DIM] wcls
and one QLinear is
  i32[OUT][IN/8] qweight | i32[OUT/8][GROUPS] qzeros | f32[OUT][GROUPS] scales | i32[IN] g_index
"""
from __future__ import annotations

import dataclasses
import struct
from typing import Dict, Tuple

import numpy as np

BITS = 4  # src/constants.rs:5
HEADER_BYTES = 28

_SHIFTS = np.arange(8, dtype=np.uint32) * 4


@dataclasses.dataclass(frozen=True)
class Dims:
    """Run-time counterpart of the compile-time constants (src/constants.rs:7-74)."""

    dim: int
    hidden_dim: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    vocab_size: int = 32000
    seq_len: int = 2048
    group_size: int = 128

    @property
    def head_size(self) -> int:
        return self.dim // self.n_heads

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_size

    @property
    def attn_groups(self) -> int:
        return self.n_heads // self.n_kv_heads


# Cargo features 7B / 13B / 70B (src/constants.rs:7-41); the group size comes
# from group_32 / group_64 / group_128 (:43-61).
PRESETS: Dict[str, Dims] = {
    "7B": Dims(4096, 11008, 32, 32, 32),
    "13B": Dims(5120, 13824, 40, 40, 40),
    "70B": Dims(8192, 28672, 80, 64, 8),
}


def preset(model_size: str, group_size: int) -> Dims:
    return dataclasses.replace(PRESETS[model_size], group_size=group_size)


def groups_of(n_in: int, group_size: int) -> int:
    return -(-n_in // group_size)  # int_div_up, src/gptq.rs:19-21


def qlinear_bytes(n_in: int, n_out: int, group_size: int) -> int:
    if group_size == 0:  # the build without quantisation: a dense Linear<IN,OUT> (src/model.rs:11-15)
        return n_out * n_in * 4
    g = groups_of(n_in, group_size)
    return n_out * (n_in // 8) * 4 + (n_out // 8) * g * 4 + n_out * g * 4 + n_in * 4


def weights_bytes(d: Dims) -> int:
    """size_of::<QTransformerWeights>() — what src/lib.rs:97 asserts the mmap length equals.
    group_size 0 (GROUPSIZE of the build without quantisation, src/constants.rs:58-61) gives
    size_of::<TransformerWeights>() (src/model.rs:36-67): the same fields, every projection dense."""
    L, G = d.n_layers, d.group_size
    n = 4 + d.vocab_size * d.dim * 4 + L * d.dim * 4
    n += L * (2 * qlinear_bytes(d.dim, d.dim, G) + 2 * qlinear_bytes(d.dim, d.kv_dim, G))
    n += L * d.dim * 4
    n += L * (2 * qlinear_bytes(d.dim, d.hidden_dim, G) + qlinear_bytes(d.hidden_dim, d.dim, G))
    n += d.dim * 4 + 2 * d.seq_len * (d.head_size // 2) * 4 + d.vocab_size * d.dim * 4
    return n


def checkpoint_bytes(d: Dims) -> int:
    return HEADER_BYTES + weights_bytes(d)


def header_bytes(d: Dims) -> bytes:
    """export.py:83-87.  n_kv_heads is written equal to n_heads there (:82); the
    loader never checks it (src/constants.rs:94-100).  A negative vocab size
    says that classifier weights are present."""
    return struct.pack("<7i", d.dim, d.hidden_dim, d.n_layers, d.n_heads, d.n_heads,
                       -d.vocab_size, d.seq_len)


def pack_nibbles(vals: np.ndarray, axis: int = 0) -> np.ndarray:
    """Pack groups of 8 values (0..15) along `axis` into int32, low nibble first."""
    v = np.moveaxis(np.asarray(vals, dtype=np.uint32), axis, 0)
    assert v.shape[0] % 8 == 0
    v = v.reshape(v.shape[0] // 8, 8, *v.shape[1:])
    sh = _SHIFTS.reshape(1, 8, *([1] * (v.ndim - 2)))
    packed = np.bitwise_or.reduce(v << sh, axis=1).astype(np.uint32)
    return np.moveaxis(packed, 0, axis).view(np.int32)


def unpack_nibbles(packed: np.ndarray, axis: int = 0) -> np.ndarray:
    """Inverse of pack_nibbles: int32 words -> 8 values each along `axis`."""
    p = np.moveaxis(np.ascontiguousarray(packed).view(np.uint32), axis, 0)
    sh = _SHIFTS.reshape(1, 8, *([1] * (p.ndim - 1)))
    v = (p[:, None] >> sh) & 15
    v = v.reshape(p.shape[0] * 8, *p.shape[1:])
    return np.moveaxis(v, 0, axis).astype(np.int32)


def export_transform(qweight: np.ndarray, qzeros: np.ndarray, scales: np.ndarray,
                     g_idx: np.ndarray) -> Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]:
    """AutoGPTQ tensors -> the four arrays of one `.bin` QLinear (export.py:50-67).

    In:  qweight i32[IN/8][OUT], qzeros i32[GROUPS][OUT/8], scales f32[GROUPS][OUT],
         g_idx i32[IN] (group of each input row).
    Out: qweight i32[OUT][IN/8] with input rows re-sorted by stable argsort of
         g_idx and re-packed, qzeros i32[OUT/8][GROUPS], scales f32[OUT][GROUPS],
         g_index i32[IN] = that argsort (not g_idx itself).
    """
    order = np.argsort(np.asarray(g_idx), kind="stable")
    rows = unpack_nibbles(qweight, axis=0)[order]          # [IN][OUT], sorted by group
    qw = pack_nibbles(rows, axis=0)                        # [IN/8][OUT]
    return (np.ascontiguousarray(qw.T), np.ascontiguousarray(np.asarray(qzeros, np.int32).T),
            np.ascontiguousarray(np.asarray(scales, np.float32).T), order.astype(np.int32))


def synth_autogptq_linear(rng: np.random.Generator, n_in: int, n_out: int, group_size: int,
                          act_order: bool = True):
    """Random AutoGPTQ-layout tensors: uniform nibbles, scales U[0.002, 0.02],
    g_idx a random permutation of i // group_size."""
    g = groups_of(n_in, group_size)
    qweight = pack_nibbles(rng.integers(0, 16, size=(n_in, n_out), dtype=np.int32), axis=0)
    qzeros = pack_nibbles(rng.integers(0, 16, size=(g, n_out), dtype=np.int32), axis=1)
    scales = rng.uniform(0.002, 0.02, size=(g, n_out)).astype(np.float32)
    g_idx = (np.arange(n_in) // group_size).astype(np.int32)
    if act_order:
        g_idx = rng.permutation(g_idx).astype(np.int32)
    return qweight, qzeros, scales, g_idx


def synth_qlinear(rng: np.random.Generator, n_in: int, n_out: int, group_size: int,
                  act_order: bool = True):
    """Random `.bin`-layout QLinear arrays (through export_transform)."""
    return export_transform(*synth_autogptq_linear(rng, n_in, n_out, group_size, act_order))


def dequant_autogptq(qweight, qzeros, scales, g_idx) -> np.ndarray:
    """fp64 dense W[IN][OUT] from AutoGPTQ tensors: s[g_idx[i]][o] * (q[i][o] - (z[g_idx[i]][o] + 1))."""
    q = unpack_nibbles(qweight, axis=0).astype(np.float64)
    z = unpack_nibbles(qzeros, axis=1).astype(np.float64) + 1.0
    s = np.asarray(scales, np.float64)
    return s[g_idx] * (q - z[g_idx])


def dequant_bin(qweight, qzeros, scales, g_index, group_size: int) -> np.ndarray:
    """fp64 dense W[OUT][IN] in ORIGINAL input order from `.bin`-layout arrays:
    y = W @ x reproduces src/gptq.rs:94-176 in exact arithmetic."""
    n_out, ing = qweight.shape
    n_in = ing * 8
    q = unpack_nibbles(qweight, axis=1).astype(np.float64)                 # [OUT][IN] sorted order
    z = unpack_nibbles(qzeros, axis=0).astype(np.float64) + 1.0            # [OUT][GROUPS]
    grp = np.arange(n_in) // group_size
    w_sorted = np.asarray(scales, np.float64)[:, grp] * (q - z[:, grp])    # column j multiplies x[g_index[j]]
    w = np.zeros_like(w_sorted)
    w[:, np.asarray(g_index)] = w_sorted
    return w


def synth_weights_image(d: Dims, seed: int = 0, act_order: bool = True,
                        rms_eps: float = 1e-5) -> np.ndarray:
    """A whole random-init weights image (bytes after the header) as uint8.

    Linear layers as synth_qlinear with one generator stream; norm weights,
    embedding and classifier ~ N(0, 0.02).  Meant for small dims: big models
    are generated natively by the library (l2_synth_image)."""
    rng = np.random.default_rng(seed)
    parts = []

    def f32(a):
        parts.append(np.ascontiguousarray(a, dtype=np.float32).view(np.uint8).reshape(-1))

    def i32(a):
        parts.append(np.ascontiguousarray(a, dtype=np.int32).view(np.uint8).reshape(-1))

    def qlin_block(n_in, n_out):
        for _ in range(d.n_layers):
            if d.group_size == 0:  # dense Linear, about the scale a trained projection has
                f32(rng.normal(0.0, 1.0 / np.sqrt(n_in), size=(n_out, n_in)))
                continue
            qw, qz, sc, gi = synth_qlinear(rng, n_in, n_out, d.group_size, act_order)
            i32(qw), i32(qz), f32(sc), i32(gi)

    def normal(*shape):
        return rng.normal(0.0, 0.02, size=shape).astype(np.float32)

    f32(np.array([rms_eps]))
    f32(normal(d.vocab_size, d.dim))
    f32(normal(d.n_layers, d.dim))
    qlin_block(d.dim, d.dim)
    qlin_block(d.dim, d.kv_dim)
    qlin_block(d.dim, d.kv_dim)
    qlin_block(d.dim, d.dim)
    f32(normal(d.n_layers, d.dim))
    qlin_block(d.dim, d.hidden_dim)
    qlin_block(d.hidden_dim, d.dim)
    qlin_block(d.dim, d.hidden_dim)
    f32(normal(d.dim))
    # deprecated tables, written as export.py:113-115 does (unused at run time)
    hs = d.head_size
    freqs = 1.0 / (10000.0 ** (np.arange(0, hs, 2)[: hs // 2].astype(np.float32) / hs))
    ang = np.outer(np.arange(d.seq_len, dtype=np.float32), freqs).astype(np.float32)
    f32(np.cos(ang)), f32(np.sin(ang))
    f32(normal(d.vocab_size, d.dim))
    img = np.concatenate(parts)
    assert img.nbytes == weights_bytes(d), (img.nbytes, weights_bytes(d))
    return img


def write_checkpoint(path: str, d: Dims, weights_image: np.ndarray) -> None:
    with open(path, "wb") as f:
        f.write(header_bytes(d))
        f.write(memoryview(np.ascontiguousarray(weights_image)))


def read_header(path: str):
    """src/constants.rs:102-119: seven i32; sign of vocab carries 'classifier present'."""
    with open(path, "rb") as f:
        h = struct.unpack("<7i", f.read(HEADER_BYTES))
    return {"dim": h[0], "hidden_dim": h[1], "n_layers": h[2], "n_heads": h[3],
            "n_kv_heads": h[4], "vocab_size": abs(h[5]), "seq_len": h[6],
            "shared_weight": h[5] > 0}
