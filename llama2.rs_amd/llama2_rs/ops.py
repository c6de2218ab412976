"""Operator- and model-level wrappers over the C ABI (numpy in, numpy out).

These mirror the reference's operator interface for the token loop:
`QLinear.matvec` (src/gptq.rs:94, src/gptq_cuda.rs:120), `Linear::matvec` for
the classifier (src/model.rs:22), `transformer::<B>` (src/models.rs:178) and
`RunState` (src/models.rs:29-42).  All compute runs in libllama2_hip.so on the
GPU.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import Dims, check, lib
from . import checkpoint as ck


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def to_cdims(d) -> Dims:
    if isinstance(d, Dims):
        return d
    return Dims(d.dim, d.hidden_dim, d.n_layers, d.n_heads, d.n_kv_heads, d.vocab_size, d.seq_len,
                d.group_size)


def from_cdims(c: Dims) -> ck.Dims:
    return ck.Dims(c.dim, c.hidden_dim, c.n_layers, c.n_heads, c.n_kv_heads, c.vocab_size, c.seq_len,
                   c.group_size)


def preset(model_size: str, group_size: int) -> ck.Dims:
    c = Dims()
    check(lib().l2_preset(model_size.encode(), group_size, C.byref(c)))
    return from_cdims(c)


def weights_bytes(d) -> int:
    return lib().l2_weights_bytes(C.byref(to_cdims(d)))


def synth_image(d, seed: int = 0) -> np.ndarray:
    """Random-init weights image generated natively (fast enough for 7B/70B)."""
    c = to_cdims(d)
    n = lib().l2_weights_bytes(C.byref(c))
    buf = np.empty(n, np.uint8)
    check(lib().l2_synth_image(C.byref(c), seed, _p(buf), n))
    return buf


class QLinear:
    """One uploaded QLinear in `.bin` layout (src/gptq.rs:68-84)."""

    def __init__(self, qweight, qzeros, scales, g_index, group_size: int):
        qweight, qzeros, scales, g_index = _i32(qweight), _i32(qzeros), _f32(scales), _i32(g_index)
        self.n_out, self.n_in = qweight.shape[0], qweight.shape[1] * 8
        self.group_size = group_size
        groups = ck.groups_of(self.n_in, group_size)
        if qzeros.shape != (self.n_out // 8, groups) or scales.shape != (self.n_out, groups) \
                or g_index.shape != (self.n_in,):
            raise ValueError("QLinear arrays do not have the .bin-layout shapes")
        self.h = C.c_void_p()
        check(lib().l2_qlinear_create(_p(qweight), _p(qzeros), _p(scales), _p(g_index), self.n_in,
                                      self.n_out, group_size, C.byref(self.h)))

    def matvec(self, x) -> np.ndarray:
        """x [IN] or [B][IN] -> y [OUT] or [B][OUT]  (QLinear::matvec<B>)."""
        x = _f32(x)
        one = x.ndim == 1
        xb = x.reshape(1, -1) if one else x
        if xb.shape[1] != self.n_in:
            raise ValueError(f"x has {xb.shape[1]} columns, the layer takes {self.n_in}")
        y = np.empty((xb.shape[0], self.n_out), np.float32)
        check(lib().l2_qlinear_matvec(self.h, _p(xb), xb.shape[0], _p(y)))
        return y[0] if one else y

    def matvec_device(self, x_dev: int, B: int, y_dev: int, stream: int = 0) -> None:
        """The same operator on DEVICE pointers (addresses as integers), enqueued on `stream` (a hipStream_t
        as an integer, 0 = the default stream) without waiting and without allocating anything: for callers
        under graph capture or in a serving loop.  B * in is bounded by the library's fixed scratch."""
        check(lib().l2_qlinear_matvec_device(self.h, C.c_void_p(x_dev), B, C.c_void_p(y_dev),
                                             C.c_void_p(stream) if stream else None))

    def close(self):
        if self.h:
            lib().l2_qlinear_free(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def qlinear_bench(qs, iters: int) -> float:
    """Total milliseconds (HIP events) of `iters` B=1 matvecs cycling through qs."""
    arr = (C.c_void_p * len(qs))(*[q.h for q in qs])
    ms = C.c_float()
    check(lib().l2_qlinear_bench(arr, len(qs), iters, C.byref(ms)))
    return ms.value


def qlinear_bench_dispatch(qs, iters: int) -> float:
    """Sum in milliseconds of the `iters` dispatch durations (each launch's own start/stop events)."""
    arr = (C.c_void_p * len(qs))(*[q.h for q in qs])
    ms = C.c_float()
    check(lib().l2_qlinear_bench_dispatch(arr, len(qs), iters, C.byref(ms)))
    return ms.value


def qlinear_kernel(q) -> str:
    """Name (as a profiler prints it) of the kernel a B=1 matvec of q runs."""
    buf = C.create_string_buffer(256)
    check(lib().l2_qlinear_kernel(q.h, buf, 256))
    return buf.value.decode()


def copy_bench(nbytes: int, iters: int) -> float:
    ms = C.c_float()
    check(lib().l2_copy_bench(nbytes, iters, C.byref(ms)))
    return ms.value


class Model:
    """Uploaded weights + one RunState."""

    def __init__(self, source, dims, max_seq: int = 0):
        """source: path of a `.bin` checkpoint, or a uint8 weights image (bytes after the header)."""
        self.dims = dims if isinstance(dims, ck.Dims) else from_cdims(dims)
        c = to_cdims(self.dims)
        self.h = C.c_void_p()
        self.state = C.c_void_p()
        if isinstance(source, (str, bytes)):
            path = source.encode() if isinstance(source, str) else source
            check(lib().l2_model_open(path, C.byref(c), max_seq, C.byref(self.h)))
        else:
            img = np.ascontiguousarray(source).view(np.uint8).reshape(-1)
            check(lib().l2_model_from_image(_p(img), img.nbytes, C.byref(c), max_seq, C.byref(self.h)))
        self.max_seq = lib().l2_model_max_seq(self.h)
        check(lib().l2_state_new(self.h, C.byref(self.state)))

    @property
    def config(self) -> _lib.Config:
        c = _lib.Config()
        check(lib().l2_model_config(self.h, C.byref(c)))
        return c

    def prefill(self) -> bool:
        return bool(lib().l2_prefill_supported(self.h))

    def reset(self):
        check(lib().l2_state_reset(self.state))

    def set_prefill_mode(self, mode: int):
        """_lib.PREFILL_FP32 (default, identical to B=1) or _lib.PREFILL_MFMA (fp16 tiles, 2e-3)."""
        check(lib().l2_model_set_prefill_mode(self.h, mode))

    def set_step_graph(self, on: bool):
        """Replay decode steps as captured HIP graphs (off by default)."""
        check(lib().l2_model_set_step_graph(self.h, 1 if on else 0))

    def qmatvec(self, layer: int, proj: int, x) -> np.ndarray:
        x = _f32(x)
        one = x.ndim == 1
        xb = x.reshape(1, -1) if one else x
        d = self.dims
        n_out = {_lib.WQ: d.dim, _lib.WK: d.kv_dim, _lib.WV: d.kv_dim, _lib.WO: d.dim, _lib.W1: d.hidden_dim,
                 _lib.W2: d.dim, _lib.W3: d.hidden_dim}[proj]
        y = np.empty((xb.shape[0], n_out), np.float32)
        check(lib().l2_model_qmatvec(self.h, layer, proj, _p(xb), xb.shape[0], _p(y)))
        return y[0] if one else y

    def classifier(self, x) -> np.ndarray:
        x = _f32(x)
        y = np.empty(self.dims.vocab_size, np.float32)
        check(lib().l2_model_classifier(self.h, _p(x), _p(y)))
        return y

    def forward(self, tokens, pos, want_logits: bool = True):
        """transformer::<B>; returns logits [vocab] when B == 1, else None."""
        tokens, pos = _i32(tokens), _i32(pos)
        B = tokens.shape[0]
        logits = np.empty(self.dims.vocab_size, np.float32) if (B == 1 and want_logits) else None
        check(lib().l2_forward(self.h, self.state, _p(tokens), _p(pos), B,
                               _p(logits) if logits is not None else None))
        return logits

    def prefill_chunks(self, tokens, pos0: int, chunk: int) -> None:
        """prefill::<A> over a whole prompt: tokens[i] at position pos0 + i, in chunks of `chunk`."""
        tokens = _i32(tokens)
        check(lib().l2_prefill_chunks(self.h, self.state, _p(tokens), tokens.shape[0], pos0, chunk))

    def decode_greedy(self, token: int, pos: int) -> int:
        nxt = C.c_int32()
        check(lib().l2_decode_greedy(self.h, self.state, token, pos, C.byref(nxt)))
        return nxt.value

    def generate_greedy(self, prompt_ids, steps: int, use_prefill: bool = True):
        """generate() at temperature 0 on ids; returns (ids, milliseconds)."""
        prompt = _i32(prompt_ids)
        out = np.empty(max(steps, 1), np.int32)
        n = C.c_int()
        ms = C.c_double()
        check(lib().l2_generate_greedy(self.h, self.state, _p(prompt) if prompt.size else None,
                                       prompt.shape[0], steps, 1 if use_prefill else 0, _p(out),
                                       C.byref(n), C.byref(ms)))
        return out[:n.value].copy(), ms.value

    def decode_bench(self, token: int, pos: int, n_tokens: int):
        out = np.empty(n_tokens, np.int32)
        ms = C.c_float()
        check(lib().l2_decode_bench(self.h, self.state, token, pos, n_tokens, _p(out), C.byref(ms)))
        return out, ms.value

    def decode_profile(self, token: int, pos: int, n_tokens: int):
        """{class name: (ms summed over the run, launches)} from per-launch HIP events."""
        n = lib().l2_kernel_class_count()
        ms = np.zeros(n, np.float32)
        cnt = np.zeros(n, np.int32)
        check(lib().l2_decode_profile(self.h, self.state, token, pos, n_tokens, _p(ms), _p(cnt)))
        return {lib().l2_kernel_class_name(i).decode(): (float(ms[i]), int(cnt[i])) for i in range(n)}

    def q4_kernels(self) -> dict:
        """{launch class: kernel name as a profiler prints it} of this model's decode step."""
        buf = C.create_string_buffer(1024)
        check(lib().l2_model_q4_kernels(self.h, buf, 1024))
        return dict(item.split("=", 1) for item in buf.value.decode().split(";") if item)

    def read_kv(self, layer: int, pos0: int, npos: int):
        d = self.dims
        k = np.empty((npos, d.n_kv_heads, d.head_size), np.float32)
        v = np.empty_like(k)
        check(lib().l2_state_read_kv(self.state, layer, pos0, npos, _p(k), _p(v)))
        return k, v

    def write_kv(self, layer: int, pos0: int, k, v):
        d = self.dims
        k = np.ascontiguousarray(k, np.float32)
        v = np.ascontiguousarray(v, np.float32)
        if k.shape != v.shape or k.shape[1:] != (d.n_kv_heads, d.head_size):
            raise ValueError(f"k, v must be [npos][{d.n_kv_heads}][{d.head_size}]")
        check(lib().l2_state_write_kv(self.state, layer, pos0, k.shape[0], _p(k), _p(v)))

    def fill_kv_synthetic(self, pos0: int, npos: int, seed: int = 0):
        check(lib().l2_state_fill_synthetic(self.state, pos0, npos, seed))

    def close(self):
        if self.state:
            lib().l2_state_free(self.state)
            self.state = C.c_void_p()
        if self.h:
            lib().l2_model_close(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
