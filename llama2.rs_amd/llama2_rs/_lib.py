"""ctypes loader for libllama2_hip.so (the C ABI declared in include/llama2_hip.h).

The library is looked up next to the package (built in-tree by build.py).  If
it is missing, or it loads but no HIP device is usable, every compute call
fails loudly: there is no CPU fallback in this package.
"""
from __future__ import annotations

import ctypes as C
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# LLAMA2_HIP_LIB names another build of the same library (e.g. an instrumented one).
LIB_PATH = os.environ.get("LLAMA2_HIP_LIB") or os.path.join(os.path.dirname(_PKG), "libllama2_hip.so")

L2_OK = 0
ERR_NAMES = {-1: "L2_ERR_ARG", -2: "L2_ERR_IO", -3: "L2_ERR_FORMAT", -4: "L2_ERR_HIP", -5: "L2_ERR_RANGE"}

WQ, WK, WV, WO, W1, W2, W3 = range(7)
PREFILL_FP32, PREFILL_MFMA = 0, 1


class L2Error(RuntimeError):
    def __init__(self, code: int, text: str):
        super().__init__(f"{ERR_NAMES.get(code, code)}: {text}")
        self.code = code


class Dims(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads",
                                         "vocab_size", "seq_len", "group_size")]


class Config(C.Structure):
    """Config of src/constants.rs:80-89 as read from the checkpoint header."""
    _fields_ = [(n, C.c_int32) for n in ("dim", "hidden_dim", "n_layers", "n_heads", "n_kv_heads",
                                         "vocab_size", "seq_len", "shared_weight")]

    def __repr__(self):
        return "Config { " + ", ".join(f"{n}: {getattr(self, n)}" for n, _ in self._fields_) + " }"


# name: (restype, argtypes) — must list every symbol include/llama2_hip.h declares
_VP, _I, _SZ = C.c_void_p, C.c_int, C.c_size_t
SIGNATURES = {
    "l2_last_error": (C.c_char_p, []),
    "l2_device_count": (_I, []),
    "l2_preset": (_I, [C.c_char_p, _I, C.POINTER(Dims)]),
    "l2_weights_bytes": (_SZ, [C.POINTER(Dims)]),
    "l2_synth_image": (_I, [C.POINTER(Dims), C.c_uint64, _VP, _SZ]),
    "l2_model_open": (_I, [C.c_char_p, C.POINTER(Dims), _I, C.POINTER(_VP)]),
    "l2_model_from_image": (_I, [_VP, _SZ, C.POINTER(Dims), _I, C.POINTER(_VP)]),
    "l2_model_close": (None, [_VP]),
    "l2_model_config": (_I, [_VP, C.POINTER(Config)]),
    "l2_model_dims": (_I, [_VP, C.POINTER(Dims)]),
    "l2_model_max_seq": (_I, [_VP]),
    "l2_prefill_supported": (_I, [_VP]),
    "l2_model_set_prefill_mode": (_I, [_VP, _I]),
    "l2_model_set_step_graph": (_I, [_VP, _I]),
    "l2_state_new": (_I, [_VP, C.POINTER(_VP)]),
    "l2_state_free": (None, [_VP]),
    "l2_state_reset": (_I, [_VP]),
    "l2_state_read_kv": (_I, [_VP, _I, _I, _I, _VP, _VP]),
    "l2_state_write_kv": (_I, [_VP, _I, _I, _I, _VP, _VP]),
    "l2_state_fill_synthetic": (_I, [_VP, _I, _I, C.c_uint64]),
    "l2_qlinear_create": (_I, [_VP, _VP, _VP, _VP, _I, _I, _I, C.POINTER(_VP)]),
    "l2_qlinear_free": (None, [_VP]),
    "l2_qlinear_matvec": (_I, [_VP, _VP, _I, _VP]),
    "l2_qlinear_matvec_device": (_I, [_VP, _VP, _I, _VP, _VP]),
    "l2_model_q4_kernels": (_I, [_VP, C.c_char_p, _SZ]),
    "l2_model_qmatvec": (_I, [_VP, _I, _I, _VP, _I, _VP]),
    "l2_model_classifier": (_I, [_VP, _VP, _VP]),
    "l2_forward": (_I, [_VP, _VP, _VP, _VP, _I, _VP]),
    "l2_prefill_chunks": (_I, [_VP, _VP, _VP, _I, _I, _I]),
    "l2_decode_greedy": (_I, [_VP, _VP, C.c_int32, C.c_int32, C.POINTER(C.c_int32)]),
    "l2_generate_greedy": (_I, [_VP, _VP, _VP, _I, _I, _I, _VP, C.POINTER(_I), C.POINTER(C.c_double)]),
    "l2_tokenizer_open": (_I, [C.c_char_p, _I, C.POINTER(_VP)]),
    "l2_tokenizer_free": (None, [_VP]),
    "l2_tokenizer_vocab_size": (_I, [_VP]),
    "l2_tokenizer_token": (_I, [_VP, _I, C.POINTER(C.c_char_p), C.POINTER(_I), C.POINTER(C.c_float)]),
    "l2_tokenizer_encode": (_I, [_VP, C.c_char_p, _VP, _I, C.POINTER(_I)]),
    "l2_random_new": (_I, [C.c_uint64, _I, C.POINTER(_VP)]),
    "l2_random_free": (None, [_VP]),
    "l2_random_f32": (C.c_float, [_VP]),
    "l2_random_sample": (_I, [_VP, _VP, _I]),
    "l2_generate": (_I, [_VP, _VP, _VP, C.c_char_p, _I, _VP, C.c_float, _I, _VP, _SZ, C.POINTER(_I),
                         C.POINTER(C.c_int64)]),
    "l2_qlinear_bench": (_I, [C.POINTER(_VP), _I, _I, C.POINTER(C.c_float)]),
    "l2_qlinear_bench_dispatch": (_I, [C.POINTER(_VP), _I, _I, C.POINTER(C.c_float)]),
    "l2_qlinear_kernel": (_I, [_VP, C.c_char_p, _SZ]),
    "l2_decode_bench": (_I, [_VP, _VP, C.c_int32, C.c_int32, _I, _VP, C.POINTER(C.c_float)]),
    "l2_kernel_class_count": (_I, []),
    "l2_kernel_class_name": (C.c_char_p, [_I]),
    "l2_decode_profile": (_I, [_VP, _VP, C.c_int32, C.c_int32, _I, _VP, _VP]),
    "l2_q4_plan": (_I, [_I, _VP, _I, _I, _I, _I, C.c_char_p, _SZ, _VP]),
    "l2_copy_bench": (_I, [_SZ, _I, C.POINTER(C.c_float)]),
}

_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python llama2.rs_amd/build.py` "
                "(hipcc, --offload-arch=gfx950).  There is no CPU fallback.")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != L2_OK:
        raise L2Error(rc, lib().l2_last_error().decode("utf-8", "replace"))
