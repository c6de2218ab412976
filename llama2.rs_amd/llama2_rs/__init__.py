"""llama2_rs — the reference's Python surface over the MI355X C ABI.

Same names as the pyO3 module that python/llama2_rs/__init__.py re-exports
(LlamaModel, Tokenizer, Random, Config, generate, START, RET), plus the
operator-level wrappers in `ops` and the checkpoint-format helpers in
`checkpoint`.  Importing the package does not load the library; the first use
of a class does, and fails loudly if it is missing.
"""
from .llama2_rs_pylib import LlamaModel, Tokenizer, Random, generate  # noqa: F401
from ._lib import Config  # noqa: F401

START = 1  # python/llama2_rs/__init__.py:4, src/tokenizer.rs:10
RET = 13   # python/llama2_rs/__init__.py:5, src/tokenizer.rs:11
