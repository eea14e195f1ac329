"""Torch operator library ``_C_gguf`` over ``libgguf_hip.so``: stands in for the reference's compiled extension module.

Importing this module defines the six operator schemas of the reference's
``vllm_gguf_plugin/csrc/torch_bindings.cpp:22-40`` and implements them for the dispatch key the reference uses
(``:42-53``: ``CUDA``, which HIP tensors dispatch on, and ``CompositeExplicitAutograd`` for the block-size query), so
``torch.ops._C_gguf.<op>`` call sites (``vllm_gguf_plugin/ops.py:181-286``) work unchanged.  The reference imports its
extension as ``vllm_gguf_plugin._C_gguf`` (``ops.py:42-48``); ``install_as("vllm_gguf_plugin._C_gguf")`` puts this
module under that name.

Two bindings define the same library.  ``_C_gguf_native.so`` (``csrc/torch_binding/gguf_torch_ops.cpp``, built by
``python -m vllm_gguf_plugin_prism_amd.build`` against the installed torch) registers the operators in C++, as the
reference's extension does, and is loaded when it is there: per call it allocates the output and the workspace with
torch and passes pointers and torch's current stream to the C ABI, without the interpreter.  Without it (or with
``GGUF_TORCH_BINDING=python`` in the environment) the same schemas are defined and implemented here in Python over
``vllm_gguf_plugin_prism_amd.ops``, which needs no build against a particular torch.  ``NATIVE`` says which one is active.

Fake (meta) functions are *not* registered on import: the reference registers its own when it finds the library
(``ops.py:110-175``) and torch refuses a second registration.  A caller without the reference's ``ops.py`` calls
``register_fakes()`` once to get the same shapes and dtypes for ``torch.compile``.
"""
from __future__ import annotations

import os
import sys
from pathlib import Path

import torch
from torch.library import Library

from . import _lib, ops

NATIVE_PATH = Path(__file__).resolve().parent / "_C_gguf_native.so"
NATIVE = False
if NATIVE_PATH.exists() and os.environ.get("GGUF_TORCH_BINDING", "native") != "python":
    _lib.lib()                                   # torch's HIP runtime and libgguf_hip.so first (see _lib.lib)
    try:
        torch.ops.load_library(str(NATIVE_PATH))
        NATIVE = True
    except OSError as exc:                       # built against another torch: the Python binding serves, and says why
        import warnings

        warnings.warn(f"{NATIVE_PATH.name} does not load with this torch ({exc}); rebuild it with "
                      "`python -m vllm_gguf_plugin_prism_amd.build`.  Using the Python binding.", RuntimeWarning)

SCHEMAS = (
    "ggml_dequantize(Tensor W, int type, SymInt m, SymInt n, ScalarType? dtype) -> Tensor",
    "ggml_mul_mat_vec_a8(Tensor W, Tensor X, int type, SymInt row) -> Tensor",
    "ggml_mul_mat_a8(Tensor W, Tensor X, int type, SymInt row) -> Tensor",
    "ggml_moe_a8(Tensor X, Tensor W, Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, "
    "int type, SymInt row, SymInt top_k, SymInt tokens) -> Tensor",
    "ggml_moe_a8_vec(Tensor X, Tensor W, Tensor topk_ids, int top_k, int type, SymInt row, SymInt tokens) -> Tensor",
    "ggml_moe_get_block_size(int type) -> int",
)

_def = None if NATIVE else Library("_C_gguf", "DEF")
for _schema in () if NATIVE else SCHEMAS:
    _def.define(_schema)


def _dequantize(W, type, m, n, dtype=None):
    return ops.ggml_dequantize(W, type, m, n, dtype)


def _mul_mat_vec_a8(W, X, type, row):
    return ops.ggml_mul_mat_vec_a8(W, X, type, row)


def _mul_mat_a8(W, X, type, row):
    return ops.ggml_mul_mat_a8(W, X, type, row)


def _moe_a8(X, W, sorted_token_ids, expert_ids, num_tokens_post_padded, type, row, top_k, tokens):
    return ops.ggml_moe_a8(X, W, sorted_token_ids, expert_ids, num_tokens_post_padded, type, row, top_k, tokens)


def _moe_a8_vec(X, W, topk_ids, top_k, type, row, tokens):
    return ops.ggml_moe_a8_vec(X, W, topk_ids, top_k, type, row, tokens)


def _moe_get_block_size(type):
    return ops.ggml_moe_get_block_size(type)


if not NATIVE:
    _def.impl("ggml_dequantize", _dequantize, "CUDA")
    _def.impl("ggml_mul_mat_vec_a8", _mul_mat_vec_a8, "CUDA")
    _def.impl("ggml_mul_mat_a8", _mul_mat_a8, "CUDA")
    _def.impl("ggml_moe_a8", _moe_a8, "CUDA")
    _def.impl("ggml_moe_a8_vec", _moe_a8_vec, "CUDA")
    _def.impl("ggml_moe_get_block_size", _moe_get_block_size, "CompositeExplicitAutograd")

_fakes_registered = False


def register_fakes() -> None:
    """Output shapes and dtypes of the five tensor operators for tracing, as the reference's ``ops.py:116-175`` has them."""
    global _fakes_registered
    if _fakes_registered:
        return
    from torch.library import register_fake

    @register_fake("_C_gguf::ggml_dequantize")
    def _(W, type, m, n, dtype=None):
        return torch.empty((m, n), dtype=dtype or torch.float16, device=W.device)

    @register_fake("_C_gguf::ggml_mul_mat_vec_a8")
    def _(W, X, type, row):
        return torch.empty((X.shape[0], row), dtype=X.dtype, device=W.device)

    @register_fake("_C_gguf::ggml_mul_mat_a8")
    def _(W, X, type, row):
        return torch.empty((X.size(0), row), dtype=X.dtype, device=W.device)

    @register_fake("_C_gguf::ggml_moe_a8")
    def _(X, W, sorted_token_ids, expert_ids, num_tokens_post_padded, type, row, top_k, tokens):
        return torch.empty((X.size(0) * top_k, row), dtype=X.dtype, device=W.device)

    @register_fake("_C_gguf::ggml_moe_a8_vec")
    def _(X, W, topk_ids, top_k, type, row, tokens):
        return torch.empty((X.size(0) * top_k, row), dtype=X.dtype, device=W.device)

    _fakes_registered = True


def install_as(module_name: str = "vllm_gguf_plugin._C_gguf") -> None:
    """Make ``import <module_name>`` (and ``from <package> import _C_gguf``) resolve to this module.

    With the parent package already imported the attribute is set on it as well, which is what
    ``from . import _C_gguf`` inside that package looks up first.
    """
    this = sys.modules[__name__]
    sys.modules[module_name] = this
    parent, _, leaf = module_name.rpartition(".")
    if parent and parent in sys.modules:
        setattr(sys.modules[parent], leaf, this)
