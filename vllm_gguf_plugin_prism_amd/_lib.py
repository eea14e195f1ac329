"""ctypes binding of libgguf_hip.so (the C ABI declared in include/gguf_hip.h)."""
from __future__ import annotations

import ctypes
import os
from pathlib import Path

_PKG = Path(__file__).resolve().parent
LIB_PATH = _PKG / "libgguf_hip.so"

ERRORS = {
    -1: "ggml type not supported by this entry point",
    -2: "unsupported dtype (need float32, float16 or bfloat16)",
    -3: "bad shape (K must be a positive multiple of the block size; sizes must be non-negative)",
    -4: "null pointer",
    -5: "kernel launch failed",
    -6: "the call needs more workspace than this entry point has",
}

_lib = None

_c = ctypes
_SIGNATURES = {
    "gguf_hip_version": (_c.c_char_p, []),
    "gguf_block_elems": (_c.c_int, [_c.c_int]),
    "gguf_block_bytes": (_c.c_int, [_c.c_int]),
    "gguf_q8_1_row_bytes": (_c.c_int64, [_c.c_int64]),
    "gguf_quantize_q8_1": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_q8_1_unpack": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_dequantize": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_void_p]),
    "gguf_dequantize_rows": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p,
                                        _c.c_int, _c.c_void_p]),
    "gguf_mmvq": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64,
                             _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_mmq": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64,
                            _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_mmvq_linear": (_c.c_int, [_c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64,
                                    _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_mmq_linear": (_c.c_int, [_c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64,
                                   _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_int64, _c.c_void_p]),
    "gguf_mmq_workspace_bytes": (_c.c_int64, [_c.c_int64, _c.c_int64, _c.c_int64]),
    "gguf_mmq_workspace_bytes_engine": (_c.c_int64, [_c.c_int64, _c.c_int64, _c.c_int64, _c.c_int]),
    "gguf_mmq_static_capacity": (_c.c_int64, []),
    "gguf_mmq_static": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64,
                                   _c.c_void_p]),
    "gguf_mmq_engine": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64,
                                   _c.c_int64, _c.c_int64, _c.c_int, _c.c_int64, _c.c_void_p]),
    "gguf_dequant_gemm": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64,
                                     _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_moe_mmq": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p,
                                _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64,
                                _c.c_int64, _c.c_void_p]),
    "gguf_moe_vec": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int,
                                _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_moe_mmq_act": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p,
                                    _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64,
                                    _c.c_int64, _c.c_int, _c.c_void_p]),
    "gguf_moe_vec_act": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int,
                                    _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int, _c.c_int64, _c.c_int64,
                                    _c.c_void_p]),
    "gguf_moe_vec_workspace_bytes": (_c.c_int64, [_c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64]),
    "gguf_moe_block_size": (_c.c_int, [_c.c_int]),
    "gguf_moe_block_size_for": (_c.c_int, [_c.c_int, _c.c_int64, _c.c_int64]),
    "gguf_moe_mmq_block": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p,
                                      _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64,
                                      _c.c_int64, _c.c_int, _c.c_int64, _c.c_int64, _c.c_void_p]),
    "gguf_moe_align_block_size": (_c.c_int, [_c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_void_p, _c.c_int64,
                                             _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p]),
    "gguf_moe_weighted_sum": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int, _c.c_int64, _c.c_int64,
                                         _c.c_int64, _c.c_void_p]),
    "gguf_moe_vec_layer_takes": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64]),
    "gguf_moe_vec_layer_workspace_bytes": (_c.c_int64, [_c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int]),
    "gguf_moe_vec_layer": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p,
                                      _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
                                      _c.c_int, _c.c_int64, _c.c_void_p]),
    "gguf_moe_mmq_layer_takes": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64]),
    "gguf_moe_mmq_layer_workspace_bytes": (_c.c_int64, [_c.c_int, _c.c_int, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
                                                        _c.c_int]),
    "gguf_moe_mmq_layer": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int, _c.c_void_p, _c.c_void_p,
                                      _c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int64,
                                      _c.c_int, _c.c_int64, _c.c_void_p]),
}
EXPORTS = tuple(_SIGNATURES)


class _Bound:
    """The library's entry points as attributes."""


def _exact_arity(fn, name: str, nargs: int):
    # ctypes accepts surplus arguments silently; one too many would land in the stream parameter
    def call(*args):
        if len(args) != nargs:
            raise TypeError(f"{name} takes {nargs} arguments, got {len(args)}")
        return fn(*args)

    call.__name__ = name
    return call


def lib() -> "_Bound":
    """Load the HIP library; there is no fallback path, a missing library is an error."""
    global _lib
    if _lib is None:
        path = os.environ.get("GGUF_HIP_LIBRARY", str(LIB_PATH))
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: build it with `python -m vllm_gguf_plugin_prism_amd.build` "
                "(hipcc, gfx950).  This package has no non-HIP implementation."
            )
        # The process must hold one HIP runtime.  torch ships its own libamdhip64; if this library were loaded first it
        # would bring in the system's copy, torch would later add its own, and kernels launched through the one on
        # pointers and streams of the other fail to launch.  With torch's copy loaded first, this library's dependency
        # on the same soname resolves to it.
        import torch  # noqa: F401

        handle = ctypes.CDLL(path)
        bound = _Bound()
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
            setattr(bound, name, _exact_arity(fn, name, len(args)))
        bound._handle = handle
        _lib = bound
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = ERRORS.get(rc, f"error {rc}")
        if rc == -1:
            raise NotImplementedError(f"{what}: {msg}")
        raise ValueError(f"{what}: {msg}")
