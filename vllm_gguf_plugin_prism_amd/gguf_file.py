"""Reader for GGUF v2/v3 files: metadata and the tensor table, with tensor data memory-mapped.

Stands in for ``gguf.GGUFReader`` as the reference's loader uses it
(vllm_gguf_plugin/weight_utils.py:150-201): tensors come back as the arrays the operators take —
``uint8[rows..., bytes_per_row]`` for quantized types, typed arrays for F32/F16, and ``uint16`` bit
patterns for BF16 — together with their ggml type id.  Files are never read whole: every array is a
view into one ``numpy.memmap``.

Layout (ggml's gguf specification): magic ``GGUF``, uint32 version, uint64 tensor count, uint64
key/value count, the key/value pairs, the tensor infos (name, dims innermost first, type, offset),
padding to ``general.alignment`` (32 if absent), tensor data.  A file written on a big-endian host is
recognised by its version field and read with swapped byte order.
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Any, Iterable, Iterator

import numpy as np

MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32

# ggml type id -> (elements per block, bytes per block); same table as triton/gemm/utils.py:28-47 of the reference
# plus the unquantized types
BLOCK_SIZES = {
    0: (1, 4), 1: (1, 2), 30: (1, 2),                                             # F32, F16, BF16
    2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
    16: (256, 66), 17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82),
    23: (256, 136), 24: (1, 1), 25: (1, 2), 26: (1, 4), 27: (1, 8), 28: (1, 8), 29: (256, 56),
}
TYPE_NAMES = {
    0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K", 11: "Q3_K",
    12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 16: "IQ2_XXS", 17: "IQ2_XS", 18: "IQ3_XXS", 19: "IQ1_S", 20: "IQ4_NL",
    21: "IQ3_S", 22: "IQ2_S", 23: "IQ4_XS", 24: "I8", 25: "I16", 26: "I32", 27: "I64", 28: "F64", 29: "IQ1_M", 30: "BF16",
}
_PLAIN_DTYPES = {0: "f4", 1: "f2", 30: "u2", 24: "i1", 25: "i2", 26: "i4", 27: "i8", 28: "f8"}
UNQUANTIZED = ("F32", "BF16", "F16")  # weight_utils.py:178

# metadata value types
_SCALARS = {0: "u1", 1: "i1", 2: "u2", 3: "i2", 4: "u4", 5: "i4", 6: "f4", 7: "?", 10: "u8", 11: "i8", 12: "f8"}
_T_STRING, _T_ARRAY = 8, 9


class GGUFError(ValueError):
    pass


@dataclass(frozen=True)
class TensorInfo:
    name: str
    ggml_type: int
    shape: tuple[int, ...]      # outermost first (numpy order); the last entry counts elements, not bytes
    offset: int                 # from the start of the file
    nbytes: int
    data: np.ndarray            # view into the file mapping, see the module docstring

    @property
    def type_name(self) -> str:
        return TYPE_NAMES.get(self.ggml_type, str(self.ggml_type))


class GGUFFile:
    """Parsed GGUF file.  ``metadata`` maps keys to Python values, ``tensors`` lists :class:`TensorInfo`."""

    def __init__(self, path: str | os.PathLike):
        self.path = os.fspath(path)
        self._map = np.memmap(self.path, dtype=np.uint8, mode="r")
        self._pos = 0
        if self._map.size < 24 or bytes(self._map[:4]) != MAGIC:
            raise GGUFError(f"{self.path}: not a GGUF file")
        self._pos = 4
        self.byte_order = "<"
        version = self._scalar("u4")
        if version & 0xFFFF == 0:  # written with the other byte order
            self.byte_order = ">"
            version = int(np.uint32(version).byteswap())
        if version not in (2, 3):
            raise GGUFError(f"{self.path}: unsupported GGUF version {version}")
        self.version = version
        n_tensors = self._scalar("u8")
        n_kv = self._scalar("u8")
        self.metadata: dict[str, Any] = {}
        for _ in range(n_kv):
            key = self._string()
            self.metadata[key] = self._value(self._scalar("u4"))
        self.alignment = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise GGUFError(f"{self.path}: alignment {self.alignment} is not a power of two")
        raw = []
        for _ in range(n_tensors):
            name = self._string()
            n_dims = self._scalar("u4")
            if n_dims > 4:
                raise GGUFError(f"{self.path}: tensor {name!r} has {n_dims} dimensions")
            dims = [self._scalar("u8") for _ in range(n_dims)]
            ggml_type = self._scalar("u4")
            offset = self._scalar("u8")
            raw.append((name, dims, ggml_type, offset))
        self.data_offset = (self._pos + self.alignment - 1) // self.alignment * self.alignment
        self.tensors: list[TensorInfo] = [self._tensor(*r) for r in raw]
        self._by_name = {t.name: t for t in self.tensors}

    # ------------------------------------------------------------------ primitives
    def _take(self, n: int) -> np.ndarray:
        if self._pos + n > self._map.size:
            raise GGUFError(f"{self.path}: truncated at byte {self._pos}")
        out = self._map[self._pos:self._pos + n]
        self._pos += n
        return out

    def _scalar(self, code: str):
        dt = np.dtype(code).newbyteorder(self.byte_order)
        return self._take(dt.itemsize).view(dt)[0].item()

    def _string(self) -> str:
        n = self._scalar("u8")
        return bytes(self._take(n)).decode("utf-8", errors="replace")

    def _value(self, vtype: int):
        if vtype in _SCALARS:
            return self._scalar(_SCALARS[vtype])
        if vtype == _T_STRING:
            return self._string()
        if vtype == _T_ARRAY:
            etype = self._scalar("u4")
            count = self._scalar("u8")
            if etype in _SCALARS:
                dt = np.dtype(_SCALARS[etype]).newbyteorder(self.byte_order)
                return self._take(dt.itemsize * count).view(dt).astype(dt.newbyteorder("=")).tolist()
            return [self._value(etype) for _ in range(count)]
        raise GGUFError(f"{self.path}: unknown metadata value type {vtype}")

    def _tensor(self, name: str, dims: list[int], ggml_type: int, rel_offset: int) -> TensorInfo:
        if ggml_type not in BLOCK_SIZES:
            raise GGUFError(f"{self.path}: tensor {name!r} has unknown ggml type {ggml_type}")
        qk, bs = BLOCK_SIZES[ggml_type]
        ne0 = dims[0] if dims else 1
        if ne0 % qk:
            raise GGUFError(f"{self.path}: tensor {name!r}: row length {ne0} is not a multiple of the block size {qk}")
        outer = [int(d) for d in reversed(dims[1:])]
        nelem = int(np.prod(dims, dtype=np.int64)) if dims else 1
        nbytes = nelem // qk * bs
        offset = self.data_offset + rel_offset
        if rel_offset % self.alignment or offset + nbytes > self._map.size:
            raise GGUFError(f"{self.path}: tensor {name!r} lies outside the file or is misaligned")
        buf = self._map[offset:offset + nbytes]
        if ggml_type in _PLAIN_DTYPES:
            dt = np.dtype(_PLAIN_DTYPES[ggml_type]).newbyteorder(self.byte_order)
            data = buf.view(dt).reshape(*outer, ne0)
            if self.byte_order == ">":
                data = data.astype(dt.newbyteorder("="))  # values in native order; a copy only for foreign files
        else:
            data = buf.reshape(*outer, ne0 // qk * bs)
        return TensorInfo(name, ggml_type, tuple(outer + [int(ne0)]), offset, nbytes, data)

    # ------------------------------------------------------------------ access
    def __getitem__(self, name: str) -> TensorInfo:
        return self._by_name[name]

    def __contains__(self, name: str) -> bool:
        return name in self._by_name

    def tensor_names(self) -> set[str]:
        return set(self._by_name)


def get_gguf_tensor_names(gguf_files: Iterable[str]) -> set[str]:
    """Raw tensor names across the files (weight_utils.py:150-156)."""
    return {t.name for f in gguf_files for t in GGUFFile(f).tensors}


def quant_weights_iterator(gguf_files: Iterable[str], name_map: dict[str, str] | None = None) -> Iterator[tuple[str, Any]]:
    """Yield ``(name, tensor)`` like ``gguf_quant_weights_iterator_multi`` (weight_utils.py:166-201).

    For every quantized tensor a ``(<name with "weight" -> "weight_type">, type id)`` entry comes first.  With a
    ``name_map`` tensors absent from it are skipped and the others renamed.  Tensors are torch tensors when torch is
    importable (BF16 as ``torch.bfloat16``), numpy arrays otherwise."""
    try:
        import torch
    except ImportError:  # pragma: no cover - torch is part of every supported environment
        torch = None
    for path in gguf_files:
        for t in GGUFFile(path).tensors:
            if name_map is not None:
                if t.name not in name_map:
                    continue
                name = name_map[t.name]
            else:
                name = t.name
            if t.type_name not in UNQUANTIZED:
                yield name.replace("weight", "weight_type"), (torch.tensor(t.ggml_type) if torch else t.ggml_type)
            if torch is None:
                yield name, t.data
            elif t.type_name == "BF16":
                yield name, torch.from_numpy(np.array(t.data)).view(torch.bfloat16)
            else:
                yield name, torch.from_numpy(np.array(t.data))
