"""The C-ABI library loads without a GPU and exports exactly what include/gguf_hip.h declares."""
import ctypes
import re
from pathlib import Path

import pytest

from vllm_gguf_plugin_prism_amd import _lib

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "gguf_hip.h"

# (elements, bytes) per block for every ggml type id of the reference's tables (triton/gemm/utils.py:28-47)
BLOCK_SIZES = {
    2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210),
    16: (256, 66), 17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82),
    23: (256, 136), 29: (256, 56),
}


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(gguf_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def handle():
    if not _lib.LIB_PATH.exists():
        from vllm_gguf_plugin_prism_amd import build

        build.build()
    return _lib.lib()


def test_header_declares_the_bound_entry_points():
    assert declared_symbols() == sorted(_lib.EXPORTS)
    assert len(declared_symbols()) == 34


def test_every_declared_symbol_is_exported(handle):
    raw = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_symbols():
        assert hasattr(raw, name), name


def test_version_names_the_target(handle):
    assert b"gfx950" in handle.gguf_hip_version()


def test_block_sizes_match_the_format_table(handle):
    for qt, (qk, nbytes) in BLOCK_SIZES.items():
        assert (handle.gguf_block_elems(qt), handle.gguf_block_bytes(qt)) == (qk, nbytes), qt
    for qt in (0, 1, 4, 5, 9, 15, 24, 30, 99, -3):
        assert handle.gguf_block_elems(qt) == 0 and handle.gguf_block_bytes(qt) == 0


def test_workspace_row_bytes(handle):
    # per 32 values of K rounded up to 512: int8 quants + three fp32 planes (44 bytes)
    assert handle.gguf_q8_1_row_bytes(4096) == 4096 // 32 * 44
    assert handle.gguf_q8_1_row_bytes(256) == 512 // 32 * 44
    assert handle.gguf_q8_1_row_bytes(14336) == 14336 // 32 * 44
    assert handle.gguf_q8_1_row_bytes(0) == 0


def test_moe_block_size(handle):
    for qt in (2, 8, 12, 14):
        assert handle.gguf_moe_block_size(qt) == 32
    assert handle.gguf_moe_block_size(99) == 0
    # blocks of 16 slots while an expert sees at most 12 pairs on average, for the formats that have such tiles
    assert handle.gguf_moe_block_size_for(2, 64 * 12, 64) == 16
    assert handle.gguf_moe_block_size_for(2, 64 * 12 + 1, 64) == 32
    assert handle.gguf_moe_block_size_for(2, 8, 0) == 32                  # expert count not stated
    assert handle.gguf_moe_block_size_for(3, 8, 64) == 32                 # Q4_1 has no 16-slot tiles
    assert handle.gguf_moe_block_size_for(99, 8, 64) == 0


def test_grouped_moe_states_its_limits_before_any_launch(handle):
    """More than 256 stated experts, a block other than 16 or 32, or blocks of 16 for a format without such tiles are
    refused by return code (the kernels would skip blocks of experts above 255 as moe.cuh:33 does)."""
    args = lambda qt, block, experts: (None, 1, None, None, 0, None, None, None, 64, None, qt, 128, 256, 2, 4, 0, block, experts, None)
    assert handle.gguf_moe_mmq_block(*args(2, 32, 257)) == -3
    assert handle.gguf_moe_mmq_block(*args(2, 8, 64)) == -3
    assert handle.gguf_moe_mmq_block(*args(3, 16, 64)) == -1
    assert handle.gguf_moe_mmq_block(*args(2, 16, 64)) == -4              # passes the checks; null pointers next


def test_workspace_sizes_by_engine(handle):
    m, n, k = 2048, 18944, 18944
    kp = (k + 511) // 512 * 512
    assert handle.gguf_q8_1_row_bytes(k) == kp // 32 * 44
    int8 = handle.gguf_mmq_workspace_bytes_engine(m, n, k, 1)
    half = handle.gguf_mmq_workspace_bytes_engine(m, n, k, 2)
    assert handle.gguf_mmq_workspace_bytes_engine(m, n, k, 0) == int8     # auto is the integer engine
    rows = m * kp // 32 * 44
    assert rows <= int8 < rows + (80 << 20)                                # quantized rows, then fp32 partial tiles
    assert half >= rows + m * 2 * (kp + 128)                               # only the half engine keeps half-precision rows
    assert handle.gguf_mmq_workspace_bytes(m, n, k) == max(int8, half)
    assert handle.gguf_mmq_workspace_bytes_engine(m, n, k, 3) == 0


def test_argument_validation_needs_no_gpu(handle):
    """Bad calls are rejected before any HIP call is made, so this runs on a machine without a GPU."""
    assert handle.gguf_dequantize(None, 99, None, 1, 256, None) == -1      # unknown type
    assert handle.gguf_dequantize(None, 12, None, 1, 100, None) == -3      # not a multiple of 256
    assert handle.gguf_dequantize(None, 12, None, 7, 256, None) == -2      # dtype code
    assert handle.gguf_dequantize(None, 12, None, 1, 256, None) == -4      # null pointers
    assert handle.gguf_dequantize(None, 12, None, 1, 0, None) == 0         # empty is fine
    assert handle.gguf_mmvq(None, None, 1, None, None, 99, 16, 256, 1, None) == -1
    assert handle.gguf_mmvq(None, None, 1, None, None, 12, 16, 100, 1, None) == -3
    assert handle.gguf_mmq(None, None, 1, None, None, 23, 16, 256, 1, None) in (-1, -4)


def _ctype_of(decl: str):
    """ctypes class of one C parameter or return type as include/gguf_hip.h spells it."""
    d = re.sub(r"\bconst\b", "", decl).strip()
    if d.startswith("char") and "*" in d:
        return ctypes.c_char_p
    if "*" in d or d.startswith("gguf_stream_t"):
        return ctypes.c_void_p            # every pointer, and the stream handle, crosses as an address
    base = d.split()[0]
    return {"int": ctypes.c_int, "int64_t": ctypes.c_int64, "void": None}[base]


def declared_prototypes():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ \*]*?)\b(gguf_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
        args = [] if params in ("", "void") else [_ctype_of(p) for p in params.split(",")]
        protos[name] = (_ctype_of(ret), args)
    return protos


def test_ctypes_signatures_match_the_header_type_for_type():
    """Argument count, order and width of every binding against the prototype it calls: an int passed where the
    header says int64_t, or two arguments swapped between a pointer and a size, would corrupt the call frame the way
    a surplus argument once did."""
    protos = declared_prototypes()
    assert sorted(protos) == sorted(_lib.EXPORTS)
    for name, (res, args) in _lib._SIGNATURES.items():
        want_res, want_args = protos[name]
        assert res is want_res, (name, res, want_res)
        assert list(args) == want_args, (name, [a.__name__ for a in args], [a.__name__ for a in want_args])


def test_two_launch_moe_layer_states_which_shapes_it_serves():
    """gguf_moe_vec_layer_takes needs no GPU: the OLMoE-like layer at one token and a Mixtral-like one are served; top_k
    times the waves a row takes beyond one workgroup, experts shared by more than 16 pairs each, unknown types and inner
    sizes that are not whole blocks are not; experts shared by a few pairs each take the tile route.  The workspace holds
    at least one q8_1 row of the inner size per pair and the quantized rows of X."""
    h = _lib.lib()
    assert h.gguf_moe_vec_layer_takes(2, 2, 2048, 1024, 2048, 8, 1, 64) == 1
    assert h.gguf_moe_vec_layer_takes(12, 14, 4096, 14336, 4096, 2, 1, 8) == 1
    assert h.gguf_moe_vec_layer_takes(2, 2, 2048, 8192, 2048, 8, 1, 64) == 0
    assert h.gguf_moe_vec_layer_takes(2, 2, 2048, 1024, 2048, 8, 64, 64) == 2      # 8 pairs per expert: the tile route
    assert h.gguf_moe_vec_layer_takes(2, 2, 2048, 1024, 2048, 8, 200, 64) == 3     # 25 pairs per expert: blocks of 32
    assert h.gguf_moe_vec_layer_takes(3, 3, 2048, 1024, 2048, 8, 64, 64) == 3       # Q4_1: blocks of 32 only
    assert h.gguf_moe_vec_layer_takes(6, 6, 2048, 1024, 2048, 8, 64, 64) == 0       # Q5_0: its tile arithmetic is not its GEMV's
    assert h.gguf_moe_vec_layer_takes(20, 20, 2048, 1024, 2048, 8, 64, 64) == 0     # IQ4_NL: shared experts, no tiles
    assert h.gguf_moe_vec_layer_takes(2, 2, 2048, 1024, 2048, 8, 200, 300) == 0     # more experts than the tiles' id guard admits
    assert h.gguf_moe_vec_layer_takes(1, 2, 2048, 1024, 2048, 8, 1, 64) == 0
    assert h.gguf_moe_vec_layer_takes(2, 12, 2048, 1120, 2048, 8, 1, 64) == 0
    assert h.gguf_moe_vec_layer_workspace_bytes(3, 8, 2048, 1024, 2048, 64, 1) >= 24 * h.gguf_q8_1_row_bytes(1024) + 3 * h.gguf_q8_1_row_bytes(2048)
    # the grouped operator's arithmetic: 1 = blocks of 16 slots (up to 16 pairs per expert on average, formats with such
    # tiles), 2 = blocks of 32, 3 = blocks of 64 in slot order on the dense engine; at most 256 experts
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 96, 64) == 1
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 128, 64) == 1
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 129, 64) == 2
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 512, 64) == 2
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 2048, 64) == 2
    assert h.gguf_moe_mmq_layer_takes(2, 14, 2048, 1024, 2048, 8, 2048, 64) == 3     # 256 pairs per expert, a 16-deep format: blocks of 64 on the dense engine
    assert h.gguf_moe_mmq_layer_takes(12, 14, 4096, 14336, 4096, 2, 512, 8) == 3
    assert h.gguf_moe_mmq_layer_workspace_bytes(2, 2, 96, 8, 2048, 1024, 2048, 64, 1) > 0
    assert h.gguf_moe_mmq_layer_workspace_bytes(2, 14, 2048, 8, 2048, 1024, 2048, 64, 1) > h.gguf_moe_mmq_layer_workspace_bytes(2, 2, 2048, 8, 2048, 1024, 2048, 64, 1)
    assert h.gguf_moe_mmq_layer_workspace_bytes(20, 2, 96, 8, 2048, 1024, 2048, 64, 1) == 0
    assert h.gguf_moe_mmq_layer_takes(3, 2, 2048, 1024, 2048, 8, 96, 64) == 2       # Q4_1: blocks of 32 only
    assert h.gguf_moe_mmq_layer_takes(20, 2, 2048, 1024, 2048, 8, 96, 64) == 0      # IQ4_NL has no tile kernel
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 96, 300) == 0
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1024, 2048, 8, 96, 0) == 0
    assert h.gguf_moe_mmq_layer_takes(2, 2, 2048, 1000, 2048, 8, 96, 64) == 0       # inner size not in whole blocks
    assert h.gguf_moe_mmq_layer(None, 1, None, 2, None, 2, None, None, None, 0, None, 2048, 1024, 2048, 8, 96, 1, 64, None) == -4
    assert h.gguf_moe_mmq_layer(None, 1, None, 2, None, 2, None, None, None, 0, None, 2048, 1024, 2048, 8, 200, 1, 300, None) == -3
    assert h.gguf_moe_vec_layer(None, 1, None, 2, None, 2, None, None, None, 0, None, 2048, 1024, 2048, 8, 1, 0, 64, None) == -3
    assert h.gguf_moe_vec_layer(None, 1, None, 2, None, 2, None, None, None, 0, None, 2048, 1024, 2048, 8, 1, 1, 64, None) == -4
