"""Codebook tables: decoded contents pinned by sha256, closed forms and value-set invariants.

The hashes in tests/golden/table_sha256.json are of the little-endian bytes of the
tables in the reference's csrc/gguf/ggml-common.h:193-1060.
"""
import hashlib
import json
import os
import re

import numpy as np
import pytest

from vllm_gguf_plugin_prism_amd.tables import grids

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "table_sha256.json")
REF_HEADER = "/root/reference/vllm_gguf_plugin/csrc/gguf/ggml-common.h"

NAMES = ["iq2xxs_grid", "iq2xs_grid", "iq2s_grid", "iq3xxs_grid", "iq3xs_grid", "iq1s_grid_gpu", "ksigns_iq2xs", "ksigns64"]


def _le_bytes(a: np.ndarray) -> bytes:
    return a.astype(a.dtype.newbyteorder("<")).tobytes()


@pytest.mark.parametrize("name", NAMES)
def test_table_sha256(name):
    sha = json.load(open(GOLDEN))
    assert hashlib.sha256(_le_bytes(getattr(grids, name)())).hexdigest() == sha[name]


def test_kvalues_sha256():
    sha = json.load(open(GOLDEN))
    assert hashlib.sha256(grids.kvalues_iq4nl().tobytes()).hexdigest() == sha["kvalues_iq4nl"]
    assert list(grids.kvalues_iq4nl()) == [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]


def test_sign_tables_closed_form():
    ks = grids.ksigns_iq2xs()
    for i in range(128):
        assert ks[i] == (i | ((bin(i).count("1") & 1) << 7))
        assert bin(int(ks[i])).count("1") % 2 == 0
    k64 = grids.ksigns64()
    for i in range(128):
        for j in range(8):
            assert (int(k64[i]) >> (8 * j)) & 0xFF == (0xFF if (int(ks[i]) >> j) & 1 else 0)
    assert list(grids.kmask_iq2xs()) == [1, 2, 4, 8, 16, 32, 64, 128]


def test_value_sets():
    # same spirit as the reference's tests/test_ggml_common_tables.py:40-44
    assert set(grids.grid_bytes(grids.iq3xs_grid()).ravel() // 4) == {1, 3, 5, 7, 9, 11, 13, 15}
    assert all(v % 4 == 0 for v in grids.grid_bytes(grids.iq3xs_grid()).ravel())
    for g in (grids.iq2xxs_grid(), grids.iq2xs_grid(), grids.iq2s_grid()):
        assert set(grids.grid_bytes(g).ravel()) == {8, 25, 43}
        assert np.all(np.diff(g.astype(np.uint64)) > 0)  # ascending, so no duplicate entries
    assert set(grids.grid_bytes(grids.iq3xxs_grid()).ravel()) == {4, 12, 20, 28, 36, 44, 52, 62}
    g1 = grids.iq1s_grid_gpu()
    assert int(g1.max()) < 1 << 32
    nib = {(int(v) >> (4 * j)) & 0xF for v in g1 for j in range(8)}
    assert nib == {0, 1, 2}


def test_c_header_matches_python_codes():
    hdr = grids.emit_c_header()
    vals = [int(v, 16) for v in re.findall(r"0x[0-9a-f]{4}", hdr)]
    assert len(vals) == 256 + 512 + 1024 + 256 + 512 + 2048


@pytest.mark.skipif(not os.path.exists(REF_HEADER), reason="reference tree not mounted")
def test_tables_against_reference_header_text():
    text = open(REF_HEADER).read()

    def words(name, bits, size):
        marker = f"static const __device__ uint{bits}_t {name}[{size}] = {{"
        start = text.index(marker) + len(marker)
        end = text.index("};", start)
        return [int(v, 16) for v in re.findall(r"0x[0-9a-fA-F]+", text[start:end])]

    for name, bits, size in [("iq2xxs_grid", 64, 256), ("iq2xs_grid", 64, 512), ("iq2s_grid", 64, 1024),
                             ("iq3xxs_grid", 32, 256), ("iq3xs_grid", 32, 512), ("iq1s_grid_gpu", 64, 2048),
                             ("ksigns64", 64, 128)]:
        assert [int(v) for v in getattr(grids, name)()] == words(name, bits, size), name
