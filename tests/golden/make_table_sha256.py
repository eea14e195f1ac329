#!/usr/bin/env python3
"""Writes tests/golden/table_sha256.json: sha256 of the little-endian bytes of every codebook table in the
reference's csrc/gguf/ggml-common.h:193-1060.  The header is read as text (it is data: nothing from the reference is
imported or run) and only the hashes leave this script, so the fixture can be checked where the reference is absent.

    python tests/golden/make_table_sha256.py [/root/reference]
"""
import hashlib
import json
import os
import re
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
TABLES = [  # name, C element type, numpy dtype, entries
    ("iq2xxs_grid", "uint64_t", "<u8", 256), ("iq2xs_grid", "uint64_t", "<u8", 512), ("iq2s_grid", "uint64_t", "<u8", 1024),
    ("iq3xxs_grid", "uint32_t", "<u4", 256), ("iq3xs_grid", "uint32_t", "<u4", 512), ("iq1s_grid_gpu", "uint64_t", "<u8", 2048),
    ("ksigns_iq2xs", "uint8_t", "u1", 128), ("ksigns64", "uint64_t", "<u8", 128), ("kvalues_iq4nl", "int8_t", "i1", 16),
]


def table(text: str, name: str, ctype: str, size: int):
    m = re.search(r"static const __device__ %s %s\[%d\] = \{" % (ctype, re.escape(name), size), text)
    if m is None:
        raise SystemExit(f"{name}[{size}] not found")
    body = text[m.end():text.index("};", m.end())]
    vals = [int(v, 0) for v in re.findall(r"-?(?:0x[0-9a-fA-F]+|\d+)", body)]
    if len(vals) != size:
        raise SystemExit(f"{name}: {len(vals)} values, expected {size}")
    return vals


def main() -> int:
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    text = open(os.path.join(root, "vllm_gguf_plugin", "csrc", "gguf", "ggml-common.h")).read()
    out = {}
    for name, ctype, dtype, size in TABLES:
        out[name] = hashlib.sha256(np.array(table(text, name, ctype, size), dtype=dtype).tobytes()).hexdigest()
    with open(os.path.join(HERE, "table_sha256.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
