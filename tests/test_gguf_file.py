"""GGUF reader against files laid out by hand from the format specification.

No GGUF file ships with the reference (its tests download theirs) and gguf-py is not installed, so agreement with
``gguf.GGUFReader`` on real files is not pinned here; what is pinned is the layout the specification fixes: header,
typed key/values incl. nested arrays, tensor infos with innermost-first dims, alignment padding, foreign byte order.
"""
import struct

import numpy as np
import pytest
import torch

from vllm_gguf_plugin_prism_amd import gguf_file as G
from vllm_gguf_plugin_prism_amd import synth


class Writer:
    """Minimal GGUF v3 writer, little- or big-endian, for test fixtures only."""

    def __init__(self, bo="<", version=3, alignment=None):
        self.bo, self.version, self.alignment = bo, version, alignment
        self.kv, self.tensors = [], []

    def s(self, text):
        b = text.encode()
        return struct.pack(self.bo + "Q", len(b)) + b

    def add_kv(self, key, vtype, payload):
        self.kv.append(self.s(key) + struct.pack(self.bo + "I", vtype) + payload)

    def add_tensor(self, name, dims_inner_first, ggml_type, raw_bytes):
        self.tensors.append((name, dims_inner_first, ggml_type, raw_bytes))

    def write(self, path):
        align = self.alignment or 32
        if self.alignment:
            self.add_kv("general.alignment", 4, struct.pack(self.bo + "I", self.alignment))
        head = b"GGUF" + struct.pack(self.bo + "IQQ", self.version, len(self.tensors), len(self.kv)) + b"".join(self.kv)
        infos, blobs, off = b"", b"", 0
        for name, dims, t, raw in self.tensors:
            infos += self.s(name) + struct.pack(self.bo + "I", len(dims)) + b"".join(struct.pack(self.bo + "Q", d) for d in dims)
            infos += struct.pack(self.bo + "IQ", t, off)
            pad = (-len(raw)) % align
            blobs += raw + b"\0" * pad
            off += len(raw) + pad
        head += infos
        head += b"\0" * ((-len(head)) % align)
        with open(path, "wb") as f:
            f.write(head + blobs)


def _fixture(tmp_path, bo="<", alignment=None):
    rng = np.random.default_rng(5)
    w = Writer(bo, alignment=alignment)
    w.add_kv("general.architecture", 8, w.s("llama"))
    w.add_kv("llama.block_count", 4, struct.pack(bo + "I", 2))
    w.add_kv("llama.rope.freq_base", 6, struct.pack(bo + "f", 10000.0))
    w.add_kv("flag", 7, b"\x01")
    w.add_kv("big", 10, struct.pack(bo + "Q", 2 ** 40 + 3))
    w.add_kv("neg", 11, struct.pack(bo + "q", -5))
    w.add_kv("pi", 12, struct.pack(bo + "d", 3.25))
    w.add_kv("tokens", 9, struct.pack(bo + "IQ", 8, 3) + w.s("a") + w.s("bc") + w.s(""))
    w.add_kv("scores", 9, struct.pack(bo + "IQ", 6, 4) + struct.pack(bo + "4f", 0.5, -1.0, 2.0, 4.0))
    w.add_kv("nested", 9, struct.pack(bo + "IQ", 9, 2) + struct.pack(bo + "IQ", 5, 2) + struct.pack(bo + "2i", 1, -2)
             + struct.pack(bo + "IQ", 5, 1) + struct.pack(bo + "i", 7))
    dt = np.dtype("f4").newbyteorder(bo)
    f32 = rng.standard_normal((3, 8)).astype(np.float32)
    w.add_tensor("output_norm.weight", [8, 3], 0, f32.astype(dt).tobytes())
    f16 = rng.standard_normal((4, 16)).astype(np.float16)
    w.add_tensor("tok.f16", [16, 4], 1, f16.astype(np.dtype("f2").newbyteorder(bo)).tobytes())
    bf = (rng.standard_normal((2, 32)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    w.add_tensor("blk.0.bf.weight", [32, 2], 30, bf.astype(np.dtype("u2").newbyteorder(bo)).tobytes())
    q8 = synth.make_weights(rng, 8, 6, 64)
    w.add_tensor("blk.0.attn_q.weight", [64, 6], 8, q8.tobytes())
    q4k = synth.make_weights(rng, 12, 5, 512)
    w.add_tensor("blk.0.ffn_up.weight", [512, 5], 12, q4k.tobytes())
    ex = np.stack([synth.random_blocks(rng, 2, 4, 64) for _ in range(3)])
    w.add_tensor("blk.0.ffn_gate_exps.weight", [64, 4, 3], 2, ex.tobytes())
    path = tmp_path / f"t_{'le' if bo == '<' else 'be'}_{alignment}.gguf"
    w.write(path)
    return path, dict(f32=f32, f16=f16, bf=bf, q8=q8, q4k=q4k, ex=ex)


@pytest.mark.parametrize("bo,alignment", [("<", None), ("<", 64), (">", None)])
def test_reads_metadata_and_tensors(tmp_path, bo, alignment):
    path, ref = _fixture(tmp_path, bo, alignment)
    g = G.GGUFFile(path)
    assert g.version == 3 and g.byte_order == bo and g.alignment == (alignment or 32)
    md = g.metadata
    assert md["general.architecture"] == "llama" and md["llama.block_count"] == 2 and md["llama.rope.freq_base"] == 10000.0
    assert md["flag"] is True and md["big"] == 2 ** 40 + 3 and md["neg"] == -5 and md["pi"] == 3.25
    assert md["tokens"] == ["a", "bc", ""] and md["scores"] == [0.5, -1.0, 2.0, 4.0] and md["nested"] == [[1, -2], [7]]
    assert [t.name for t in g.tensors] == ["output_norm.weight", "tok.f16", "blk.0.bf.weight", "blk.0.attn_q.weight",
                                           "blk.0.ffn_up.weight", "blk.0.ffn_gate_exps.weight"]
    assert all(t.offset % g.alignment == 0 for t in g.tensors)
    t = g["output_norm.weight"]
    assert t.type_name == "F32" and t.shape == (3, 8) and np.array_equal(t.data, ref["f32"])
    t = g["tok.f16"]
    assert t.shape == (4, 16) and t.data.dtype.itemsize == 2 and np.array_equal(np.asarray(t.data, dtype=np.float16), ref["f16"])
    t = g["blk.0.bf.weight"]
    assert t.type_name == "BF16" and np.array_equal(np.asarray(t.data, dtype=np.uint16), ref["bf"])
    t = g["blk.0.attn_q.weight"]
    assert t.ggml_type == 8 and t.shape == (6, 64) and t.data.dtype == np.uint8 and t.data.shape == (6, 68)
    assert np.array_equal(t.data, ref["q8"])
    t = g["blk.0.ffn_up.weight"]
    assert t.shape == (5, 512) and t.data.shape == (5, 288) and np.array_equal(t.data, ref["q4k"])
    t = g["blk.0.ffn_gate_exps.weight"]
    assert t.shape == (3, 4, 64) and t.data.shape == (3, 4, 36) and np.array_equal(t.data, ref["ex"])
    assert "tok.f16" in g and g.tensor_names() == {x.name for x in g.tensors}


def test_weight_iterator_contract(tmp_path):
    path, ref = _fixture(tmp_path)
    items = list(G.quant_weights_iterator([str(path)]))
    names = [n for n, _ in items]
    # unquantized tensors have no type entry; every quantized one is preceded by its "<...>weight_type" id
    assert names == ["output_norm.weight", "tok.f16", "blk.0.bf.weight", "blk.0.attn_q.weight_type", "blk.0.attn_q.weight",
                     "blk.0.ffn_up.weight_type", "blk.0.ffn_up.weight", "blk.0.ffn_gate_exps.weight_type",
                     "blk.0.ffn_gate_exps.weight"]
    d = dict(items)
    assert int(d["blk.0.attn_q.weight_type"]) == 8 and int(d["blk.0.ffn_up.weight_type"]) == 12
    assert d["blk.0.bf.weight"].dtype == torch.bfloat16
    assert torch.equal(d["blk.0.bf.weight"].view(torch.int16), torch.from_numpy(ref["bf"].view(np.int16)))
    assert d["blk.0.ffn_up.weight"].dtype == torch.uint8 and tuple(d["blk.0.ffn_up.weight"].shape) == (5, 288)
    mapped = list(G.quant_weights_iterator([str(path)], {"tok.f16": "model.embed.weight", "blk.0.attn_q.weight": "q.weight"}))
    assert [n for n, _ in mapped] == ["model.embed.weight", "q.weight_type", "q.weight"]
    assert G.get_gguf_tensor_names([str(path)]) == {t for t in names if not t.endswith("_type")}


def test_rejects_malformed_files(tmp_path):
    p = tmp_path / "x.gguf"
    p.write_bytes(b"NOPE" + b"\0" * 40)
    with pytest.raises(G.GGUFError):
        G.GGUFFile(p)
    w = Writer(version=1)
    w.write(p)
    with pytest.raises(G.GGUFError):
        G.GGUFFile(p)
    w = Writer()
    w.add_tensor("bad", [100], 12, b"\0" * 144)   # Q4_K row of 100 elements is not a whole number of blocks
    w.write(p)
    with pytest.raises(G.GGUFError):
        G.GGUFFile(p)
    path, _ = _fixture(tmp_path)
    data = path.read_bytes()
    p.write_bytes(data[:-200])                     # truncated tensor data
    with pytest.raises(G.GGUFError):
        G.GGUFFile(p)


def test_block_size_table_matches_the_library():
    from vllm_gguf_plugin_prism_amd import _lib

    if not _lib.LIB_PATH.exists():
        pytest.skip("library not built")
    L = _lib.lib()
    for t, (qk, bs) in G.BLOCK_SIZES.items():
        if L.gguf_block_elems(t):
            assert (L.gguf_block_elems(t), L.gguf_block_bytes(t)) == (qk, bs)
