"""The callers' layer on the GPU: dense dispatch, the two-stage MoE pipeline and embedding lookup,
each checked against the numpy oracle (the in-tree definition of the MoE result is the per-token
loop at quantization/fused_moe.py:119-132)."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd import dispatch as D
from vllm_gguf_plugin_prism_amd import synth

pytestmark = pytest.mark.gpu


def _moe_oracle(x, w1, w2, tw, ids, qt, qt2, path):
    """Two-stage MoE in fp64 with the activations re-quantised to q8_1 before each GEMM, as the kernels see them.
    The intermediate is rounded to fp16 where the device stores it."""
    tokens, top_k = ids.shape
    n1, n2 = w1.shape[1], w2.shape[1]
    h = o.moe_a8_vec(x, w1, ids.reshape(-1), top_k, qt, n1, tokens) if path == "vec" else None
    if h is None:
        blk = 32
        s, e, n = o.moe_align_block_size(ids, blk, w1.shape[0])
        h = o.moe_a8(x, w1, s, e, n, qt, n1, top_k, tokens, blk)
    h = h.astype(np.float16)
    a = o.silu_and_mul(h.astype(np.float64)).astype(np.float16)
    y = o.moe_a8_vec(a, w2, ids.reshape(-1), 1, qt2, n2, tokens * top_k).astype(np.float16).astype(np.float64)
    y = y.reshape(tokens, top_k, n2) * tw.astype(np.float16).astype(np.float64)[:, :, None]
    return y.astype(np.float16).astype(np.float64).sum(1)


@pytest.mark.parametrize("tokens,expected_path", [(1, "vec"), (9, "vec"), (96, "grouped")])
def test_fused_moe_pipeline_q4_0(tokens, expected_path):
    """Reduced shape of the Q4_0 MoE config: 8 experts, hidden 512, intermediate 256, top-2."""
    rng = np.random.default_rng(tokens)
    E, H, I, top_k = 8, 512, 256, 2
    w1 = np.stack([synth.make_weights(rng, o.Q4_0, 2 * I, H) for _ in range(E)])
    w2 = np.stack([synth.make_weights(rng, o.Q4_0, H, I) for _ in range(E)])
    # weights ~N(0,0.02) give tiny activations; scale x so intermediate values are O(1)
    x = (rng.standard_normal((tokens, H)) * 4).astype(np.float16)
    logits = rng.standard_normal((tokens, E))
    ids = np.argsort(-logits, axis=1)[:, :top_k].astype(np.int32)
    sel = np.take_along_axis(logits, ids, 1)
    tw = (np.exp(sel) / np.exp(sel).sum(1, keepdims=True)).astype(np.float32)
    assert D.select_moe_path(o.Q4_0, o.Q4_0, tokens) == expected_path
    got = D.fused_moe_gguf(torch.from_numpy(x).cuda(), torch.from_numpy(w1).cuda(), torch.from_numpy(w2).cuda(),
                           torch.from_numpy(tw).cuda().half(), torch.from_numpy(ids).cuda(), o.Q4_0, o.Q4_0, "silu")
    torch.cuda.synchronize()
    assert got.shape == (tokens, H) and got.dtype == torch.float16
    want = _moe_oracle(x, w1, w2, tw, ids, o.Q4_0, o.Q4_0, expected_path)
    # fp16 storage between stages and the re-quantisation of a slightly different intermediate bound the error
    assert o.rel_l2(got.float().cpu().numpy(), want) <= 1e-2


@pytest.mark.parametrize("qt,qt2", [(o.Q4_0, o.Q4_0), (o.Q4_K, o.Q6_K)])
@pytest.mark.parametrize("tokens", [2, 30, 100, 400])
def test_fused_moe_with_activations_of_one_sign(tokens, qt, qt2):
    """The MoE layer on token rows whose values share a sign (block sums of the quantized rows far from zero, the offset
    terms of Q4_0 / Q4_K as large as their product terms), through every route of the layer: two launches (2 tokens),
    16-slot tiles (30), 32-slot tiles (100) and, for the Q6_K down projection, the slot order on the dense engine (400
    tokens, 200 pairs per expert).  Two links: each separate operator against the a8 oracle on the inputs it was given,
    and the layer against the separate operators chained with the reference's roundings between them
    (fused_moe.py:62-95).  (The layer is not held to an oracle that forms its own intermediate: on these inputs one
    intermediate value in a hundred moved by a half-precision step flips the roundings of the half-precision block sums
    that Q4_0's offset term multiplies (vecdotq.cuh:46-66) and moves the oracle's own result by 8e-4 while one q8_1 code
    in 30000 changes, so such a comparison measures the conditioning of the reference's arithmetic, not the kernels.)"""
    from vllm_gguf_plugin_prism_amd import ops
    rng = np.random.default_rng(7000 + tokens + qt)
    E, H, I, top_k = 4, 512, 256, 2
    w1 = np.stack([synth.make_weights(rng, qt, 2 * I, H) for _ in range(E)])
    w2 = np.stack([synth.make_weights(rng, qt2, H, I) for _ in range(E)])
    x = (4.0 * (1.0 + 0.3 * rng.standard_normal((tokens, H)))).astype(np.float16)
    logits = rng.standard_normal((tokens, E))
    ids = np.argsort(-logits, axis=1)[:, :top_k].astype(np.int32)
    sel = np.take_along_axis(logits, ids, 1)
    tw = (np.exp(sel) / np.exp(sel).sum(1, keepdims=True)).astype(np.float32)
    xd, w1d, w2d, idd = torch.from_numpy(x).cuda(), torch.from_numpy(w1).cuda(), torch.from_numpy(w2).cuda(), torch.from_numpy(ids).cuda()
    got = D.fused_moe_gguf(xd, w1d, w2d, torch.from_numpy(tw).cuda().half(), idd, qt, qt2, "silu")
    torch.cuda.synchronize()
    assert got.shape == (tokens, H) and torch.isfinite(got).all()
    pairs, flat = tokens * top_k, ids.reshape(-1)
    if D.select_moe_path(qt, qt2, tokens) == "vec":
        h = ops.ggml_moe_a8_vec(xd, w1d, idd, top_k, qt, 2 * I, tokens)
        h_or = o.moe_a8_vec(x.astype(np.float32), w1, flat, top_k, qt, 2 * I, tokens)
        a = o.silu_and_mul(h.cpu().numpy(), stored=np.float16)
        y = ops.ggml_moe_a8_vec(torch.from_numpy(a).cuda(), w2d, idd.reshape(-1, 1).contiguous(), 1, qt2, H, pairs)
        y_or = o.moe_a8_vec(a.astype(np.float32), w2, flat, 1, qt2, H, pairs)
    else:
        blk = ops.ggml_moe_get_block_size(qt)
        s_, eids, npost = o.moe_align_block_size(ids, blk, E)
        sd, ed, nd = (torch.from_numpy(np.ascontiguousarray(v)).cuda() for v in (s_, eids, npost))
        h = ops.ggml_moe_a8(xd, w1d, sd, ed, nd, qt, 2 * I, top_k, tokens)
        h_or = o.moe_a8(x.astype(np.float32), w1, s_, eids, npost, qt, 2 * I, top_k, tokens, blk)
        a = o.silu_and_mul(h.cpu().numpy(), stored=np.float16)
        y = ops.ggml_moe_a8(torch.from_numpy(a).cuda(), w2d, sd, ed, nd, qt2, H, 1, pairs)
        y_or = o.moe_a8(a.astype(np.float32), w2, s_, eids, npost, qt2, H, 1, pairs, blk)
    assert o.rel_l2(h.float().cpu().numpy(), h_or) <= 1e-3 and o.rel_l2(y.float().cpu().numpy(), y_or) <= 1e-3
    yy = y.cpu().numpy().astype(np.float64).reshape(tokens, top_k, H)
    want = (yy * tw.astype(np.float16).astype(np.float64)[:, :, None]).astype(np.float16).astype(np.float64).sum(1)
    err = o.rel_l2(got.float().cpu().numpy(), want)
    assert err <= 5e-4, (tokens, o.TYPE_NAMES[qt], o.TYPE_NAMES[qt2], err)    # (the result's own rounding to half: 2.2e-4)


@pytest.mark.parametrize("qt,batch,rows,path", [(o.Q4_K, 2, 64, "mmvq"), (o.Q4_K, 7, 64, "mmq"),
                                                (o.IQ4_XS, 3, 64, "mmvq"), (o.IQ4_XS, 40, 64, "dequant")])
def test_fused_mul_mat_routes(qt, batch, rows, path):
    rng = np.random.default_rng(rows + batch)
    k = 512
    w = synth.make_weights(rng, qt, rows, k)
    x = rng.standard_normal((batch, k)).astype(np.float16)
    assert D.select_mul_mat_path(qt, batch, rows) == path
    got = D.fused_mul_mat_gguf(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), qt).float().cpu().numpy()
    if path == "dequant":
        want = o.mul_mat_f32(w, x, qt, rows)
        assert o.rel_l2(got, want) <= 2e-3          # fp16 dense GEMM on exactly dequantised weights
    else:
        want = o.mul_mat_a8(w, x, qt, rows, path=path)
        assert o.rel_l2(got, want) <= 1e-3


@pytest.mark.parametrize("qt", [o.Q8_0, o.Q4_K, o.IQ2_XXS, o.Q5_1, o.Q3_K, o.IQ1_M, o.IQ3_S])
def test_embedding_lookup_is_gather_of_exact_dequant(qt):
    rng = np.random.default_rng(qt)
    vocab, hidden = 50, 512
    table = synth.make_weights(rng, qt, vocab, hidden)
    ids = rng.integers(0, vocab, size=(3, 5))
    got = D.apply_gguf_embedding(torch.from_numpy(ids).cuda(), torch.from_numpy(table).cuda(), qt, hidden, torch.float16)
    assert got.shape == (3, 5, hidden)
    dense = o.dequantize(table, qt, "f16").reshape(vocab, hidden)
    assert np.array_equal(got.cpu().numpy().view(np.uint16), dense[ids].view(np.uint16))


@pytest.mark.parametrize("tokens,top_k,experts,block", [(1, 8, 64, 32), (7, 2, 4, 32), (512, 8, 64, 32), (33, 3, 5, 4),
                                                        (2000, 2, 300, 32), (5, 1, 3, 8), (9000, 8, 1024, 16),
                                                        (4096, 8, 64, 64), (100, 1, 1, 32)])
def test_native_moe_align_block_size_matches_checker(tokens, top_k, experts, block):
    from vllm_gguf_plugin_prism_amd import ops

    rng = np.random.default_rng(tokens * 7 + experts)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    s, e, n = ops.moe_align_block_size(torch.from_numpy(ids).cuda(), block, experts)
    so, eo, no = o.moe_align_block_size(ids, block, experts)
    total = int(no[0])
    assert int(n.item()) == total
    s, e = s.cpu().numpy(), e.cpu().numpy()
    assert len(s) == ids.size + experts * (block - 1)
    assert np.array_equal(s[:total], so[:total])          # stable order: identical, slot by slot
    assert (s[total:] == ids.size).all()
    assert np.array_equal(e[: total // block], eo[: total // block])
    assert (e[total // block:] == -1).all()
    # the torch statement of the same sort agrees too
    st, et, nt = D.moe_align_block_size(torch.from_numpy(ids), block, experts)
    assert int(nt[0]) == total and np.array_equal(st.numpy()[:total], s[:total])


def test_native_moe_align_skips_experts_out_of_range():
    from vllm_gguf_plugin_prism_amd import ops

    rng = np.random.default_rng(77)
    experts, block = 12, 8
    ids = rng.integers(-2, experts + 3, size=(300, 4)).astype(np.int32)   # some ids name no expert
    s, e, n = ops.moe_align_block_size(torch.from_numpy(ids).cuda(), block, experts)
    s, e, total = s.cpu().numpy(), e.cpu().numpy(), int(n.item())
    flat = ids.reshape(-1)
    pos = 0
    for ex in range(experts):
        mine = np.nonzero(flat == ex)[0]
        padded = (len(mine) + block - 1) // block * block
        assert np.array_equal(s[pos:pos + len(mine)], mine)               # ascending pair index inside the run
        assert (s[pos + len(mine):pos + padded] == flat.size).all()
        assert (e[pos // block:(pos + padded) // block] == ex).all()
        pos += padded
    assert pos == total and (s[total:] == flat.size).all() and (e[total // block:] == -1).all()


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16, torch.float32])
def test_moe_weighted_sum_matches_mul_then_sum(dt):
    from vllm_gguf_plugin_prism_amd import ops

    torch.manual_seed(3)
    t, k, n = 37, 8, 520
    y = torch.randn(t, k, n, device="cuda").to(dt)
    w = torch.softmax(torch.randn(t, k, device="cuda"), dim=1)
    out = torch.empty(t, n, device="cuda", dtype=dt)
    ops.moe_weighted_sum(y, w, out)
    ref = y.clone().mul_(w.view(t, k, 1))                # rounds every product to dt, as the reference's mul_ does
    want = ref.float().sum(dim=1).to(dt)                 # fp32 accumulation, one rounding
    # identical products; only the fp32 summation order may differ, so at most the last bit of dt moves
    assert torch.allclose(out.float(), want.float(), rtol=2 ** -7 if dt == torch.bfloat16 else 2 ** -10, atol=1e-6)
    if dt != torch.float32:  # in fp32 the summation order itself is visible in the last bit
        assert (out == want).float().mean().item() > 0.95


def test_embedding_rows_out_of_range_are_zero():
    from vllm_gguf_plugin_prism_amd import ops

    rng = np.random.default_rng(9)
    table = synth.make_weights(rng, o.Q4_K, 10, 256)
    ids = torch.tensor([0, 9, 10, -1, 3], device="cuda")
    got = ops.ggml_dequantize_rows(torch.from_numpy(table).cuda(), o.Q4_K, ids, 256, torch.float32).cpu().numpy()
    dense = o.dequantize(table, o.Q4_K, "f32").reshape(10, 256)
    assert np.array_equal(got[[0, 1, 4]], dense[[0, 9, 3]])
    assert (got[[2, 3]] == 0).all()


def test_gguf_file_to_gemv(tmp_path):
    """A packed tensor read from a GGUF file goes straight into the operators."""
    import struct

    from test_gguf_file import Writer
    from vllm_gguf_plugin_prism_amd import gguf_file

    rng = np.random.default_rng(21)
    w = synth.make_weights(rng, o.Q6_K, 48, 512)
    wr = Writer()
    wr.add_kv("general.architecture", 8, wr.s("test"))
    wr.add_tensor("blk.0.ffn_down.weight", [512, 48], o.Q6_K, w.tobytes())
    path = tmp_path / "m.gguf"
    wr.write(path)
    items = dict(gguf_file.quant_weights_iterator([str(path)]))
    qt = int(items["blk.0.ffn_down.weight_type"])
    wt = items["blk.0.ffn_down.weight"].cuda()
    x = rng.standard_normal((2, 512)).astype(np.float16)
    y = D.fused_mul_mat_gguf(torch.from_numpy(x).cuda(), wt, qt).float().cpu().numpy()
    assert o.rel_l2(y, o.mul_mat_a8(w, x, o.Q6_K, 48)) <= 1e-3


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16, torch.float32])
def test_fused_activation_equals_separate_activation(act, dt):
    """The gated activation folded into the quantisation of the second MoE GEMM sees the same dtype-rounded values a
    separate activation kernel would have written, so both routes give the same output."""
    from vllm_gguf_plugin_prism_amd import ops

    rng = np.random.default_rng(17)
    E, I, H, pairs = 4, 256, 96, 11
    w2 = torch.from_numpy(np.stack([synth.make_weights(rng, o.Q4_0, H, I) for _ in range(E)])).cuda()
    h = (torch.randn(pairs, 2 * I, device="cuda") * 2).to(dt)
    ids = torch.from_numpy(rng.integers(0, E, size=pairs).astype(np.int32)).cuda()
    fn = torch.nn.functional.silu if act == "silu" else torch.nn.functional.gelu
    sep_in = (fn(h[:, :I]) * h[:, I:]).contiguous()
    want = ops.ggml_moe_a8_vec(sep_in, w2, ids, 1, o.Q4_0, H, pairs)
    got = ops.ggml_moe_a8_vec(h, w2, ids, 1, o.Q4_0, H, pairs, activation=act)
    # torch's and the kernel's exp/erf may differ in the last bit of a few activations; that moves a quant by one step
    # at most, far below the 1e-3 contract
    assert o.rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy()) <= (2e-3 if dt == torch.bfloat16 else 5e-4)
    # grouped path, same check
    s_, e_, n_ = ops.moe_align_block_size(ids.view(pairs, 1), 32, E)
    want = ops.ggml_moe_a8(sep_in, w2, s_, e_, n_, o.Q4_0, H, 1, pairs)
    got = ops.ggml_moe_a8(h, w2, s_, e_, n_, o.Q4_0, H, 1, pairs, activation=act)
    assert o.rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy()) <= (2e-3 if dt == torch.bfloat16 else 5e-4)


def _merged_layer(rng, shards, k):
    """A padded merged tensor like quantization/linear.py:150-219 builds: shards stacked by rows, every row padded to
    the widest shard's row bytes.  shards: list of (id, ggml type, rows)."""
    parts, offsets, start = [], {}, 0
    for sid, qt, rows in shards:
        w = o.make_weights(rng, qt, rows, k)
        parts.append(w)
        offsets[sid] = (start, start + rows, w.shape[1])
        start += rows
    width = max(p.shape[1] for p in parts)
    merged = np.full((start, width), 0xA5, dtype=np.uint8)   # padding bytes that would show if a kernel read them
    for (sid, _, _), p in zip(shards, parts):
        s, e, rb = offsets[sid]
        merged[s:e, :rb] = p
    return merged, offsets, parts


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m", [1, 3, 5, 40, 300])
def test_apply_linear_mixed_type_shards_in_place(m, dt):
    """q and k in Q4_K, v in Q6_K (what Q4_K_M checkpoints hold): the reference multiplies a .contiguous() copy of every
    shard, concatenates and adds the bias (linear.py:247-262).  apply_linear must give the same bits while reading the
    shards inside the padded tensor and writing into the merged result directly, for every path (GEMV, both MMQ
    engines) the batch size selects."""
    from vllm_gguf_plugin_prism_amd import ops
    rng = np.random.default_rng(2000 + m)
    k = 1024
    shards = [("q", o.Q4_K, 512), ("k", o.Q4_K, 128), ("v", o.Q6_K, 130)]
    merged, offsets, parts = _merged_layer(rng, shards, k)
    wd = torch.from_numpy(merged).cuda()
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(dt).cuda()
    bias = torch.from_numpy(rng.standard_normal(770).astype(np.float32)).to(dt).cuda()
    types = {"q": o.Q4_K, "k": o.Q4_K, "v": o.Q6_K}
    got = D.apply_linear(x, wd, o.Q4_K, shard_ids=["q", "k", "v"], shard_offset_map=offsets, shard_weight_types=types, bias=bias)
    # the reference's sequence, with the same operators on contiguous copies
    ref = torch.cat([D.fused_mul_mat_gguf(x, torch.from_numpy(p).cuda(), qt) for (_, qt, _), p in zip(shards, parts)], dim=1)
    ref.add_(bias)
    assert got.shape == (m, 770) and got.dtype == dt
    assert torch.equal(got, ref)
    # and against the oracle, so that "the same bits" is not two equal mistakes
    xv = x.float().cpu().numpy()
    path = D.select_mul_mat_path(o.Q4_K, m, 512)
    exp = np.concatenate([o.mul_mat_a8(p, xv, qt, p.shape[0], path) for (_, qt, _), p in zip(shards, parts)], axis=1)
    exp = exp + bias.float().cpu().numpy()
    tol = {torch.float16: 2e-3, torch.bfloat16: 8e-3, torch.float32: 1e-5}[dt]
    assert o.rel_l2(got.float().cpu().numpy(), exp) <= tol


def test_apply_linear_single_type_and_plain_layers():
    rng = np.random.default_rng(2100)
    k = 512
    merged, offsets, parts = _merged_layer(rng, [(0, o.Q8_0, 96), (1, o.Q8_0, 160)], k)
    wd = torch.from_numpy(merged).cuda()
    x = torch.from_numpy(rng.standard_normal((2, k)).astype(np.float32)).to(torch.float16).cuda()
    bias = torch.from_numpy(rng.standard_normal(256).astype(np.float32)).to(torch.float16).cuda()
    one = D.apply_linear(x, wd, o.Q8_0, shard_ids=[0, 1], shard_offset_map=offsets, bias=bias)
    plain = D.apply_linear(x, wd, o.Q8_0, bias=bias)
    ref = D.fused_mul_mat_gguf(x, wd, o.Q8_0)
    ref.add_(bias)
    assert torch.equal(one, ref) and torch.equal(plain, ref)


def test_shard_operators_reject_bad_views():
    from vllm_gguf_plugin_prism_amd import ops
    rng = np.random.default_rng(2200)
    w = torch.from_numpy(o.make_weights(rng, o.Q4_K, 64, 512)).cuda()
    x = torch.randn(2, 512, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        ops.ggml_mul_mat_vec_a8(w[:, :100], x, o.Q4_K, 64)                       # rows shorter than K needs
    with pytest.raises(ValueError):
        ops.ggml_mul_mat_vec_a8(w, x, o.Q4_K, 64, out=torch.empty(2, 63, dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError):
        ops.ggml_mul_mat_a8(w, x, o.Q4_K, 64, bias=torch.zeros(64, dtype=torch.float32, device="cuda"))
    with pytest.raises(ValueError):
        ops.ggml_mul_mat_a8(w.t(), x, o.Q4_K, 64)
    # packed blocks at an odd address or rows an odd number of bytes apart cannot be GGUF data
    buf = torch.zeros(64 * 289 + 1, dtype=torch.uint8, device="cuda")
    odd_base = buf[1:1 + 64 * 288].view(64, 288)
    odd_pitch = buf[:64 * 289].view(64, 289)[:, :288]
    for bad in (odd_base, odd_pitch):
        with pytest.raises(ValueError):
            ops.ggml_mul_mat_vec_a8(bad, x, o.Q4_K, 64)
        with pytest.raises(ValueError):
            ops.ggml_mul_mat_a8(bad, x, o.Q4_K, 64)
