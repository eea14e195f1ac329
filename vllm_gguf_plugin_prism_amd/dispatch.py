"""Path selection above the operators: which kernel a (type, batch, rows) call takes.

Restates the policy of the reference's callers so a maintainer can see that the
drop-in operators are reached with the same arguments:

* dense layers   ``_fused_mul_mat_gguf``  (vllm_gguf_plugin/quantization/linear.py:35-58)
* MoE layers     ``_fused_moe_gguf``      (vllm_gguf_plugin/quantization/fused_moe.py:34-133)
* embeddings     ``_apply_gguf_embedding`` (vllm_gguf_plugin/quantization/vocal_embeds.py:79-98)

The pure functions :func:`select_mul_mat_path` and :func:`select_moe_path` take
only integers, import nothing heavy and are what the table-driven tests pin; the
tensor functions below them run the selected path through :mod:`.ops`.
"""
from __future__ import annotations

# ggml type ids (vllm_gguf_plugin/quantization/utils.py:46-78; gguf.GGMLQuantizationType)
F32, F16, BF16 = 0, 1, 30
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 = 2, 3, 6, 7, 8, 9
Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 10, 11, 12, 13, 14
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ4_NL, IQ3_S, IQ2_S, IQ4_XS, IQ1_M = 16, 17, 18, 19, 20, 21, 22, 23, 29

UNQUANTIZED_TYPES = frozenset({F32, F16, BF16})
STANDARD_QUANT_TYPES = frozenset({Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1})
KQUANT_TYPES = frozenset({Q2_K, Q3_K, Q4_K, Q5_K, Q6_K})
IMATRIX_QUANT_TYPES = frozenset({IQ1_M, IQ1_S, IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S, IQ4_XS, IQ4_NL})
DEQUANT_TYPES = STANDARD_QUANT_TYPES | KQUANT_TYPES | IMATRIX_QUANT_TYPES
MMVQ_QUANT_TYPES = DEQUANT_TYPES
MMQ_QUANT_TYPES = STANDARD_QUANT_TYPES | KQUANT_TYPES

MOE_VEC_MAX_TOKENS = 64  # grouped kernel only above this many tokens (fused_moe.py:57)


def mmvq_safe(weight_type: int, rows: int) -> int:
    """Largest batch that still takes the GEMV path (linear.py:38-41)."""
    if weight_type in IMATRIX_QUANT_TYPES:
        return 8 if rows > 5120 else 16
    return 2 if rows > 5120 else 6


def select_mul_mat_path(weight_type: int, batch: int, rows: int) -> str:
    """One of ``"empty" | "unquantized" | "mmvq" | "mmq" | "dequant"``; unknown types raise as the reference does."""
    if batch == 0:
        return "empty"
    if weight_type in UNQUANTIZED_TYPES:
        return "unquantized"
    if batch <= mmvq_safe(weight_type, rows) and weight_type in MMVQ_QUANT_TYPES:
        return "mmvq"
    if weight_type in MMQ_QUANT_TYPES:
        return "mmq"
    if weight_type in DEQUANT_TYPES:
        return "dequant"
    raise NotImplementedError(f"Unsupported GGUF quantization type: {weight_type}")


def select_moe_path(weight_type: int, weight_type2: int, tokens: int) -> str:
    """One of ``"grouped" | "vec" | "loop"`` (fused_moe.py:53-57,99,112)."""
    if weight_type2 in MMQ_QUANT_TYPES and weight_type in MMQ_QUANT_TYPES and tokens > MOE_VEC_MAX_TOKENS:
        return "grouped"
    if weight_type2 in MMVQ_QUANT_TYPES and weight_type in MMVQ_QUANT_TYPES:
        return "vec"
    return "loop"


# ---------------------------------------------------------------------------------------- tensor level


def fused_mul_mat_gguf(x, weight, weight_type: int, *, out=None, bias=None):
    """``x @ dequant(weight).T`` through the path the reference would pick (linear.py:35-58).

    ``weight`` may be a slice ``merged[start:end, :row_bytes]`` of a padded merged tensor, ``out`` a column slice of the
    merged result and ``bias`` the matching slice of the layer bias: the a8 kernels address all three in place."""
    import torch

    from . import ops

    rows = weight.shape[0]
    path = select_mul_mat_path(int(weight_type), x.shape[0], rows)
    if path == "mmvq":
        return ops.ggml_mul_mat_vec_a8(weight, x, weight_type, rows, out=out, bias=bias)
    if path == "mmq":
        return ops.ggml_mul_mat_a8(weight, x, weight_type, rows, out=out, bias=bias)
    if path == "empty":
        y = torch.empty(x.shape[0], rows, dtype=x.dtype, device=x.device)
    elif path == "unquantized":
        y = x @ weight.T
    else:
        # ops.ggml_dequant_gemm forms the same product without the dense copy of the weights; measured on MI355X it is
        # faster than the two steps below only for few tokens (IQ4_XS [5120,5120]: 40 vs 68 us at M=256, 213 vs 116 us
        # at M=2048, where the library GEMM runs near 900 TFLOP/s), so the reference's two steps stay the default here.
        block_size, type_size = ops.quant_sizes(weight_type)
        packed = weight if weight.is_contiguous() else weight.contiguous()
        dense = ops.ggml_dequantize(packed, weight_type, rows, packed.shape[1] // type_size * block_size, x.dtype)
        y = x @ dense.T
    if bias is not None:
        y.add_(bias)
    if out is not None:
        out.copy_(y)
        return out
    return y


def apply_linear(x, weight, weight_type: int, *, shard_ids=(), shard_offset_map=None, shard_weight_types=None, bias=None):
    """The forward pass of a GGUF linear layer (quantization/linear.py:221-262).

    ``weight`` is the layer's packed tensor.  For a merged layer (q/k/v, gate/up) ``shard_ids`` lists the shards in
    output order, ``shard_offset_map[id] = (start_row, end_row, row_bytes)`` locates each one in the padded tensor and
    ``shard_weight_types[id]`` gives its ggml type (default ``weight_type``).  Shards of one type are multiplied in one
    call, as in the reference.  Shards of different types are multiplied one by one, but where the reference copies
    every shard out of the padded tensor on every call and concatenates the results, each call here reads its rows in
    place and writes its columns of the merged result, bias included."""
    import torch

    shard_ids = list(shard_ids)
    if not shard_ids:
        return fused_mul_mat_gguf(x, weight, weight_type, bias=bias)
    shard_ids = ["q", "k", "v"] if "q" in shard_ids else shard_ids
    types = [int((shard_weight_types or {}).get(i, weight_type)) for i in shard_ids]
    if len(set(types)) == 1:
        return fused_mul_mat_gguf(x, weight, types[0], bias=bias)
    widths = [shard_offset_map[i][1] - shard_offset_map[i][0] for i in shard_ids]
    out = torch.empty(x.shape[0], sum(widths), dtype=x.dtype, device=x.device)
    col = 0
    for i, t, w in zip(shard_ids, types, widths):
        start, end, row_bytes = shard_offset_map[i]
        fused_mul_mat_gguf(x, weight[start:end, :row_bytes], t, out=out[:, col:col + w],
                           bias=None if bias is None else bias[col:col + w])
        col += w
    return out


def _activation(name: str, inp):
    """Gated activation ``act(inp[..., :d]) * inp[..., d:]``: what vLLM's apply_moe_activation computes for the two
    activations GGUF MoE models use (fused_moe.py:44-51)."""
    import torch

    d = inp.shape[-1] // 2
    gate, up = inp[..., :d], inp[..., d:]
    if name == "silu":
        return torch.nn.functional.silu(gate) * up
    if name == "gelu":
        return torch.nn.functional.gelu(gate) * up
    raise ValueError(f"unsupported MoE activation {name!r}")


def moe_align_block_size(topk_ids, block_size: int, num_experts: int):
    """Torch statement of the routing sort (device-agnostic; the GPU path uses ``ops.moe_align_block_size``).

    Sort (token, choice) pairs by expert and pad every expert's run to a multiple of ``block_size``.

    Returns ``(sorted_token_ids, expert_ids, num_tokens_post_padded)`` with the meaning ``moe.cuh:20-45`` gives them:
    entries of ``sorted_token_ids`` are flat pair indices ``token * top_k + choice``, padding entries hold
    ``topk_ids.numel()``; ``expert_ids[b]`` is the expert of the b-th block.  Any order inside an expert's run is valid
    for the kernel; this one is stable by pair index."""
    import torch

    flat = topk_ids.reshape(-1).to(torch.int64)
    numel = flat.numel()
    counts = torch.bincount(flat, minlength=num_experts)
    padded = (counts + block_size - 1) // block_size * block_size
    starts = torch.cumsum(padded, 0) - padded
    total = int(padded.sum().item())
    order = torch.argsort(flat, stable=True)
    sorted_experts = flat[order]
    first = torch.cumsum(counts, 0) - counts
    rank = torch.arange(numel, device=flat.device) - first[sorted_experts]
    capacity = numel + num_experts * (block_size - 1)
    sorted_ids = torch.full((capacity,), numel, dtype=torch.int32, device=flat.device)
    sorted_ids[starts[sorted_experts] + rank] = order.to(torch.int32)
    nblocks = (capacity + block_size - 1) // block_size
    block_starts = torch.arange(nblocks, device=flat.device) * block_size
    ends = torch.cumsum(padded, 0)
    expert_ids = torch.searchsorted(ends, block_starts, right=True).clamp_(max=num_experts - 1).to(torch.int32)
    return sorted_ids, expert_ids, torch.tensor([total], dtype=torch.int32, device=flat.device)


def fused_moe_gguf(x, w1, w2, topk_weights, topk_ids, weight_type: int, weight_type2: int, activation: str = "silu"):
    """Two-stage GGUF MoE layer (fused_moe.py:34-133): gate/up GEMM, gated activation, down GEMM, weighted sum."""
    import torch

    from . import ops

    tokens = x.shape[0]
    top_k = topk_ids.shape[1]
    out_hidden = torch.empty_like(x)
    path = select_moe_path(int(weight_type), int(weight_type2), tokens)
    if path == "grouped" and w1.shape[0] > ops.MOE_GROUPED_MAX_EXPERTS:
        # The reference's grouped kernel drops expert ids above 255 without a word (moe.cuh:33) and the one here keeps
        # that guard; the per-pair operator computes every expert, so a layer with more experts takes it at any batch.
        path = "vec"
    topk_ids = topk_ids.to(torch.int32).contiguous()
    if path == "grouped":
        experts, rows, _ = w1.shape
        if activation in ("silu", "gelu") and w2.shape[0] == experts and ops.moe_mmq_layer_takes(
                weight_type, weight_type2, x.shape[1], rows // 2, w2.shape[1], top_k, tokens, experts):
            # the layer in one call of four launches (one sort for both GEMMs, the activation and the quantisation of its
            # result in the first one's epilogue): on 16-slot tiles while experts see at most 16 pairs each, else on 32
            return ops.moe_mmq_layer(x, w1, w2, topk_weights, topk_ids, weight_type, weight_type2, activation, out_hidden)
        # the reference sorts with ggml_moe_get_block_size(type); here a layer whose experts see few pairs each (65 .. 128
        # tokens of a 64-expert top-8 layer) sorts with blocks of 16 slots where both formats have such tiles, so that the
        # tiles are not mostly padding
        block = min(ops.moe_block_size_for(weight_type, tokens * top_k, experts), ops.moe_block_size_for(weight_type2, tokens * top_k, experts))
        if block != 16:
            block = ops.ggml_moe_get_block_size(weight_type)
        sorted_ids, expert_ids, post_padded = ops.moe_align_block_size(topk_ids, block, experts)
        out = ops.ggml_moe_a8(x, w1, sorted_ids, expert_ids, post_padded, weight_type, rows, top_k, tokens, block_size=block)
        # act() of the reference is applied inside the second call, while its rows are quantized
        out = ops.ggml_moe_a8(out, w2, sorted_ids, expert_ids, post_padded, weight_type2, w2.shape[1], 1, tokens * top_k,
                              activation=activation, block_size=block)
    elif path == "vec":
        rows = w1.shape[1]
        if activation in ("silu", "gelu") and w1.shape[0] == w2.shape[0] and ops.moe_vec_layer_takes(
                weight_type, weight_type2, x.shape[1], rows // 2, w2.shape[1], top_k, tokens, w1.shape[0]):
            # the layer in one call: two launches where nothing is shared between pairs (the activation in the first GEMV's
            # epilogue, the routing weights and the sum over the top-k axis in the second's), four on the tile kernels where
            # a few pairs share each expert (one routing sort, no separate activation-and-quantize launch)
            return ops.moe_vec_layer(x, w1, w2, topk_weights, topk_ids, weight_type, weight_type2, activation, out_hidden)
        out = ops.ggml_moe_a8_vec(x, w1, topk_ids, top_k, weight_type, rows, tokens)
        out = ops.ggml_moe_a8_vec(out, w2, topk_ids, 1, weight_type2, w2.shape[1], tokens * top_k, activation=activation)
    else:
        for tok in range(tokens):
            inp = x[tok : tok + 1]
            acc = None
            for ww, ii in zip(topk_weights[tok], topk_ids[tok]):
                h = _activation(activation, fused_mul_mat_gguf(inp, w1[ii], weight_type)).contiguous()
                cur = fused_mul_mat_gguf(h, w2[ii], weight_type2).mul_(ww)
                acc = cur if acc is None else acc.add_(cur)
            out_hidden[tok] = acc
        return out_hidden
    ops.moe_weighted_sum(out.reshape(tokens, top_k, w2.shape[1]), topk_weights, out_hidden)  # mul_ by weights + moe_sum
    return out_hidden


def apply_gguf_embedding(x, weight, weight_type: int, hidden_size: int, dtype=None):
    """Embedding lookup from a packed table (vocal_embeds.py:79-98); the reference gathers the packed rows with
    index_select and dequantizes the copy, here one kernel reads the rows in place."""
    import torch

    from . import ops

    if weight_type in UNQUANTIZED_TYPES:
        return torch.embedding(weight, x)
    if weight_type in DEQUANT_TYPES:
        block_size, type_size = ops.quant_sizes(weight_type)
        flat = x.flatten()
        assert hidden_size == weight.shape[1] // type_size * block_size
        dense = ops.ggml_dequantize_rows(weight, weight_type, flat, hidden_size, dtype)  # gather + dequantize, one kernel
        return dense.view(*x.shape, hidden_size)
    raise NotImplementedError(f"Unsupported GGUF quantization type: {weight_type}")
