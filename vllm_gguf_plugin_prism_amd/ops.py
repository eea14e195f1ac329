"""Operator façade, drop-in for ``vllm_gguf_plugin/ops.py:181-286`` of the reference.

Same function names, positional orders, output shapes and dtypes.  Every call
lands in the hand-written gfx950 kernels of ``libgguf_hip.so`` through its C ABI;
there is no Triton or other fallback, so a ggml type a kernel does not cover
raises ``NotImplementedError`` instead of silently taking another path.

Outputs and the activation workspace are allocated with torch, and kernels are
launched on torch's current HIP stream, so calls are asynchronous and
graph-capturable like the reference's (``csrc/gguf/gguf_kernel.cu:24-29,104-118``).
"""
from __future__ import annotations

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}; need float32, float16 or bfloat16") from None


def _stream(t: torch.Tensor) -> int:
    # (the raw handle of torch's current stream on the tensor's device: a Stream object per call costs 4 us)
    return torch._C._cuda_getCurrentRawStream(t.device.index if t.device.index is not None else torch.cuda.current_device())


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()


def _on_device_of(t: torch.Tensor):
    """Context in which the tensor's device is current: nothing to do (and 3 us less to pay) when it already is."""
    idx = t.device.index
    return _NO_SWITCH if idx is None or idx == torch._C._cuda_getDevice() else torch.cuda.device(t.device)


def _check_inputs(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise ValueError("GGUF ops need tensors on the GPU")
        if not t.is_contiguous():
            raise ValueError("GGUF ops need contiguous tensors")


_ACT_CODE = {None: 0, "silu": 1, "gelu": 2}


def _act_code(name: str | None) -> int:
    try:
        return _ACT_CODE[name]
    except KeyError:
        raise ValueError(f"unsupported MoE activation {name!r}; need 'silu' or 'gelu'") from None


_ROW_BYTES: dict[int, int] = {}


def _workspace(x: torch.Tensor, rows: int, k: int) -> torch.Tensor:
    rb = _ROW_BYTES.get(k)
    if rb is None:
        rb = _ROW_BYTES[k] = _lib.lib().gguf_q8_1_row_bytes(k)
    return torch.empty(max(rows * rb, 16), dtype=torch.uint8, device=x.device)


_QUANT_SIZES: dict[int, tuple[int, int]] = {}


def quant_sizes(quant_type: int) -> tuple[int, int]:
    """(elements, bytes) of one block; stands in for ``gguf.GGML_QUANT_SIZES`` (quantization/linear.py:51)."""
    hit = _QUANT_SIZES.get(quant_type)
    if hit is not None:
        return hit
    L = _lib.lib()
    qk, bs = L.gguf_block_elems(int(quant_type)), L.gguf_block_bytes(int(quant_type))
    if qk == 0:
        raise NotImplementedError(f"Unsupported GGUF quantization type: {quant_type}")
    _QUANT_SIZES[quant_type] = (qk, bs)
    return qk, bs


def ggml_dequantize(W: torch.Tensor, quant_type: int, m: int, n: int, dtype: torch.dtype | None) -> torch.Tensor:
    """Dense ``[m, n]`` values of the packed tensor ``W`` (reference: gguf_kernel.cu:87-102)."""
    _check_inputs(W)
    out_dtype = dtype or torch.float16
    with _on_device_of(W):
        out = torch.empty((m, n), dtype=out_dtype, device=W.device)
        rc = _lib.lib().gguf_dequantize(W.data_ptr(), int(quant_type), out.data_ptr(), _code(out_dtype), m * n, _stream(W))
    _lib.check(rc, "ggml_dequantize")
    return out


def ggml_dequantize_rows(W: torch.Tensor, quant_type: int, row_ids: torch.Tensor, hidden_size: int,
                         dtype: torch.dtype | None) -> torch.Tensor:
    """Dense ``[row_ids.numel(), hidden_size]`` values of the selected rows of the packed table ``W``: the embedding
    lookup of quantization/vocal_embeds.py:90-96 (index_select, then ggml_dequantize) in one kernel."""
    _check_inputs(W, row_ids)
    out_dtype = dtype or torch.float16
    ids = row_ids.reshape(-1).to(torch.int64)
    with _on_device_of(W):
        out = torch.empty((ids.numel(), hidden_size), dtype=out_dtype, device=W.device)
        rc = _lib.lib().gguf_dequantize_rows(W.data_ptr(), int(quant_type), ids.data_ptr(), ids.numel(), W.shape[0],
                                             hidden_size, out.data_ptr(), _code(out_dtype), _stream(W))
    _lib.check(rc, "ggml_dequantize_rows")
    return out


def _shard_args(W: torch.Tensor, X: torch.Tensor, quant_type: int, row: int, out: torch.Tensor | None,
                bias: torch.Tensor | None) -> tuple[torch.Tensor, int, int]:
    """Validate one shard of a (possibly merged, padded) linear layer; returns (output, bytes between rows of W,
    elements between rows of the output).  ``W`` may be a row/column slice of a wider uint8 tensor and ``out`` a column
    slice of a wider result (quantization/linear.py:247-257 copies such slices with ``.contiguous()`` and concatenates
    the results; here the kernels address them in place)."""
    for t in (W, X) + ((out,) if out is not None else ()) + ((bias,) if bias is not None else ()):
        if not t.is_cuda:
            raise ValueError("GGUF ops need tensors on the GPU")
    if not X.is_contiguous() or X.dim() != 2:
        raise ValueError("GGUF ops need a contiguous 2-D activation tensor")
    qk, bs = quant_sizes(quant_type)
    vecs, col = X.shape
    if col % qk:
        raise ValueError(f"K = {col} is not a multiple of the block size {qk}")
    if W.dim() != 2 or W.dtype != torch.uint8 or (W.shape[1] > 1 and W.stride(1) != 1):
        raise ValueError("the packed weights must be a 2-D uint8 tensor with contiguous rows")
    if W.shape[0] < row or W.shape[1] < col // qk * bs:
        raise ValueError("the packed weights are smaller than [row, K / block * block_bytes]")
    w_pitch = W.stride(0) if W.shape[0] > 1 else col // qk * bs
    if out is None:
        out = torch.empty((vecs, row), dtype=X.dtype, device=W.device)
    elif out.shape != (vecs, row) or out.dtype != X.dtype or (row > 1 and out.stride(1) != 1):
        raise ValueError("out must be [X.shape[0], row] of X's dtype with contiguous rows")
    ldy = out.stride(0) if vecs > 1 else row
    if bias is not None and (bias.shape != (row,) or bias.dtype != X.dtype or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous [row] tensor of X's dtype")
    return out, w_pitch, ldy


def ggml_mul_mat_vec_a8(W: torch.Tensor, X: torch.Tensor, quant_type: int, row: int, *, out: torch.Tensor | None = None,
                        bias: torch.Tensor | None = None) -> torch.Tensor:
    """Decode GEMV ``q8_1(X) @ W^T`` -> ``[X.shape[0], row]`` (reference: gguf_kernel.cu:104-218).

    ``W`` may be a slice of a wider tensor (rows any pitch apart), ``out`` a column slice of a wider result, and
    ``bias`` is added the way ``out.add_(bias)`` would (quantization/linear.py:243-262)."""
    out, w_pitch, ldy = _shard_args(W, X, quant_type, row, out, bias)
    vecs, col = X.shape
    with _on_device_of(X):
        ws = _workspace(X, vecs, col)
        rc = _lib.lib().gguf_mmvq_linear(W.data_ptr(), w_pitch, X.data_ptr(), _code(X.dtype), ws.data_ptr(), out.data_ptr(), ldy,
                                         bias.data_ptr() if bias is not None else None, int(quant_type), row, col, vecs,
                                         _stream(X))
    _lib.check(rc, "ggml_mul_mat_vec_a8")
    return out


MMQ_ENGINES = {"auto": 0, "int8": 1, "half": 2}


def ggml_mul_mat_a8(W: torch.Tensor, X: torch.Tensor, quant_type: int, row: int, *, engine: str = "auto",
                    out: torch.Tensor | None = None, bias: torch.Tensor | None = None) -> torch.Tensor:
    """Prefill GEMM ``q8_1(X) @ W^T`` on MFMA (reference: gguf_kernel.cu:220-290).

    ``engine``: ``"int8"`` keeps the reference's integer arithmetic (exact int8 dot products per block on int8 MFMA,
    block scales in fp32) and is what ``"auto"`` means; ``"half"`` is opt-in and multiplies the dequantized operands
    on half-precision MFMA (faster, about 2e-4 relative deviation from the integer result, half and bfloat16 results
    only).  ``out`` / ``bias`` / sliced ``W``: as for :func:`ggml_mul_mat_vec_a8`."""
    out, w_pitch, ldy = _shard_args(W, X, quant_type, row, out, bias)
    vecs, col = X.shape
    with _on_device_of(X):
        # (only the half engine pays for the half-precision copy of the rows)
        nbytes = max(_lib.lib().gguf_mmq_workspace_bytes_engine(vecs, row, col, MMQ_ENGINES[engine]), 16)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=X.device)
        rc = _lib.lib().gguf_mmq_linear(W.data_ptr(), w_pitch, X.data_ptr(), _code(X.dtype), ws.data_ptr(), out.data_ptr(), ldy,
                                        bias.data_ptr() if bias is not None else None, int(quant_type), row, col, vecs,
                                        MMQ_ENGINES[engine], nbytes, _stream(X))
    _lib.check(rc, "ggml_mul_mat_a8")
    return out


DEQUANT_GEMM_TYPES = frozenset({2, 3, 6, 7, 8, 10, 11, 12, 13, 14, 16, 23})


def ggml_dequant_gemm(W: torch.Tensor, X: torch.Tensor, quant_type: int, row: int) -> torch.Tensor:
    """``X @ dequant(W)^T`` -> ``[X.shape[0], row]`` in one kernel, activations not quantized: the reference's
    ``ggml_dequantize`` + ``x @ weight.T`` fallback (quantization/linear.py:50-58) without the dense copy of W.
    fp16 / bf16 only; raises ``NotImplementedError`` for types outside ``DEQUANT_GEMM_TYPES``."""
    _check_inputs(W, X)
    vecs, col = X.shape
    with _on_device_of(X):
        out = torch.empty((vecs, row), dtype=X.dtype, device=W.device)
        nbytes = max(_lib.lib().gguf_mmq_workspace_bytes_engine(vecs, row, col, MMQ_ENGINES["half"]), 16)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=X.device)
        rc = _lib.lib().gguf_dequant_gemm(W.data_ptr(), X.data_ptr(), _code(X.dtype), ws.data_ptr(), out.data_ptr(),
                                          int(quant_type), row, col, vecs, nbytes, _stream(X))
    _lib.check(rc, "ggml_dequant_gemm")
    return out


MOE_GROUPED_MAX_EXPERTS = 256


def ggml_moe_a8(
    X: torch.Tensor,
    W: torch.Tensor,
    sorted_token_ids: torch.Tensor,
    expert_ids: torch.Tensor,
    num_tokens_post_padded: torch.Tensor,
    quant_type: int,
    row: int,
    top_k: int,
    tokens: int,
    *,
    activation: str | None = None,
    block_size: int | None = None,
) -> torch.Tensor:
    """Grouped MoE GEMM -> ``[tokens * top_k, row]`` (reference: gguf_kernel.cu:292-393).

    ``activation`` ("silu" / "gelu") is an extension: X then holds ``[gate | up]`` rows of twice the inner dimension and
    the gated activation is applied while the rows are quantized, instead of by a separate kernel beforehand.
    ``block_size`` is the block the routing was sorted with when it is not ``ggml_moe_get_block_size(quant_type)``:
    :func:`moe_block_size_for` picks blocks of 16 slots for a layer whose experts see few pairs each."""
    _check_inputs(X, W, sorted_token_ids, expert_ids, num_tokens_post_padded)
    for t in (sorted_token_ids, expert_ids, num_tokens_post_padded):
        if t.dtype != torch.int32:
            raise ValueError("MoE index tensors must be int32")
    if W.dim() == 3 and W.shape[0] > MOE_GROUPED_MAX_EXPERTS:
        # the kernel keeps the reference's guard and leaves the rows of experts past 255 zero (moe.cuh:33): refuse rather
        # than return a result with holes; ggml_moe_a8_vec has no such limit
        raise NotImplementedError(f"ggml_moe_a8 takes at most {MOE_GROUPED_MAX_EXPERTS} experts, got {W.shape[0]}")
    act = _act_code(activation)
    col = X.shape[1] // 2 if act else X.shape[1]
    with _on_device_of(X):
        out = torch.empty((tokens * top_k, row), dtype=X.dtype, device=W.device)
        ws = _workspace(X, tokens, col)
        rc = _lib.lib().gguf_moe_mmq_block(
            X.data_ptr(), _code(X.dtype), ws.data_ptr(), W.data_ptr(), W.stride(0) * W.element_size(),
            sorted_token_ids.data_ptr(), expert_ids.data_ptr(), num_tokens_post_padded.data_ptr(),
            sorted_token_ids.shape[0], out.data_ptr(), int(quant_type), row, col, top_k, tokens, act,
            int(block_size) if block_size else ggml_moe_get_block_size(quant_type), W.shape[0] if W.dim() == 3 else 0, _stream(X))
    _lib.check(rc, "ggml_moe_a8")
    return out


def moe_block_size_for(quant_type: int, pairs: int, num_experts: int) -> int:
    """Block size to sort the routing with for :func:`ggml_moe_a8` (``block_size=``): 16 while an expert sees 12 pairs or
    fewer on average and the format has 16-slot tiles, else ``ggml_moe_get_block_size(quant_type)``; 0 for unknown types."""
    return int(_lib.lib().gguf_moe_block_size_for(int(quant_type), int(pairs), int(num_experts)))


def ggml_moe_a8_vec(
    X: torch.Tensor,
    W: torch.Tensor,
    topk_ids: torch.Tensor,
    top_k: int,
    quant_type: int,
    row: int,
    tokens: int,
    *,
    activation: str | None = None,
) -> torch.Tensor:
    """Per-pair MoE GEMV -> ``[tokens * top_k, row]`` (reference: gguf_kernel.cu:395-530).  ``activation``: see
    :func:`ggml_moe_a8`."""
    _check_inputs(X, W, topk_ids)
    if topk_ids.dtype != torch.int32:
        raise ValueError("topk_ids must be int32")
    act = _act_code(activation)
    col = X.shape[1] // 2 if act else X.shape[1]
    L = _lib.lib()
    with _on_device_of(X):
        out = torch.empty((tokens * top_k, row), dtype=X.dtype, device=W.device)
        nbytes = max(16, L.gguf_moe_vec_workspace_bytes(tokens, top_k, col, W.shape[0]))  # quantized rows + routing sort
        ws = torch.empty(nbytes, dtype=torch.uint8, device=X.device)
        rc = L.gguf_moe_vec_act(X.data_ptr(), _code(X.dtype), ws.data_ptr(), W.data_ptr(), topk_ids.data_ptr(),
                                out.data_ptr(), int(quant_type), row, col, top_k, tokens, act, W.shape[0], nbytes, _stream(X))
    _lib.check(rc, "ggml_moe_a8_vec")
    return out


def ggml_moe_get_block_size(quant_type: int) -> int:
    """Token-tile size for ``moe_align_block_size`` (reference: gguf_kernel.cu:532-566)."""
    return int(_lib.lib().gguf_moe_block_size(int(quant_type)))


def moe_sum(input: torch.Tensor, output: torch.Tensor) -> None:
    """``output[t, :] = sum_k input[t, k, :]`` (the reference forwards to vLLM's ``_moe_C.moe_sum``, ops.py:285-286)."""
    torch.sum(input, dim=1, out=output)


def quantize_q8_1(X: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The q8_1 activation quantizer on its own (reference: gguf_kernel.cu:32-85).

    Returns ``(q, ds)``: int8 ``[M, Kp]`` quants and float32 ``[M, Kp/32, 2]`` (scale, sum) pairs holding the
    half-rounded values, with ``Kp`` = K rounded up to 512.
    """
    _check_inputs(X)
    m, k = X.shape
    kp = (k + 511) // 512 * 512
    with _on_device_of(X):
        ws = _workspace(X, m, k)
        q = torch.empty((m, kp), dtype=torch.int8, device=X.device)
        ds = torch.empty((m, kp // 32, 2), dtype=torch.float32, device=X.device)
        L = _lib.lib()
        _lib.check(L.gguf_quantize_q8_1(X.data_ptr(), _code(X.dtype), ws.data_ptr(), m, k, _stream(X)), "quantize_q8_1")
        _lib.check(L.gguf_q8_1_unpack(ws.data_ptr(), q.data_ptr(), ds.data_ptr(), m, k, _stream(X)), "q8_1_unpack")
    return q, ds


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """``(sorted_token_ids, expert_ids, num_tokens_post_padded)`` for the grouped kernel, in one launch.

    Same contract as vLLM's ``moe_align_block_size`` as the reference calls it (quantization/fused_moe.py:62-66):
    int32 outputs, padding slots hold ``topk_ids.numel()``, the order inside an expert's run is ascending pair index."""
    _check_inputs(topk_ids)
    ids = topk_ids.reshape(-1)
    if ids.dtype != torch.int32:
        ids = ids.to(torch.int32)
    numel = ids.numel()
    capacity = numel + num_experts * (block_size - 1)
    nblocks = (capacity + block_size - 1) // block_size
    with _on_device_of(ids):
        sorted_ids = torch.empty(capacity, dtype=torch.int32, device=ids.device)
        expert_ids = torch.empty(nblocks, dtype=torch.int32, device=ids.device)
        post = torch.empty(1, dtype=torch.int32, device=ids.device)
        rc = _lib.lib().gguf_moe_align_block_size(ids.data_ptr(), numel, int(num_experts), int(block_size),
                                                  sorted_ids.data_ptr(), capacity, expert_ids.data_ptr(), nblocks,
                                                  post.data_ptr(), _stream(ids))
    _lib.check(rc, "moe_align_block_size")
    return sorted_ids, expert_ids, post


def moe_vec_layer_takes(quant_type: int, quant_type2: int, hidden: int, inner: int, out_features: int, top_k: int, tokens: int,
                        num_experts: int) -> bool:
    """Whether :func:`moe_vec_layer` serves a layer of this shape: a few tokens whose experts are not shared (two
    launches) or experts shared by at most 16 pairs each on average (four launches on the tile kernels)."""
    return bool(_lib.lib().gguf_moe_vec_layer_takes(int(quant_type), int(quant_type2), int(hidden), int(inner), int(out_features),
                                                    int(top_k), int(tokens), int(num_experts)))


def moe_mmq_layer_takes(quant_type: int, quant_type2: int, hidden: int, inner: int, out_features: int, top_k: int, tokens: int,
                        num_experts: int) -> bool:
    """Whether :func:`moe_mmq_layer` serves a layer of this shape: two tile formats (the twelve of ``ggml_moe_a8``), at
    most 256 experts, an inner size in whole blocks."""
    return bool(_lib.lib().gguf_moe_mmq_layer_takes(int(quant_type), int(quant_type2), int(hidden), int(inner), int(out_features),
                                                    int(top_k), int(tokens), int(num_experts)))


def moe_mmq_layer(X, W13, W2, topk_weights, topk_ids, quant_type: int, quant_type2: int, activation: str,
                  output: torch.Tensor | None = None) -> torch.Tensor:
    """The reference's MoE layer on its grouped operator (quantization/fused_moe.py:62-95) in one call of four launches:
    one routing sort (on blocks of 16 slots while experts see at most 16 pairs each, else 32) for both ``ggml_moe_a8`` GEMMs, ``act`` and the q8_1 quantisation of its
    result in the first one's epilogue, ``mul_`` by the routing weights and ``moe_sum`` -> ``[tokens, W2.shape[1]]``.
    Same roundings as those steps run one by one; raises ``ValueError`` for shapes :func:`moe_mmq_layer_takes` declines."""
    return _moe_layer("gguf_moe_mmq_layer", X, W13, W2, topk_weights, topk_ids, quant_type, quant_type2, activation, output)


def moe_vec_layer(
    X: torch.Tensor,
    W13: torch.Tensor,
    W2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    quant_type: int,
    quant_type2: int,
    activation: str,
    output: torch.Tensor | None = None,
) -> torch.Tensor:
    """The reference's MoE layer on its per-pair operators (quantization/fused_moe.py:98-111) in one call:
    ``ggml_moe_a8_vec`` with ``act`` and the q8_1 quantisation of its result in the epilogue, then the second
    ``ggml_moe_a8_vec`` with ``mul_`` by the routing weights and ``moe_sum`` -> ``[tokens, W2.shape[1]]`` (two launches
    where experts are not shared, four on the tile kernels where a few pairs share each).  Same roundings as those steps
    run one by one; raises ``ValueError`` for shapes :func:`moe_vec_layer_takes` declines."""
    return _moe_layer("gguf_moe_vec_layer", X, W13, W2, topk_weights, topk_ids, quant_type, quant_type2, activation, output)


def _moe_layer(entry, X, W13, W2, topk_weights, topk_ids, quant_type, quant_type2, activation, output):
    _check_inputs(X, W13, W2, topk_ids)
    if topk_ids.dtype != torch.int32:
        raise ValueError("topk_ids must be int32")
    act = _act_code(activation)
    if not act:
        raise ValueError("the layer entry points need an activation")
    tokens, top_k = topk_ids.shape
    hidden, inner, n_out = X.shape[1], W13.shape[1] // 2, W2.shape[1]
    w = topk_weights.reshape(tokens, top_k)
    if w.dtype != torch.float32 or not w.is_contiguous():
        w = w.to(torch.float32).contiguous()
    L = _lib.lib()
    with _on_device_of(X):
        out = output if output is not None else torch.empty((tokens, n_out), dtype=X.dtype, device=W2.device)
        if entry == "gguf_moe_mmq_layer":
            nbytes = L.gguf_moe_mmq_layer_workspace_bytes(int(quant_type), int(quant_type2), tokens, top_k, hidden, inner, n_out, W13.shape[0],
                                                          _code(X.dtype))
        else:
            nbytes = L.gguf_moe_vec_layer_workspace_bytes(tokens, top_k, hidden, inner, n_out, W13.shape[0], _code(X.dtype))
        nbytes = max(16, nbytes)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=X.device)
        rc = getattr(L, entry)(X.data_ptr(), _code(X.dtype), W13.data_ptr(), int(quant_type), W2.data_ptr(), int(quant_type2),
                               topk_ids.data_ptr(), w.data_ptr(), ws.data_ptr(), nbytes, out.data_ptr(), hidden, inner, n_out, top_k,
                               tokens, act, W13.shape[0], _stream(X))
    _lib.check(rc, entry[len("gguf_"):])
    return out


def moe_weighted_sum(expert_out: torch.Tensor, topk_weights: torch.Tensor, output: torch.Tensor) -> None:
    """``output[t] = sum_k expert_out[t, k] * topk_weights[t, k]``: the ``mul_`` by the routing weights and the
    ``moe_sum`` that end the reference's MoE layer (quantization/fused_moe.py:87-95), fused."""
    tokens, top_k, n = expert_out.shape
    _check_inputs(expert_out, output)
    w = topk_weights.reshape(tokens, top_k).to(torch.float32).contiguous()
    with _on_device_of(expert_out):
        rc = _lib.lib().gguf_moe_weighted_sum(expert_out.data_ptr(), w.data_ptr(), output.data_ptr(), _code(expert_out.dtype),
                                              tokens, top_k, n, _stream(expert_out))
    _lib.check(rc, "moe_weighted_sum")
