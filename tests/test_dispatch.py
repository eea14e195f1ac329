"""Path-selection policy above the operators, pinned by tables over (type, batch, rows).

The expected values are read off the reference's callers (quantization/linear.py:35-58,
quantization/fused_moe.py:53-112); they are written out as literals, not recomputed.
"""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as oracle
from vllm_gguf_plugin_prism_amd import dispatch as D

MUL_MAT_CASES = [
    # (type, batch, rows, expected)
    (D.Q4_K, 0, 4096, "empty"),
    (D.F16, 0, 4096, "empty"),
    (D.F16, 3, 4096, "unquantized"),
    (D.BF16, 300, 14336, "unquantized"),
    (D.F32, 1, 8, "unquantized"),
    # standard / K quants: GEMV up to 6 rows of X when W has <= 5120 rows, up to 2 above
    (D.Q4_K, 1, 4096, "mmvq"),
    (D.Q4_K, 6, 4096, "mmvq"),
    (D.Q4_K, 7, 4096, "mmq"),
    (D.Q4_K, 6, 5120, "mmvq"),
    (D.Q4_K, 2, 5121, "mmvq"),
    (D.Q4_K, 3, 5121, "mmq"),
    (D.Q4_K, 1, 14336, "mmvq"),
    (D.Q4_K, 2, 14336, "mmvq"),
    (D.Q4_K, 4, 14336, "mmq"),   # decode batch 4 on the wide projection already takes the GEMM
    (D.Q4_K, 8, 14336, "mmq"),
    (D.Q4_K, 8, 4096, "mmq"),
    (D.Q6_K, 128, 18944, "mmq"),
    (D.Q6_K, 512, 3584, "mmq"),
    (D.Q8_0, 1, 3072, "mmvq"),
    (D.Q4_0, 2048, 2048, "mmq"),
    (D.Q5_1, 6, 100, "mmvq"),
    (D.Q2_K, 7, 100, "mmq"),
    # i-quants: GEMV up to 16 rows (8 above 5120 rows of W), then dequantize + dense GEMM
    (D.IQ4_XS, 1, 5120, "mmvq"),
    (D.IQ4_XS, 16, 5120, "mmvq"),
    (D.IQ4_XS, 17, 5120, "dequant"),
    (D.IQ4_XS, 256, 5120, "dequant"),
    (D.IQ2_XXS, 8, 17408, "mmvq"),
    (D.IQ2_XXS, 9, 17408, "dequant"),
    (D.IQ2_XXS, 256, 17408, "dequant"),
    (D.IQ1_M, 16, 5120, "mmvq"),
    (D.IQ3_S, 1000, 64, "dequant"),
]


@pytest.mark.parametrize("qt,batch,rows,expected", MUL_MAT_CASES)
def test_mul_mat_path(qt, batch, rows, expected):
    assert D.select_mul_mat_path(qt, batch, rows) == expected


@pytest.mark.parametrize("qt", [4, 5, 15, 24, 28, 31, 99, -1])
def test_unknown_type_raises(qt):
    with pytest.raises(NotImplementedError):
        D.select_mul_mat_path(qt, 1, 64)
    assert D.select_mul_mat_path(qt, 0, 64) == "empty"  # the empty check comes first (linear.py:42-43)


MOE_CASES = [
    (D.Q4_0, D.Q4_0, 1, "vec"),
    (D.Q4_0, D.Q4_0, 64, "vec"),
    (D.Q4_0, D.Q4_0, 65, "grouped"),
    (D.Q4_0, D.Q4_0, 512, "grouped"),
    (D.Q4_K, D.Q6_K, 512, "grouped"),
    (D.Q4_K, D.IQ4_XS, 512, "vec"),      # one i-quant operand: no grouped kernel, per-pair GEMV at any size
    (D.IQ2_XXS, D.IQ2_XXS, 4096, "vec"),
    (D.F16, D.F16, 8, "loop"),
    (D.Q4_0, D.F16, 100, "loop"),
]


@pytest.mark.parametrize("qt,qt2,tokens,expected", MOE_CASES)
def test_moe_path(qt, qt2, tokens, expected):
    assert D.select_moe_path(qt, qt2, tokens) == expected


def test_type_sets_partition():
    assert D.MMQ_QUANT_TYPES < D.MMVQ_QUANT_TYPES
    assert not (D.UNQUANTIZED_TYPES & D.DEQUANT_TYPES)
    assert len(D.DEQUANT_TYPES) == 20
    assert D.MMVQ_QUANT_TYPES - D.MMQ_QUANT_TYPES == D.IMATRIX_QUANT_TYPES


def test_mmvq_safe_values():
    assert [D.mmvq_safe(D.Q4_K, r) for r in (1, 5120, 5121)] == [6, 6, 2]
    assert [D.mmvq_safe(D.IQ4_XS, r) for r in (1, 5120, 5121)] == [16, 16, 8]


@pytest.mark.parametrize("tokens,top_k,experts,block", [(1, 8, 64, 32), (7, 2, 4, 32), (64, 8, 64, 32), (33, 3, 5, 4),
                                                        (5, 1, 3, 8)])
def test_moe_align_block_size_contract(tokens, top_k, experts, block):
    """Every real pair appears exactly once inside a block of its own expert, padding holds the sentinel, the padded
    total is the sum of per-expert padded counts; the numpy checker's layout is reproduced exactly."""
    rng = np.random.default_rng(tokens * 131 + top_k)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    s, e, n = D.moe_align_block_size(torch.from_numpy(ids), block, experts)
    s, e, n = s.numpy(), e.numpy(), int(n[0])
    numel = ids.size
    counts = np.bincount(ids.reshape(-1), minlength=experts)
    assert n == int((((counts + block - 1) // block) * block).sum())
    assert len(s) == numel + experts * (block - 1)
    real = s[s < numel]
    assert sorted(real.tolist()) == list(range(numel))
    assert (s[n:] == numel).all()
    for pos in range(n):
        if s[pos] < numel:
            assert ids.reshape(-1)[s[pos]] == e[pos // block]
    so, eo, no = oracle.moe_align_block_size(ids, block, experts)
    assert int(no[0]) == n
    assert (so[:n] == s[:n]).all()
    assert (eo[: n // block] == e[: n // block]).all()


def test_empty_batch_returns_empty_without_touching_the_library():
    x = torch.empty(0, 64, dtype=torch.float16)
    w = torch.empty(16, 36, dtype=torch.uint8)
    y = D.fused_mul_mat_gguf(x, w, D.Q4_K)
    assert y.shape == (0, 16) and y.dtype == torch.float16


def test_unquantized_is_plain_matmul():
    x = torch.randn(3, 8)
    w = torch.randn(5, 8)
    assert torch.equal(D.fused_mul_mat_gguf(x, w, D.F32), x @ w.T)
