"""The two benchmark configurations that have no full-size test elsewhere, at their real shapes: the codebook i-quants
(IQ4_XS [5120,5120], IQ2_XXS [17408,5120], M = 1 and 256) and the 64-expert top-8 Q4_0 MoE layer (T = 1, 64, 512).
The fp64 oracle checks a sample of output rows / tokens (rows and tokens are independent of each other); properties
that do not depend on the size cover the whole output: doubling the activations doubles the result exactly, and the
a8 product agrees with the product of the unquantized activations with the dequantized weights to within the
activations' quantization error."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd import dispatch as D
from vllm_gguf_plugin_prism_amd import ops, synth

pytestmark = pytest.mark.gpu

IQ_SHAPES = [(o.IQ4_XS, 5120, 5120), (o.IQ2_XXS, 17408, 5120)]


def _row_sample(n, rng, count=96):
    return np.unique(np.concatenate([np.arange(8), np.arange(n - 8, n), rng.integers(0, n, count)]))


@pytest.mark.parametrize("qt,n,k", IQ_SHAPES)
def test_config4_iquant_gemv_full_size(qt, n, k):
    rng = np.random.default_rng(40 + qt)
    w = synth.random_blocks(rng, qt, n, k)            # raw valid blocks, d ~ U(1e-4, 1e-2)
    x = rng.standard_normal((1, k)).astype(np.float16)
    wd, xd = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
    assert D.select_mul_mat_path(qt, 1, n) == "mmvq"
    y = D.fused_mul_mat_gguf(xd, wd, qt)
    assert y.shape == (1, n) and y.dtype == torch.float16
    rows = _row_sample(n, rng)
    want = o.mul_mat_a8(w[rows], x.astype(np.float32), qt, len(rows), "mmvq")
    assert o.rel_l2(y[:, rows].float().cpu().numpy(), want) <= 1e-3
    # doubling x doubles every q8_1 scale and sum exactly, hence every fp32 result and its fp16 rounding
    y2 = D.fused_mul_mat_gguf(xd * 2, wd, qt)
    assert torch.equal(y2, y * 2)
    # whole output against the unquantized product (q8_1 rounding of x is about 0.4 % per element)
    dense = ops.ggml_dequantize(wd, qt, n, k, torch.float32)
    ref = xd.float() @ dense.T
    assert o.rel_l2(y.float().cpu().numpy(), ref.cpu().numpy()) <= 1e-2


@pytest.mark.parametrize("qt,n,k", IQ_SHAPES)
def test_config4_iquant_batch_256_full_size(qt, n, k):
    rng = np.random.default_rng(44 + qt)
    m = 256
    w = synth.random_blocks(rng, qt, n, k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    wd, xd = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
    rows = _row_sample(n, rng, 40)
    # (i) the reference's route for i-quants at this batch: dequantize, then a dense product (linear.py:50-58)
    assert D.select_mul_mat_path(qt, m, n) == "dequant"
    dense16 = ops.ggml_dequantize(wd, qt, n, k, torch.float16)
    assert np.array_equal(dense16[rows].cpu().numpy().view(np.uint16),
                          o.dequantize(w[rows], qt, "f16").reshape(len(rows), k).view(np.uint16))
    y = D.fused_mul_mat_gguf(xd, wd, qt)
    assert y.shape == (m, n) and y.dtype == torch.float16
    ref = (xd.float() @ dense16.float().T).cpu().numpy()
    assert o.rel_l2(y.float().cpu().numpy(), ref) <= 2e-3          # fp16 product with fp32 accumulation, fp16 result
    # (ii) the a8 GEMM on these formats (no counterpart in the reference, same semantics as its GEMV)
    ya = ops.ggml_mul_mat_a8(wd, xd, qt, n)
    want = o.mul_mat_a8(w[rows], x.astype(np.float32), qt, len(rows), "mmq")
    assert o.rel_l2(ya[:, rows].float().cpu().numpy(), want) <= 1e-3
    assert o.rel_l2(ya.float().cpu().numpy(), ref) <= 1e-2


@pytest.fixture(scope="module")
def moe_weights():
    rng = np.random.default_rng(5)
    E, H, I, qt = 64, 2048, 1024, o.Q4_0
    w13 = np.stack([synth.make_weights(rng, qt, 2 * I, H) for _ in range(E)])     # [64, 2048, 1152 B]
    w2 = np.stack([synth.make_weights(rng, qt, H, I) for _ in range(E)])          # [64, 2048, 576 B]
    assert w13.shape == (E, 2048, 1152) and w2.shape == (E, 2048, 576)
    return w13, w2


@pytest.mark.parametrize("tokens", [1, 64, 512])
def test_config5_moe_layer_full_size(tokens, moe_weights):
    rng = np.random.default_rng(50 + tokens)
    E, H, I, top_k, qt = 64, 2048, 1024, 8, o.Q4_0
    w13, w2 = moe_weights
    x = (rng.standard_normal((tokens, H)) * 4).astype(np.float16)   # weights ~ N(0, 0.02): keep the intermediate O(1)
    logits = rng.standard_normal((tokens, E))
    ids = np.argsort(-logits, axis=1)[:, :top_k].astype(np.int32)
    sel = np.take_along_axis(logits, ids, 1)
    tw = (np.exp(sel) / np.exp(sel).sum(1, keepdims=True)).astype(np.float32)
    assert D.select_moe_path(qt, qt, tokens) == ("grouped" if tokens > 64 else "vec")
    got = D.fused_moe_gguf(torch.from_numpy(x).cuda(), torch.from_numpy(w13).cuda(), torch.from_numpy(w2).cuda(),
                           torch.from_numpy(tw).cuda().half(), torch.from_numpy(ids).cuda(), qt, qt, "silu")
    torch.cuda.synchronize()
    assert got.shape == (tokens, H) and got.dtype == torch.float16
    assert torch.isfinite(got).all()
    # per-token definition of the layer (fused_moe.py:119-132) on a sample of tokens, in fp64 on a8 operands
    sample = np.unique(np.concatenate([[0, tokens - 1], rng.integers(0, tokens, 4)]))
    xs, ids_s, tw_s = x[sample], ids[sample], tw[sample]
    h = o.moe_a8_vec(xs.astype(np.float32), w13, ids_s.reshape(-1), top_k, qt, 2 * I, len(sample)).astype(np.float16)
    a = o.silu_and_mul(h.astype(np.float64)).astype(np.float16)
    y = o.moe_a8_vec(a.astype(np.float32), w2, ids_s.reshape(-1), 1, qt, H, len(sample) * top_k)
    y = y.astype(np.float16).astype(np.float64).reshape(len(sample), top_k, H)
    want = (y * tw_s.astype(np.float16).astype(np.float64)[:, :, None]).astype(np.float16).astype(np.float64).sum(1)
    # fp16 storage between the stages and the re-quantization of a slightly different intermediate bound the error
    assert o.rel_l2(got[sample].float().cpu().numpy(), want) <= 1e-2
