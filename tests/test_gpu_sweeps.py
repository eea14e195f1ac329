"""Seeded sweeps over shapes, formats, row counts and dtypes that the hand-picked cases of the other files do not name:
every draw is one call of an operator against the oracle at the tolerance of its result dtype (dequantize: bit for
bit).  The draws are fixed by the seeds, so a failure names a reproducible case."""
import numpy as np
import pytest
import torch

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd import dispatch as D
from vllm_gguf_plugin_prism_amd import synth

pytestmark = pytest.mark.gpu

ALL = sorted(t for t in o.QUANT_SIZES if t in o.TYPE_NAMES)
MMQ_TYPES = [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS]
TORCH_DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def _ops():
    from vllm_gguf_plugin_prism_amd import ops
    return ops


@pytest.mark.parametrize("seed", [1, 2])
def test_dequantize_sweep_bit_exact(seed):
    """150 draws per seed: any of the 19 formats, 1 to 257 rows, 1 to 150 blocks (24 super-blocks) per row, raw random
    block bytes (seven in ten) or quantized N(0, 0.02) weights, all three output dtypes."""
    ops = _ops()
    rng = np.random.default_rng(9100 + seed)
    for case in range(150):
        qt = int(rng.choice(ALL))
        qk = o.QUANT_SIZES[qt][0]
        n = int(rng.choice([1, 2, 3, 7, 16, 33, 100, 257]))
        k = qk * int(rng.integers(1, (24 if qk == 256 else 150) + 1))
        dt = str(rng.choice(["f32", "f16", "bf16"]))
        w = o.random_blocks(rng, qt, n, k) if rng.random() < 0.7 else o.make_weights(rng, qt, n, k)
        out = ops.ggml_dequantize(torch.from_numpy(w).cuda(), qt, n, k, TORCH_DT[dt])
        exp = o.dequantize(w, qt, dt, "ref")
        got = out.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1) if dt == "bf16" else out.cpu().numpy().reshape(-1)
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (case, o.TYPE_NAMES[qt], n, k, dt)


@pytest.mark.parametrize("seed", [1, 2])
def test_dense_operators_sweep(seed):
    """150 draws per seed of ggml_mul_mat_vec_a8 (19 formats, 1 to 33 rows of X) or ggml_mul_mat_a8 (its 12 formats and
    two extensions, 1 to 300 rows): 1 to 1100 rows of W, K any whole number of blocks up to 6400 (10240 for 256-value
    blocks), results in fp32 / fp16 / bf16 at 1e-5 / 1e-3 / 4e-3 of the a8 oracle (four times that where fewer than 64
    results leave no averaging over cancellations)."""
    ops = _ops()
    rng = np.random.default_rng(9200 + seed)
    for case in range(150):
        op = str(rng.choice(["mmvq", "mmq"]))
        qt = int(rng.choice(ALL if op == "mmvq" else MMQ_TYPES))
        qk = o.QUANT_SIZES[qt][0]
        n = int(rng.choice([1, 2, 17, 63, 64, 65, 130, 257, 500, 1100]))
        k = qk * int(rng.integers(1, (40 if qk == 256 else 200) + 1))
        m = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 100, 128, 129, 300] if op == "mmq" else [1, 2, 3, 4, 5, 7, 8, 9, 12, 16, 20, 33]))
        dt = str(rng.choice(["f32", "f16", "bf16"]))
        w = synth.make_weights(rng, qt, n, k)
        xd = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(TORCH_DT[dt]).cuda()
        f = ops.ggml_mul_mat_vec_a8 if op == "mmvq" else ops.ggml_mul_mat_a8
        y = f(torch.from_numpy(w).cuda(), xd, qt, n)
        assert y.shape == (m, n) and y.dtype == TORCH_DT[dt]
        err = o.rel_l2(y.float().cpu().numpy(), o.mul_mat_a8(w, xd.float().cpu().numpy(), qt, n, op))
        tol = {"f32": 1e-5, "f16": 1e-3, "bf16": 4e-3}[dt] * (4 if n * m < 64 else 1)
        assert np.isfinite(err) and err <= tol, (case, op, o.TYPE_NAMES[qt], n, k, m, dt, err)


@pytest.mark.parametrize("seed", [1, 2])
def test_moe_layer_sweep_against_the_chained_operators(seed):
    """100 draws per seed of the MoE layer through dispatch.fused_moe_gguf -- 14 formats for either projection, 1 to 40
    experts, top-1 to top-8, 1 to 600 tokens, hidden and inner sizes that end inside tiles -- whichever route the layer
    takes (two launches, 16- or 32-slot tiles, the slot order on the dense engine, or the separate operators) against
    the reference's sequence of operators (fused_moe.py:62-95) run one by one on the same inputs: only the result's own
    rounding to half separates the two."""
    ops = _ops()
    rng = np.random.default_rng(9300 + seed)
    fmts = [o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1, o.Q8_0, o.Q2_K, o.Q3_K, o.Q4_K, o.Q5_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS, o.IQ4_NL, o.IQ3_S]
    for case in range(100):
        qt, qt2 = int(rng.choice(fmts)), int(rng.choice(fmts))
        qk1, qk2 = o.QUANT_SIZES[qt][0], o.QUANT_SIZES[qt2][0]
        E = int(rng.choice([1, 2, 3, 5, 8, 17, 40]))
        top_k = int(rng.integers(1, min(E, 8) + 1))
        tokens = int(rng.choice([1, 2, 3, 7, 16, 33, 64, 65, 100, 257, 600]))
        H = int(rng.choice([256, 512, 768, 1024] if qk1 == 256 else [256, 288, 512, 736, 1024]))
        I = int(rng.choice([256, 512, 768] if qk2 == 256 else [128, 160, 256, 352, 512, 768]))
        w1 = np.stack([synth.make_weights(rng, qt, 2 * I, H) for _ in range(E)])
        w2 = np.stack([synth.make_weights(rng, qt2, H, I) for _ in range(E)])
        x = (4.0 * rng.standard_normal((tokens, H))).astype(np.float16)
        logits = rng.standard_normal((tokens, E))
        ids = np.argsort(-logits, axis=1)[:, :top_k].astype(np.int32)
        sel = np.take_along_axis(logits, ids, 1)
        tw = (np.exp(sel) / np.exp(sel).sum(1, keepdims=True)).astype(np.float32)
        w1d, w2d, idd = torch.from_numpy(w1).cuda(), torch.from_numpy(w2).cuda(), torch.from_numpy(ids).cuda()
        pairs, flat1 = tokens * top_k, idd.reshape(-1, 1).contiguous()
        for _ in range(4):   # keep the intermediate and the result inside the half range whatever the synthetic scales are
            xd = torch.from_numpy(x).cuda()
            h32 = ops.ggml_moe_a8_vec(xd.float(), w1d, idd, top_k, qt, 2 * I, tokens)
            a64 = o.silu_and_mul(h32.cpu().numpy().astype(np.float64))
            y32 = ops.ggml_moe_a8_vec(torch.from_numpy(a64.astype(np.float32)).cuda(), w2d, flat1, 1, qt2, H, pairs)
            big = max(float(h32.abs().max()), float(np.abs(a64).max()), float(y32.abs().max()))
            if big < 200.0:
                break
            x = (x.astype(np.float32) * np.sqrt(20.0 / big)).astype(np.float16)
        path = D.select_moe_path(qt, qt2, tokens)
        got = D.fused_moe_gguf(xd, w1d, w2d, torch.from_numpy(tw).cuda().half(), idd, qt, qt2, "silu")
        if path == "vec":
            h = ops.ggml_moe_a8_vec(xd, w1d, idd, top_k, qt, 2 * I, tokens)
            a = o.silu_and_mul(h.cpu().numpy(), stored=np.float16)
            y = ops.ggml_moe_a8_vec(torch.from_numpy(a).cuda(), w2d, flat1, 1, qt2, H, pairs)
        elif path == "grouped":
            blk = ops.ggml_moe_get_block_size(qt)
            s_, eids, npost = o.moe_align_block_size(ids, blk, E)
            sd, ed, nd = (torch.from_numpy(np.ascontiguousarray(v)).cuda() for v in (s_, eids, npost))
            h = ops.ggml_moe_a8(xd, w1d, sd, ed, nd, qt, 2 * I, top_k, tokens)
            a = o.silu_and_mul(h.cpu().numpy(), stored=np.float16)
            y = ops.ggml_moe_a8(torch.from_numpy(a).cuda(), w2d, sd, ed, nd, qt2, H, 1, pairs)
        else:
            continue   # (the reference's loop over experts: dense products, covered elsewhere)
        yy = y.cpu().numpy().astype(np.float64).reshape(tokens, top_k, H)
        want = (yy * tw.astype(np.float16).astype(np.float64)[:, :, None]).astype(np.float16).astype(np.float64).sum(1)
        err = o.rel_l2(got.float().cpu().numpy(), want)
        assert np.isfinite(err) and err <= 5e-4, (case, o.TYPE_NAMES[qt], o.TYPE_NAMES[qt2], E, top_k, tokens, H, I, path, err)
