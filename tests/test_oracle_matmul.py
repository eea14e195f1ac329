"""Pins the oracle's q8_1 quantizer and a8 matmuls.

The matmul checks re-derive every output from the reference's *per-thread* dot
product code (csrc/gguf/vecdotq.cuh, the ``vec_dot_<fmt>_q8_1`` entry points
with their ``iqs`` indexing) written as scalar Python loops over raw block
bytes, which shares no code with the vectorised oracle.  A transposed
sub-block, a wrong scale index, a dropped offset term or the wrong "sum" in the
offset term each fail at least one of them.
"""
import numpy as np
import pytest

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd.tables import grids


# ---------------------------------------------------------------- q8_1
def test_q8_1_properties():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 700)).astype(np.float16)
    x[0, :32] = 0          # an all-zero block
    x[1, 40] = 6.0e4       # near fp16 max
    q, d, s = o.quantize_q8_1(x)
    assert q.shape == (5, 1024) and d.shape == (5, 32) and s.shape == (5, 32)
    assert np.all(q[:, 700:] == 0) and np.all(np.abs(q.astype(int)) <= 127)
    assert np.all(q[0, :32] == 0) and d[0, 0] == 0 and s[0, 0] == 0
    xf = np.zeros((5, 1024), dtype=np.float32)
    xf[:, :700] = x.astype(np.float32)
    blk = xf.reshape(5, 32, 32)
    amax = np.abs(blk).max(axis=2)
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float16))
    # each block's max-magnitude element quantizes to +-127
    nz = amax > 0
    assert np.all(np.abs(q.reshape(5, 32, 32)).max(axis=2)[nz] == 127)
    # |x - d32*q| <= d32/2 with the unrounded fp32 scale
    d32 = (amax / np.float32(127))[:, :, None]
    assert np.all(np.abs(blk - d32 * q.reshape(5, 32, 32)) <= d32 * 0.50002)
    # the stored sum is the fp32 butterfly tree sum rounded to half
    tree = blk.copy()
    for mask in (16, 8, 4, 2, 1):
        tree = np.array([[[tree[m, b, i] + tree[m, b, i ^ mask] for i in range(32)] for b in range(32)] for m in range(5)], dtype=np.float32)
    assert np.array_equal(s, tree[:, :, 0].astype(np.float16))


def test_q8_1_round_half_away_from_zero():
    # amax = 127 -> d = 1 exactly, so x/d = x: 0.5 -> 1, -0.5 -> -1, 2.5 -> 3, 1.49 -> 1
    x = np.zeros((1, 32), dtype=np.float32)
    x[0, :6] = [127.0, 0.5, -0.5, 2.5, -2.5, 1.4990234]
    q, d, _ = o.quantize_q8_1(x)
    assert d[0, 0] == 1.0
    assert list(q[0, :6]) == [127, 1, -1, 3, -3, 1]
    # 0.49999997 must not round up (the trunc(v + 0.5) shortcut would give 1)
    x[0, 1] = np.float32(0.49999997)
    q, _, _ = o.quantize_q8_1(x)
    assert q[0, 1] == 0


# ---------------------------------------------------------------- scalar per-thread dots
def _dp4a(a, b):
    return int(np.dot(a.astype(np.int64), b.astype(np.int64)))


def _f16(buf, off):
    return float(buf[off:off + 2].view("<f2")[0])


def _dot_q4_0(blk, q8, d8, s8, path):  # vecdotq.cuh:46-66, 493-509
    d4 = _f16(blk, 0)
    qs = blk[2:18]
    sumi = _dp4a(qs & 15, q8[:16]) + _dp4a(qs >> 4, q8[16:])
    return d4 * (sumi * d8 - 8 * s8)


def _dot_q8_0(blk, q8, d8, s8, path):  # vecdotq.cuh:165-177, 852-867
    return _f16(blk, 0) * d8 * _dp4a(blk[2:34].view(np.int8), q8)


def _dot_q4_k(blk, q8, d8, s8, path):  # vecdotq.cuh:328-379, 1159-1202; q8/d8/s8 cover 8 blocks
    d, dmin = _f16(blk, 0), _f16(blk, 2)
    sc12 = blk[4:16]
    qs = blk[16:144]
    total = 0.0
    for iqs in range(0, 32, 2):                 # one reference thread each
        bq8 = 2 * ((iqs // 2) // 4)
        off = 16 * bq8 + 4 * ((iqs // 2) % 4)
        v0, v1 = qs[off:off + 4], qs[off + 16:off + 20]
        j = bq8 // 2
        s16 = sc12.view("<u2")
        if j < 2:
            a0, a1 = int(s16[j]) & 0x3F3F, int(s16[j + 2]) & 0x3F3F
        else:
            a0 = (int(s16[j + 2]) & 0x0F0F) | ((int(s16[j - 2]) & 0xC0C0) >> 2)
            a1 = ((int(s16[j + 2]) >> 4) & 0x0F0F) | ((int(s16[j]) & 0xC0C0) >> 2)
        sc = [a0 & 0xFF, a0 >> 8]
        mn = [a1 & 0xFF, a1 >> 8]
        sumf_d = sumf_m = 0.0
        for i in range(2):
            u0 = q8[32 * (bq8 + i) + 4 * ((iqs // 2) % 4):][:4]
            u1 = q8[32 * (bq8 + i) + 16 + 4 * ((iqs // 2) % 4):][:4]
            dot1 = _dp4a((v0 >> (4 * i)) & 15, u0) + _dp4a((v1 >> (4 * i)) & 15, u1)
            dot2 = int(u0.astype(int).sum() + u1.astype(int).sum())
            sumf_d += d8[bq8 + i] * (dot1 * sc[i])
            if path == "mmvq":
                sumf_m += d8[bq8 + i] * (dot2 * mn[i])
            else:  # MMQ: stored block sum; every one of the 4 threads of a sub-block pair adds a quarter
                sumf_m += s8[bq8 + i] * mn[i] / 4.0
        total += d * sumf_d - dmin * sumf_m
    return total


def _dot_q6_k(blk, q8, d8, s8, path):  # vecdotq.cuh:447-465, 1417-1441
    ql, qh = blk[0:128], blk[128:192]
    sc = blk[192:208].view(np.int8)
    d = _f16(blk, 208)
    total = 0.0
    for iqs in range(32):
        bq8 = 4 * (iqs // 16) + (iqs % 16) // 8
        so = 8 * (iqs // 16) + (iqs % 16) // 4
        sh = 2 * ((iqs % 16) // 8)
        vl = ql[4 * iqs:4 * iqs + 4]
        vh = qh[4 * (8 * (iqs // 16) + iqs % 8):][:4] >> sh
        sumf = 0.0
        for i in range(2):
            vi = (((vl >> (4 * i)) & 15) | (((vh >> (4 * i)) & 3) << 4)).astype(int) - 32
            u = q8[32 * (bq8 + 2 * i) + 4 * (iqs % 8):][:4]
            sumf += d8[bq8 + 2 * i] * (_dp4a(vi, u) * int(sc[so + 4 * i]))
        total += d * sumf
    return total


def _dot_iq4_xs(blk, q8, d8, s8, path):  # vecdotq.cuh:1791-1811
    kv = grids.kvalues_iq4nl().astype(int)
    d = _f16(blk, 0)
    sh = int(blk[2:4].view("<u2")[0])
    total = 0.0
    for ib in range(8):
        ls = ((int(blk[4 + ib // 2]) >> (4 * (ib % 2))) & 15) | (((sh >> (2 * ib)) & 3) << 4)
        q4 = blk[8 + 16 * ib:8 + 16 * ib + 16]
        u = q8[32 * ib:32 * ib + 32]
        sumi = _dp4a(kv[q4 & 15], u[:16]) + _dp4a(kv[q4 >> 4], u[16:])
        total += d * (ls - 32) * d8[ib] * sumi
    return total


def _dot_iq2_xxs(blk, q8, d8, s8, path):  # vecdotq.cuh:1531-1552
    grid = grids.grid_bytes(grids.iq2xxs_grid()).astype(int)
    ks = grids.ksigns_iq2xs()
    d = _f16(blk, 0)
    total = 0.0
    for ib in range(8):
        g = blk[2 + 8 * ib:2 + 8 * ib + 8]
        aux = int(g[4:8].view("<u4")[0])
        sumi = 0
        for l in range(4):
            signs = int(ks[(aux >> (7 * l)) & 127])
            for j in range(8):
                sumi += int(q8[32 * ib + 8 * l + j]) * grid[g[l], j] * (-1 if signs & (1 << j) else 1)
        total += d * (0.5 + (aux >> 28)) * d8[ib] * 0.25 * sumi
    return total


SCALAR = {o.Q4_0: _dot_q4_0, o.Q8_0: _dot_q8_0, o.Q4_K: _dot_q4_k, o.Q6_K: _dot_q6_k, o.IQ4_XS: _dot_iq4_xs, o.IQ2_XXS: _dot_iq2_xxs}


def _scalar_matmul(w, x, qtype, n, path):
    qk, bs = o.QUANT_SIZES[qtype]
    m, k = x.shape
    q, d8, s8 = o.quantize_q8_1(x)
    d8 = d8.astype(np.float64)
    s8 = s8.astype(np.float64)
    wb = w.reshape(n, k // qk, bs)
    y = np.zeros((m, n))
    r = qk // 32
    for mi in range(m):
        for ni in range(n):
            acc = 0.0
            for b in range(k // qk):
                qq = q[mi, b * qk:(b + 1) * qk]
                if r == 1:
                    acc += SCALAR[qtype](wb[ni, b], qq, d8[mi, b], s8[mi, b], path)
                else:
                    acc += SCALAR[qtype](wb[ni, b], qq, d8[mi, b * r:(b + 1) * r], s8[mi, b * r:(b + 1) * r], path)
            y[mi, ni] = acc
    return y


@pytest.mark.parametrize("path", ["mmvq", "mmq"])
@pytest.mark.parametrize("qtype", sorted(SCALAR))
def test_a8_matmul_against_per_thread_form(qtype, path):
    rng = np.random.default_rng(10 + qtype)
    n, k, m = 3, 768, 2      # K is not a multiple of 512: padded q8_1 columns must not matter
    w = o.make_weights(rng, qtype, n, k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    got = o.mul_mat_a8(w, x, qtype, n, path)
    exp = _scalar_matmul(w, x, qtype, n, path)
    assert np.allclose(got, exp, rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize("qtype", [o.Q8_0, o.Q6_K, o.IQ4_XS, o.IQ2_XXS, o.Q3_K, o.IQ4_NL, o.IQ2_XS, o.IQ2_S, o.IQ3_XXS, o.IQ3_S])
def test_cross_identity_no_offset_formats(qtype):
    # formats without an offset term: Y == exact-dequant(W) @ dequant(q8_1(X))^T, integer-exact per block
    rng = np.random.default_rng(30 + qtype)
    n, k, m = 5, 1024, 3
    w = o.make_weights(rng, qtype, n, k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    q, d8, _ = o.quantize_q8_1(x)
    xh = o.dequant_q8_1(q, d8)[:, :k]
    wd = o.dequant_exact(w, qtype).reshape(n, k)
    assert np.allclose(o.mul_mat_a8(w, x, qtype, n), xh @ wd.T, rtol=1e-12, atol=1e-14)


def test_q4_0_offset_uses_stored_half_sum():
    # the a8 result differs from the generic product by 8*d4*(s8 - d8*sum(u)): non-zero in general
    rng = np.random.default_rng(40)
    w = o.make_weights(rng, o.Q4_0, 4, 256)
    x = rng.standard_normal((2, 256)).astype(np.float16)
    q, d8, s8 = o.quantize_q8_1(x)
    xh = o.dequant_q8_1(q, d8)[:, :256]
    generic = xh @ o.dequant_exact(w, o.Q4_0).reshape(4, 256).T
    got = o.mul_mat_a8(w, x, o.Q4_0, 4)
    d4 = w.reshape(4, 8, 18)[:, :, 0:2].copy().view("<f2")[:, :, 0].astype(np.float64)
    usum = q.reshape(2, -1, 32).sum(axis=2)[:, :8].astype(np.float64) * d8[:, :8].astype(np.float64)
    corr = 8 * (usum - s8[:, :8].astype(np.float64)) @ d4.T
    assert np.allclose(got, generic + corr, rtol=1e-12, atol=1e-14)
    assert np.abs(corr).max() > 0


def test_a8_close_to_unquantized_oracle():
    rng = np.random.default_rng(50)
    for qtype in (o.Q4_0, o.Q8_0, o.Q4_K, o.Q6_K, o.IQ4_XS, o.IQ2_XXS):
        w = o.make_weights(rng, qtype, 64, 1024)
        x = rng.standard_normal((4, 1024)).astype(np.float16)
        assert o.rel_l2(o.mul_mat_a8(w, x, qtype, 64), o.mul_mat_f32(w, x, qtype, 64)) < 2e-2


# ---------------------------------------------------------------- MoE
def test_moe_align_block_size_contract():
    rng = np.random.default_rng(60)
    t, top_k, e, blk = 13, 4, 16, 8
    ids = np.stack([rng.choice(e, size=top_k, replace=False) for _ in range(t)]).astype(np.int32)
    ids[ids == 3] = 5      # expert 3 gets no tokens (duplicates in a row are fine for this contract)
    s, eids, npost = o.moe_align_block_size(ids, blk, e)
    numel = t * top_k
    assert npost[0] % blk == 0 and npost[0] <= len(s) and len(s) % blk == 0
    real = s[s < numel]
    assert sorted(real.tolist()) == list(range(numel))          # every pair exactly once
    assert np.all(s[npost[0]:] == numel)
    flat = ids.reshape(-1)
    for b in range(npost[0] // blk):
        seg = s[b * blk:(b + 1) * blk]
        assert np.all(flat[seg[seg < numel]] == eids[b])
        assert np.any(seg < numel)
    assert 3 not in eids[: npost[0] // blk]


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q4_K])
def test_moe_oracles_against_token_loop(qtype):
    # quantization/fused_moe.py:119-132 of the reference defines the result as a per-token, per-expert loop
    rng = np.random.default_rng(70)
    t, top_k, e, n, k, blk = 9, 2, 6, 8, 256, 8
    w = np.stack([o.make_weights(rng, qtype, n, k) for _ in range(e)])
    x = rng.standard_normal((t, k)).astype(np.float16)
    ids = np.stack([rng.choice(e, size=top_k, replace=False) for _ in range(t)]).astype(np.int32)
    exp_vec = np.zeros((t * top_k, n))
    exp_mmq = np.zeros((t * top_k, n))
    for tok in range(t):
        for j in range(top_k):
            exp_vec[tok * top_k + j] = o.mul_mat_a8(w[ids[tok, j]], x[tok:tok + 1], qtype, n, "mmvq")[0]
            exp_mmq[tok * top_k + j] = o.mul_mat_a8(w[ids[tok, j]], x[tok:tok + 1], qtype, n, "mmq")[0]
    assert np.allclose(o.moe_a8_vec(x, w, ids, top_k, qtype, n, t), exp_vec, rtol=1e-12, atol=1e-14)
    s, eids, npost = o.moe_align_block_size(ids, blk, e)
    got = o.moe_a8(x, w, s, eids, npost, qtype, n, top_k, t, blk)
    assert np.allclose(got, exp_mmq, rtol=1e-12, atol=1e-14)
    # blocks at or past the padded count, and out-of-range expert ids, write nothing
    eids2 = eids.copy()
    eids2[0] = 300
    got2 = o.moe_a8(x, w, s, eids2, npost, qtype, n, top_k, t, blk)
    skipped = s[:blk][s[:blk] < t * top_k]
    assert np.all(got2[skipped] == 0)
    keep = np.setdiff1d(np.arange(t * top_k), skipped)
    assert np.allclose(got2[keep], exp_mmq[keep], rtol=1e-12, atol=1e-14)


def test_silu_and_mul():
    x = np.array([[0.0, 1.0, -2.0, 3.0, 4.0, 5.0]])
    out = o.silu_and_mul(x)
    exp = np.array([[0.0 * 3.0, 1 / (1 + np.exp(-1.0)) * 4.0, -2 / (1 + np.exp(2.0)) * 5.0]])
    assert np.allclose(out, exp)


def test_silu_and_mul_as_stored_in_half_matches_the_library_sequence():
    """The intermediate of the MoE layer is act(gate) rounded to half, times up, rounded again (fused_moe.py:44-51).
    torch's CPU half kernels do exactly that sequence (silu evaluated in fp32, stored as half; half product rounded
    once), an implementation that shares nothing with the oracle."""
    import torch

    rng = np.random.default_rng(77)
    x = (rng.standard_normal((64, 512)) * 4).astype(np.float16)
    got = o.silu_and_mul(x, stored=np.float16)
    t = torch.from_numpy(x)
    want = (torch.nn.functional.silu(t[:, :256]) * t[:, 256:]).numpy()
    assert got.dtype == np.float16
    mism = np.count_nonzero(got.view(np.uint16) != want.view(np.uint16))
    assert mism <= got.size // 2000      # fp64 against fp32 evaluation of exp: a last-place tie now and then
    assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=1e-7)
    single = o.silu_and_mul(x.astype(np.float64)).astype(np.float16)
    assert np.count_nonzero(single.view(np.uint16) != got.view(np.uint16)) > got.size // 20   # one rounding is a different function
