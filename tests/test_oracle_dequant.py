"""Pins the oracle's dequantisation without any import of the reference.

Each check is chosen so a plausible slip (wrong nibble half, transposed sub-block,
wrong scale index, dropped offset, wrong rounding point) fails it:
closed forms on hand-built blocks, exhaustive sweeps of small index spaces, a
single walking code against the per-thread index arithmetic of
csrc/gguf/dequantize.cuh written out as scalar loops, and ulp distances between
the two rounding flavours.
"""
import numpy as np
import pytest

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd.tables import grids


def f16b(v):
    return np.frombuffer(np.float16(v).tobytes(), dtype=np.uint8)


def test_block_sizes():
    # triton/gemm/utils.py:28-47 of the reference lists the same byte sizes
    expect = {2: 18, 3: 20, 6: 22, 7: 24, 8: 34, 9: 36, 10: 84, 11: 110, 12: 144, 13: 176, 14: 210,
              16: 66, 17: 74, 18: 98, 19: 50, 20: 18, 21: 110, 22: 82, 23: 136, 29: 56}
    assert {k: v[1] for k, v in o.QUANT_SIZES.items()} == expect
    assert all(v[0] == (32 if k in (2, 3, 6, 7, 8, 9, 20) else 256) for k, v in o.QUANT_SIZES.items())


def test_q8_0_closed_form_all_bytes():
    blk = np.zeros((8, 34), dtype=np.uint8)
    blk[:, 0:2] = f16b(1.0)
    blk[:, 2:] = np.arange(256, dtype=np.uint8).reshape(8, 32)
    out = o.dequantize(blk, o.Q8_0, "f32")
    assert np.array_equal(out, np.arange(256, dtype=np.uint8).view(np.int8).astype(np.float32))
    blk[:, 0:2] = f16b(-0.5)
    assert np.array_equal(o.dequantize(blk, o.Q8_0, "f32"), -0.5 * np.arange(256, dtype=np.uint8).view(np.int8).astype(np.float32))


def test_q4_0_closed_form_all_bytes():
    blk = np.zeros((16, 18), dtype=np.uint8)
    blk[:, 0:2] = f16b(1.0)
    blk[:, 2:] = np.arange(256, dtype=np.uint8).reshape(16, 16)
    out = o.dequantize(blk, o.Q4_0, "f32").reshape(16, 32)
    qs = np.arange(256).reshape(16, 16)
    assert np.array_equal(out[:, :16], (qs & 15) - 8)      # low nibbles -> first half of the block
    assert np.array_equal(out[:, 16:], (qs >> 4) - 8)      # high nibbles -> second half


def test_get_scale_min_k4_bruteforce():
    rng = np.random.default_rng(1)
    sc12 = rng.integers(0, 256, size=(4096, 12), dtype=np.uint8)
    sc, mn = o.get_scale_min_k4(sc12)
    # direct bit description: 8 scales and 8 mins of 6 bits each;
    # j<4: low 6 bits of bytes j / j+4; j>=4: low/high nibble of byte j+4 plus the top 2 bits of bytes j-4 / j
    for j in range(8):
        if j < 4:
            e_sc = sc12[:, j] & 0x3F
            e_mn = sc12[:, j + 4] & 0x3F
        else:
            e_sc = (sc12[:, j + 4] & 0x0F) + 16 * (sc12[:, j - 4] // 64)
            e_mn = (sc12[:, j + 4] // 16) + 16 * (sc12[:, j] // 64)
        assert np.array_equal(sc[:, j], e_sc) and np.array_equal(mn[:, j], e_mn)
    # uint16-lane form used by the reference's vec-dot (vecdotq.cuh:1179-1190)
    s16 = sc12.view("<u2")
    for g in range(4):
        if g < 2:
            a0 = s16[:, g] & 0x3F3F
            a1 = s16[:, g + 2] & 0x3F3F
        else:
            a0 = (s16[:, g + 2] & 0x0F0F) | ((s16[:, g - 2] & 0xC0C0) >> 2)
            a1 = ((s16[:, g + 2] >> 4) & 0x0F0F) | ((s16[:, g] & 0xC0C0) >> 2)
        assert np.array_equal(a0 & 0xFF, sc[:, 2 * g]) and np.array_equal(a0 >> 8, sc[:, 2 * g + 1])
        assert np.array_equal(a1 & 0xFF, mn[:, 2 * g]) and np.array_equal(a1 >> 8, mn[:, 2 * g + 1])


def _q4k_block(d=1.0, dmin=0.0, sc=None, mn=None, qs=None):
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = f16b(d)
    blk[2:4] = f16b(dmin)
    sc = np.zeros(8, dtype=np.uint8) if sc is None else np.asarray(sc, dtype=np.uint8)
    mn = np.zeros(8, dtype=np.uint8) if mn is None else np.asarray(mn, dtype=np.uint8)
    for j in range(4):
        blk[4 + j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        blk[8 + j] = (mn[j] & 63) | ((mn[j + 4] >> 4) << 6)
        blk[12 + j] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    if qs is not None:
        blk[16:] = qs
    return blk


def test_q4_k_walking_nibble():
    # one non-zero nibble walks all 256 positions; scale of sub-block j is j+1 so a
    # wrong sub-block assignment changes the value
    sc = np.arange(1, 9)
    for pos in range(256):
        qs = np.zeros(128, dtype=np.uint8)
        g, r = divmod(pos, 64)           # 64 elements share 32 bytes: low nibbles first
        byte = 32 * g + (r % 32)
        qs[byte] = 5 << (4 * (r // 32))
        out = o.dequantize(_q4k_block(sc=sc, qs=qs)[None], o.Q4_K, "f32").reshape(256)
        exp = np.zeros(256, dtype=np.float32)
        exp[pos] = 5 * sc[pos // 32]
        assert np.array_equal(out, exp), pos


def test_q4_k_min_term_and_rounding_flavours():
    sc = [63, 1, 2, 3, 40, 50, 60, 33]
    mn = [1, 63, 5, 7, 9, 11, 35, 62]
    qs = np.full(128, 0xA3, dtype=np.uint8)
    blk = _q4k_block(d=0.5, dmin=0.25, sc=sc, mn=mn, qs=qs)[None]
    out = o.dequantize(blk, o.Q4_K, "f32").reshape(8, 32)
    for j in range(8):
        q = 3 if j % 2 == 0 else 10
        assert np.all(out[j] == 0.5 * sc[j] * q - 0.25 * mn[j])
    # random blocks: fused vs unfused vs fp32 differ by a few half ulps at most, never more than the
    # reference's own tolerance atol=1e-2, rtol=4e-2 (tests/test_kernels.py:99)
    rng = np.random.default_rng(2)
    w = o.make_weights(rng, o.Q4_K, 64, 1024)
    a = o.dequantize(w, o.Q4_K, "f16", "ref", contract=True).astype(np.float64)
    b = o.dequantize(w, o.Q4_K, "f16", "ref", contract=False).astype(np.float64)
    c = o.dequantize(w, o.Q4_K, "f16", "f32").astype(np.float64)
    for u, v in ((a, b), (a, c), (b, c)):
        assert np.all(np.abs(u - v) <= 1e-2 + 4e-2 * np.abs(v))
    assert np.any(a != b)  # the contraction choice is observable, so it has to be pinned


def _q6k_scalar(blk):
    """dequantize_block_q6_K written per thread (dequantize.cuh:232-256), fp64 exact."""
    ql, qh = blk[0:128], blk[128:192]
    sc = blk[192:208].view(np.int8)
    d = float(blk[208:210].view("<f2")[0])
    y = np.zeros(256)
    for tid in range(64):
        ip, il = divmod(tid, 32)
        isx = 8 * ip + il // 16
        base = 128 * ip + il
        h = int(qh[32 * ip + il])
        lo0, lo1 = int(ql[64 * ip + il]), int(ql[64 * ip + il + 32])
        y[base + 0] = d * sc[isx + 0] * (((lo0 & 0xF) | (((h >> 0) & 3) << 4)) - 32)
        y[base + 32] = d * sc[isx + 2] * (((lo1 & 0xF) | (((h >> 2) & 3) << 4)) - 32)
        y[base + 64] = d * sc[isx + 4] * (((lo0 >> 4) | (((h >> 4) & 3) << 4)) - 32)
        y[base + 96] = d * sc[isx + 6] * (((lo1 >> 4) | (((h >> 6) & 3) << 4)) - 32)
    return y


def test_q6_k_against_thread_index_form():
    rng = np.random.default_rng(3)
    w = o.random_blocks(rng, o.Q6_K, 2, 1024)
    got = o.dequant_exact(w, o.Q6_K).reshape(-1, 256)
    for i, blk in enumerate(w.reshape(-1, 210)):
        assert np.array_equal(got[i], _q6k_scalar(blk))


def test_q6_k_int2half_rounding_point():
    # sc*(q-32) = 127*31 = 3937 is not representable in half: int2half_rn gives 3936, then * d
    blk = np.zeros(210, dtype=np.uint8)
    blk[0:128] = 0xFF
    blk[128:192] = 0xFF          # q = 63 everywhere
    blk[192:208] = 127
    blk[208:210] = f16b(1.0)
    ref = o.dequantize(blk[None], o.Q6_K, "f32", "ref")
    f32 = o.dequantize(blk[None], o.Q6_K, "f32", "f32")
    assert np.all(ref == 3936.0) and np.all(f32 == 3937.0)
    # quantizer round trip: |w - dq| <= half a step
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((8, 512)) * 0.02).astype(np.float32)
    dq = o.dequantize(o.quantize_q6_k(x), o.Q6_K, "f32", "f32").reshape(8, 512)
    assert o.rel_l2(dq, x) < 2e-2


def test_iq4_xs_exhaustive_indices_and_scales():
    kv = grids.kvalues_iq4nl().astype(np.float64)
    # every byte value in every position; 6-bit scale sweeps 0..63 over the blocks
    blocks = []
    for ls in range(64):
        blk = np.zeros(136, dtype=np.uint8)
        blk[0:2] = f16b(1.0)
        lsv = [(ls + 7 * ib) % 64 for ib in range(8)]
        sh = 0
        for ib in range(8):
            sh |= (lsv[ib] >> 4) << (2 * ib)
            blk[4 + ib // 2] |= (lsv[ib] & 15) << (4 * (ib % 2))
        blk[2:4] = np.frombuffer(np.uint16(sh).tobytes(), dtype=np.uint8)
        blk[8:] = (np.arange(128) * 2 + ls * 5) % 256
        blocks.append((blk, lsv))
    w = np.stack([b for b, _ in blocks])
    out = o.dequantize(w, o.IQ4_XS, "f32").reshape(64, 8, 32)
    for i, (blk, lsv) in enumerate(blocks):
        for ib in range(8):
            q = blk[8 + 16 * ib:8 + 16 * ib + 16]
            exp = np.concatenate([kv[q & 15], kv[q >> 4]]) * (lsv[ib] - 32)
            assert np.array_equal(out[i, ib], exp.astype(np.float32))


def test_iq2_xxs_exhaustive():
    grid = grids.grid_bytes(grids.iq2xxs_grid()).astype(np.float64)
    ks = grids.ksigns_iq2xs()
    # all 256 grid indices x all 128 sign indices x all 16 scales, spread over blocks
    rng = np.random.default_rng(5)
    combos = [(gi, si, (gi + si) % 16) for gi in range(256) for si in range(0, 128, 1)]
    rng.shuffle(combos)
    combos = combos[:4096]
    nblk = len(combos) // 8
    w = np.zeros((nblk, 66), dtype=np.uint8)
    w[:, 0:2] = f16b(2.0)
    for b in range(nblk):
        for ib in range(8):
            gi, si, s = combos[8 * b + ib]
            idx = [gi, (gi * 7 + 3) % 256, (gi * 13 + 5) % 256, (gi + 128) % 256]
            sg = [si, (si * 3 + 1) % 128, (si + 64) % 128, (127 - si)]
            aux = sg[0] | (sg[1] << 7) | (sg[2] << 14) | (sg[3] << 21) | (s << 28)
            w[b, 2 + 8 * ib:2 + 8 * ib + 4] = idx
            w[b, 2 + 8 * ib + 4:2 + 8 * ib + 8] = np.frombuffer(np.uint32(aux).tobytes(), dtype=np.uint8)
    out = o.dequantize(w, o.IQ2_XXS, "f32").reshape(nblk, 8, 4, 8)
    for b in range(0, nblk, 7):
        for ib in range(8):
            gi, si, s = combos[8 * b + ib]
            idx = [gi, (gi * 7 + 3) % 256, (gi * 13 + 5) % 256, (gi + 128) % 256]
            sg = [si, (si * 3 + 1) % 128, (si + 64) % 128, (127 - si)]
            for l in range(4):
                sign = np.array([-1.0 if (int(ks[sg[l]]) >> j) & 1 else 1.0 for j in range(8)])
                exp = 2.0 * (0.5 + s) * 0.25 * grid[idx[l]] * sign
                assert np.array_equal(out[b, ib, l], exp.astype(np.float32)), (b, ib, l)


@pytest.mark.parametrize("qtype", [o.Q4_0, o.Q8_0, o.IQ4_XS, o.IQ2_XXS, o.IQ4_NL, o.IQ2_XS, o.IQ2_S, o.IQ3_XXS, o.IQ3_S])
def test_single_rounding_formats_flavours_agree(qtype):
    # one rounding of an exactly representable product: both flavours give the same bits
    rng = np.random.default_rng(6)
    w = o.random_blocks(rng, qtype, 8, 1024)
    for dt in ("f16", "f32", "bf16"):
        a = o.dequantize(w, qtype, dt, "ref")
        b = o.dequantize(w, qtype, dt, "f32")
        if dt != "f16" and qtype in o.HALF_MATH_TYPES:
            continue  # fp32/bf16 outputs of the half-math kernels are converted from the half result
        if dt == "bf16":
            a, b = o.bf16_bits_to_f32(a), o.bf16_bits_to_f32(b)
        assert np.array_equal(a, b)  # value equality: the sign of a zero may differ


def test_bf16_rounding_helper():
    x = np.array([1.0, 1.00390625, 1.01171875, -3.0e38, 1e-40, np.inf], dtype=np.float32)
    bits = o.f32_to_bf16_bits(x)
    back = o.bf16_bits_to_f32(bits)
    assert back[0] == 1.0 and back[1] == 1.0 and back[2] == np.float32(1.015625)  # ties to even, then up
    assert np.isinf(back[5])


@pytest.mark.parametrize("qtype", sorted(t for t in o.QUANT_SIZES if t != o.Q8_1))
def test_exact_vs_ref_within_reference_tolerance(qtype):
    rng = np.random.default_rng(7)
    w = o.random_blocks(rng, qtype, 4, 1024)
    ex = o.dequant_exact(w, qtype)
    for dt in ("f16", "f32"):
        r = o.dequantize(w, qtype, dt, "ref").astype(np.float64)
        assert np.all(np.abs(r - ex) <= 1e-2 + 4e-2 * np.abs(ex))
