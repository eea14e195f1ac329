"""Independent pins for the oracle on the thirteen formats beyond the six headline ones.

Every function below restates one reference kernel thread by thread, in plain Python loops, straight from the cited
source lines and without touching ``oracle.unpack`` or any other vectorised helper; the oracle has to reproduce them
bit for bit (dequantize, fp16 output) or to fp64 round-off (a8 dot products, both the MMVQ and the MMQ semantics).
A transposed index, a dropped high bit, a wrong scale nibble or the wrong "sum" in an offset term fails here.
"""
import numpy as np
import pytest

from oracle import gguf_oracle as o
from vllm_gguf_plugin_prism_amd.tables import grids

H = np.float16


def hmul(a, b):
    return H(np.float32(a) * np.float32(b))


def hfma(a, b, c):  # one rounding; the exact value fits a double
    return H(np.float64(a) * np.float64(b) + np.float64(c))


def f16_at(blk, off):
    return blk[off:off + 2].view("<f2")[0]


def u16_at(blk, off):
    return int(blk[off:off + 2].view("<u2")[0])


def u32_at(blk, off):
    return int(blk[off:off + 4].view("<u4")[0])


KMASK = [1 << j for j in range(8)]


# ------------------------------------------------------------------------------------------------ dequantize
def dq_q4_1(blk):  # dequantize.cuh:17-30 via dequantize_block: v.x -> y[iqs], v.y -> y[iqs + 16]
    d, m = f16_at(blk, 0), f16_at(blk, 2)
    y = np.zeros(32, H)
    for iqs in range(16):
        vui = int(blk[4 + iqs])
        y[iqs] = hfma(H(vui & 0xF), d, m)
        y[iqs + 16] = hfma(H(vui >> 4), d, m)
    return y


def dq_q5(blk, has_m):  # dequantize.cuh:32-67
    off = 4 if has_m else 2
    d = f16_at(blk, 0)
    m = f16_at(blk, 2) if has_m else None
    qh = u32_at(blk, off)
    y = np.zeros(32, H)
    for iqs in range(16):
        xh0 = ((qh >> (iqs + 0)) << 4) & 0x10
        xh1 = (qh >> (iqs + 12)) & 0x10
        q = int(blk[off + 4 + iqs])
        v0, v1 = (q & 0xF) | xh0, (q >> 4) | xh1
        if has_m:
            y[iqs], y[iqs + 16] = hfma(H(v0), d, m), hfma(H(v1), d, m)
        else:
            y[iqs], y[iqs + 16] = hmul(H(v0) - H(16), d), hmul(H(v1) - H(16), d)
    return y


def dq_q2_k(blk):  # dequantize.cuh:101-121, 64 threads
    scales, qs = blk[0:16], blk[16:80]
    dall, dmin = f16_at(blk, 80), f16_at(blk, 82)
    y = np.zeros(256, H)
    for tid in range(64):
        n, l = tid // 32, tid % 32
        is_ = 8 * n + l // 16
        q = int(qs[32 * n + l])
        for s in range(4):
            sc = int(scales[is_ + 2 * s])
            y[128 * n + l + 32 * s] = hfma(dall, H((sc & 0xF) * ((q >> (2 * s)) & 3)), -hmul(dmin, H(sc >> 4)))
    return y


def dq_q3_k(blk):  # dequantize.cuh:123-154, 64 threads
    hm, qs, sc, d_all = blk[0:32], blk[32:96], blk[96:108], f16_at(blk, 108)
    y = np.zeros(256, H)
    for t in range(64):
        r = t // 4
        tid, is0 = r // 2, r % 2
        l0 = 16 * is0 + 4 * (t % 4)
        n, j = tid // 4, tid % 4
        m = 1 << (4 * n + j)
        is_ = 8 * n + 2 * j + is0
        shift = 2 * j
        s = [int(v) for v in sc]
        if is_ < 4:
            us = (s[is_] & 0xF) | (((s[is_ + 8] >> 0) & 3) << 4)
        elif is_ < 8:
            us = (s[is_] & 0xF) | (((s[is_ + 4] >> 2) & 3) << 4)
        elif is_ < 12:
            us = (s[is_ - 8] >> 4) | (((s[is_] >> 4) & 3) << 4)
        else:
            us = (s[is_ - 8] >> 4) | (((s[is_ - 4] >> 6) & 3) << 4)
        dl = hmul(d_all, H(us - 32))
        for l in range(l0, l0 + 4):
            q = ((int(qs[32 * n + l]) >> shift) & 3) - (0 if int(hm[l]) & m else 4)
            y[128 * n + 32 * j + l] = hmul(dl, H(q))
    return y


def scale_min_k4(j, q):  # dequantize.cuh:156-163
    if j < 4:
        return int(q[j]) & 63, int(q[j + 4]) & 63
    return (int(q[j + 4]) & 0xF) | ((int(q[j - 4]) >> 6) << 4), (int(q[j + 4]) >> 4) | ((int(q[j]) >> 6) << 4)


def dq_q5_k(blk):  # dequantize.cuh:198-230, 64 threads
    dall, dmin = f16_at(blk, 0), f16_at(blk, 2)
    scales, qh, qs = blk[4:16], blk[16:48], blk[48:176]
    y = np.zeros(256, H)
    for tid in range(64):
        il, ir = tid // 16, tid % 16
        is_ = 2 * il
        base = 64 * il + 2 * ir
        sc, m = scale_min_k4(is_, scales)
        d1, m1 = hmul(dall, H(sc)), hmul(dmin, H(m))
        sc, m = scale_min_k4(is_ + 1, scales)
        d2, m2 = hmul(dall, H(sc)), hmul(dmin, H(m))
        hm = 1 << (2 * il)
        for e in range(2):
            ql = int(qs[32 * il + 2 * ir + e])
            hb = int(qh[2 * ir + e])
            y[base + e] = hfma(d1, H((ql & 0xF) + (16 if hb & hm else 0)), -m1)
            y[base + 32 + e] = hfma(d2, H((ql >> 4) + (16 if hb & (hm << 1) else 0)), -m2)
    return y


def _grid_bytes(table, idx, n):
    v = int(table[idx])
    return [(v >> (8 * j)) & 0xFF for j in range(n)]


def dq_iq2_xs(blk):  # dequantize.cuh:277-293, 32 threads; fp32 math
    d0 = np.float32(f16_at(blk, 0))
    grid, ks = grids.iq2xs_grid(), grids.ksigns_iq2xs()
    y = np.zeros(256, np.float32)
    for tid in range(32):
        il, ib = tid // 8, tid % 8
        q2 = u16_at(blk, 2 + 2 * (4 * ib + il))
        g = _grid_bytes(grid, q2 & 511, 8)
        d = d0 * (np.float32(0.5) + np.float32((int(blk[66 + ib]) >> (4 * (il // 2))) & 0xF)) * np.float32(0.25)
        signs = int(ks[q2 >> 9])
        for j in range(8):
            y[32 * ib + 8 * il + j] = d * np.float32(g[j]) * np.float32(-1.0 if signs & KMASK[j] else 1.0)
    return y


def dq_iq2_s(blk):  # dequantize.cuh:295-309
    d0 = np.float32(f16_at(blk, 0))
    grid = grids.iq2s_grid()
    y = np.zeros(256, np.float32)
    for tid in range(32):
        il, ib = tid // 8, tid % 8
        idx = int(blk[2 + 4 * ib + il]) | ((int(blk[66 + ib]) << (8 - 2 * il)) & 0x300)
        g = _grid_bytes(grid, idx, 8)
        d = d0 * (np.float32(0.5) + np.float32((int(blk[74 + ib]) >> (4 * (il // 2))) & 0xF)) * np.float32(0.25)
        signs = int(blk[2 + 32 + 4 * ib + il])
        for j in range(8):
            y[32 * ib + 8 * il + j] = d * np.float32(g[j]) * np.float32(-1.0 if signs & KMASK[j] else 1.0)
    return y


def dq_iq3_xxs(blk):  # dequantize.cuh:311-332
    d0 = np.float32(f16_at(blk, 0))
    grid, ks = grids.iq3xxs_grid(), grids.ksigns_iq2xs()
    y = np.zeros(256, np.float32)
    for tid in range(32):
        il, ib = tid // 8, tid % 8
        q3 = blk[2 + 8 * ib:2 + 8 * ib + 8]
        aux32 = u16_at(blk, 66 + 4 * ib) | (u16_at(blk, 68 + 4 * ib) << 16)
        g1, g2 = _grid_bytes(grid, int(q3[2 * il]), 4), _grid_bytes(grid, int(q3[2 * il + 1]), 4)
        d = d0 * (np.float32(0.5) + np.float32(aux32 >> 28)) * np.float32(0.5)
        signs = int(ks[(aux32 >> (7 * il)) & 127])
        for j in range(4):
            y[32 * ib + 8 * il + j] = d * np.float32(g1[j]) * np.float32(-1.0 if signs & KMASK[j] else 1.0)
            y[32 * ib + 8 * il + j + 4] = d * np.float32(g2[j]) * np.float32(-1.0 if signs & KMASK[j + 4] else 1.0)
    return y


def dq_iq3_s(blk):  # dequantize.cuh:334-353
    d0 = np.float32(f16_at(blk, 0))
    grid = grids.iq3xs_grid()
    y = np.zeros(256, np.float32)
    for tid in range(32):
        il, ib = tid // 8, tid % 8
        qs = blk[2 + 8 * ib:2 + 8 * ib + 8]
        qh = int(blk[66 + ib])
        g1 = _grid_bytes(grid, int(qs[2 * il]) | ((qh << (8 - 2 * il)) & 256), 4)
        g2 = _grid_bytes(grid, int(qs[2 * il + 1]) | ((qh << (7 - 2 * il)) & 256), 4)
        d = d0 * (np.float32(0.5) + np.float32((int(blk[106 + ib // 2]) >> (4 * (ib % 2))) & 0xF)) * np.float32(0.5)
        signs = int(blk[74 + 4 * ib + il])
        for j in range(4):
            y[32 * ib + 8 * il + j] = d * np.float32(g1[j]) * np.float32(-1.0 if signs & KMASK[j] else 1.0)
            y[32 * ib + 8 * il + j + 4] = d * np.float32(g2[j]) * np.float32(-1.0 if signs & KMASK[j + 4] else 1.0)
    return y


def _iq1_q(grid_word):  # dequantize.cuh:368-370: even nibbles, then odd nibbles, as int8
    lo, hi = grid_word & 0x0F0F0F0F, (grid_word >> 4) & 0x0F0F0F0F
    return [(lo >> (8 * j)) & 0xFF for j in range(4)] + [(hi >> (8 * j)) & 0xFF for j in range(4)]


def dq_iq1_s(blk):  # dequantize.cuh:355-374
    d0 = np.float32(f16_at(blk, 0))
    grid = grids.iq1s_grid_gpu()
    y = np.zeros(256, np.float32)
    for tid in range(32):
        il, ib = tid // 8, tid % 8
        qh = u16_at(blk, 34 + 2 * ib)
        delta = np.float32(-1 - 0.125) if qh & 0x8000 else np.float32(-1 + 0.125)
        d = d0 * np.float32(2 * ((qh >> 12) & 7) + 1)
        q = _iq1_q(int(grid[int(blk[2 + 4 * ib + il]) | (((qh >> (3 * il)) & 7) << 8)]))
        for j in range(8):
            y[32 * ib + 8 * il + j] = d * (np.float32(q[j]) + delta)
    return y


def _iq1m_scale(blk):
    sc = [u16_at(blk, 48 + 2 * i) for i in range(4)]
    bits = (sc[0] >> 12) | ((sc[1] >> 8) & 0x00F0) | ((sc[2] >> 4) & 0x0F00) | (sc[3] & 0xF000)
    return np.array([bits], dtype=np.uint16).view(H)[0], sc


def dq_iq1_m(blk):  # dequantize.cuh:376-399
    dh, sc = _iq1m_scale(blk)
    grid = grids.iq1s_grid_gpu()
    y = np.zeros(256, np.float32)
    for tid in range(32):
        il, ib = tid // 8, tid % 8
        ib16 = 2 * ib + il // 2
        d = np.float32(dh) * np.float32(2 * ((sc[ib16 // 4] >> (3 * (ib16 % 4))) & 7) + 1)
        qh = int(blk[32 + 2 * ib + il // 2])
        delta = np.float32(-1 - 0.125) if qh & (0x08 << (4 * (il % 2))) else np.float32(-1 + 0.125)
        q = _iq1_q(int(grid[int(blk[4 * ib + il]) | (((qh >> (4 * (il % 2))) & 7) << 8)]))
        for j in range(8):
            y[32 * ib + 8 * il + j] = d * (np.float32(q[j]) + delta)
    return y


def dq_iq4_nl(blk):  # dequantize.cuh:401-418 (one 32-block)
    d = np.float32(f16_at(blk, 0))
    kv = grids.kvalues_iq4nl()
    y = np.zeros(32, np.float32)
    for il in range(4):
        for j in range(4):
            q = int(blk[2 + 4 * il + j])
            y[4 * il + j] = d * np.float32(kv[q & 0xF])
            y[4 * il + j + 16] = d * np.float32(kv[q >> 4])
    return y


DEQUANT = {
    o.Q4_1: dq_q4_1, o.Q5_0: lambda b: dq_q5(b, False), o.Q5_1: lambda b: dq_q5(b, True), o.Q2_K: dq_q2_k, o.Q3_K: dq_q3_k,
    o.Q5_K: dq_q5_k, o.IQ2_XS: dq_iq2_xs, o.IQ2_S: dq_iq2_s, o.IQ3_XXS: dq_iq3_xxs, o.IQ3_S: dq_iq3_s, o.IQ1_S: dq_iq1_s,
    o.IQ1_M: dq_iq1_m, o.IQ4_NL: dq_iq4_nl,
}


@pytest.mark.parametrize("qtype", sorted(DEQUANT))
def test_dequantize_against_thread_form(qtype):
    rng = np.random.default_rng(3000 + qtype)
    qk, bs = o.QUANT_SIZES[qtype]
    w = o.random_blocks(rng, qtype, 3, 2 * qk)                      # six blocks of arbitrary bits
    want = np.concatenate([DEQUANT[qtype](blk) for blk in w.reshape(-1, bs)])
    got16 = o.dequantize(w, qtype, "f16", "ref")
    assert np.array_equal(got16.view(np.uint16), want.astype(H).view(np.uint16)), o.TYPE_NAMES[qtype]
    if want.dtype == np.float32:                                     # i-quants: the fp32 result itself is the contract
        assert np.array_equal(o.dequantize(w, qtype, "f32", "ref").view(np.uint32), want.view(np.uint32))


# ------------------------------------------------------------------------------------------------ a8 dot products
def dp4a(a, b):
    return int(np.dot(np.asarray(a, dtype=np.int64), np.asarray(b, dtype=np.int64)))


def _f(x):
    return float(x)


def dot_q4_1(blk, q8, d8, s8, path):  # vecdotq.cuh:71-93, 573-646: half-rounded d*d8 and m*s8
    d, m = f16_at(blk, 0), f16_at(blk, 2)
    qs = blk[4:20]
    sumi = dp4a(qs & 15, q8[:16]) + dp4a(qs >> 4, q8[16:])
    return sumi * _f(hmul(d, d8)) + _f(hmul(m, s8))


def _q5_codes(blk, off):
    qh = u32_at(blk, off)
    qs = blk[off + 4:off + 20]
    lo = [(int(qs[j]) & 0xF) | (((qh >> j) & 1) << 4) for j in range(16)]
    hi = [(int(qs[j]) >> 4) | (((qh >> (j + 16)) & 1) << 4) for j in range(16)]
    return lo + hi


def dot_q5_0(blk, q8, d8, s8, path):  # MMVQ vecdotq.cuh:98-125 (unsigned codes, -16*s8); MMQ :668-749 (codes - 16, no sum)
    d = _f(f16_at(blk, 0))
    v = _q5_codes(blk, 2)
    if path == "mmvq":
        return d * (dp4a(v, q8) * _f(d8) - 16 * _f(s8))
    return d * _f(d8) * dp4a([c - 16 for c in v], q8)


def dot_q5_1(blk, q8, d8, s8, path):  # vecdotq.cuh:131-160, 179-198
    d, m = f16_at(blk, 0), f16_at(blk, 2)
    return dp4a(_q5_codes(blk, 4), q8) * _f(hmul(d, d8)) + _f(hmul(m, s8))


def dot_iq4_nl(blk, q8, d8, s8, path):  # vecdotq.cuh:1766-1788
    kv = grids.kvalues_iq4nl().astype(int)
    qs = blk[2:18]
    return _f(f16_at(blk, 0)) * _f(d8) * (dp4a(kv[qs & 15], q8[:16]) + dp4a(kv[qs >> 4], q8[16:]))


def dot_q2_k(blk, q8, d8, s8, path):  # vecdotq.cuh:204-263, 923-944: one thread per int of qs
    scales, qs = blk[0:16], blk[16:80]
    d, dmin = _f(f16_at(blk, 80)), _f(f16_at(blk, 82))
    total = 0.0
    for iqs in range(16):
        bq8 = 4 * (iqs // 8)
        so = iqs - iqs % 8 + (iqs % 8) // 4
        v = qs[4 * iqs:4 * iqs + 4]
        sd = sm = 0.0
        for i in range(4):
            sc = int(scales[so + 2 * i])
            u = q8[32 * (bq8 + i) + 4 * (iqs % 8):][:4]
            sd += _f(d8[bq8 + i]) * (dp4a((v >> (2 * i)) & 3, u) * (sc & 0xF))
            sm += _f(d8[bq8 + i]) * dp4a([sc >> 4] * 4, u)
        total += d * sd - dmin * sm
    return total


def dot_q3_k(blk, q8, d8, s8, path):  # vecdotq.cuh:269-322, 1024-1049
    hm, qs, scales = blk[0:32], blk[32:96], blk[96:108]
    d = _f(f16_at(blk, 108))
    total = 0.0
    for iqs in range(16):
        bq8 = 4 * (iqs // 8)
        so = iqs - iqs % 8 + (iqs % 8) // 4
        vl = qs[4 * iqs:4 * iqs + 4]
        vh = (~hm[4 * (iqs % 8):4 * (iqs % 8) + 4]) >> bq8          # inverted mask: 1 means "subtract 4"
        sf = 0.0
        for i in range(4):
            isc = so + 2 * i
            sc_low = (int(scales[isc % 8]) >> (4 * (isc // 8))) & 0xF
            sc_high = ((int(scales[8 + isc % 4]) >> (2 * (isc // 4))) & 3) << 4
            sc = (sc_low | sc_high) - 32
            vi = ((vl >> (2 * i)) & 3).astype(int) - (((vh >> i) << 2) & 4).astype(int)
            u = q8[32 * (bq8 + i) + 4 * (iqs % 8):][:4]
            sf += _f(d8[bq8 + i]) * (dp4a(vi, u) * sc)
        total += d * sf
    return total


def dot_q5_k(blk, q8, d8, s8, path):  # vecdotq.cuh:384-441, 1279-1323
    d, dmin = _f(f16_at(blk, 0)), _f(f16_at(blk, 2))
    scales, qh, qs = blk[4:16], blk[16:48], blk[48:176]
    total = 0.0
    for iqs in range(0, 32, 2):
        bq8 = 2 * ((iqs // 2) // 4)
        c = 4 * ((iqs // 2) % 4)
        vl = [qs[16 * bq8 + c:][:4], qs[16 * bq8 + c + 16:][:4]]
        vh = [qh[c:c + 4] >> bq8, qh[c + 16:c + 20] >> bq8]
        sc = [scale_min_k4(bq8 + i, scales) for i in range(2)]
        sd = sm = 0.0
        for i in range(2):
            v0 = ((vl[0] >> (4 * i)) & 15) | (((vh[0] >> i) & 1) << 4)
            v1 = ((vl[1] >> (4 * i)) & 15) | (((vh[1] >> i) & 1) << 4)
            u0 = q8[32 * (bq8 + i) + c:][:4]
            u1 = q8[32 * (bq8 + i) + 16 + c:][:4]
            sd += _f(d8[bq8 + i]) * ((dp4a(v0, u0) + dp4a(v1, u1)) * sc[i][0])
            if path == "mmvq":
                sm += _f(d8[bq8 + i]) * ((int(u0.astype(int).sum()) + int(u1.astype(int).sum())) * sc[i][1])
            else:  # MMQ takes the stored block sum; the four threads of a sub-block pair share it (vecdotq.cuh:415-441)
                sm += _f(s8[bq8 + i]) * sc[i][1] / 4.0
        total += d * sd - dmin * sm
    return total


def _signed_grid_dot(gbytes, signs, u):
    return sum(int(u[j]) * gbytes[j] * (-1 if signs & KMASK[j] else 1) for j in range(len(gbytes)))


def dot_iq2_xs(blk, q8, d8, s8, path):  # vecdotq.cuh:1554-1583
    grid, ks = grids.iq2xs_grid(), grids.ksigns_iq2xs()
    total = 0.0
    for ib in range(8):
        ls1, ls2 = int(blk[66 + ib]) & 0xF, int(blk[66 + ib]) >> 4
        s = [0, 0]
        for l in range(4):
            q2 = u16_at(blk, 2 + 2 * (4 * ib + l))
            s[l // 2] += _signed_grid_dot(_grid_bytes(grid, q2 & 511, 8), int(ks[q2 >> 9]), q8[32 * ib + 8 * l:])
        total += _f(f16_at(blk, 0)) * _f(d8[ib]) * 0.25 * ((0.5 + ls1) * s[0] + (0.5 + ls2) * s[1])
    return total


def dot_iq2_s(blk, q8, d8, s8, path):  # vecdotq.cuh:1585-1620
    grid = grids.iq2s_grid()
    total = 0.0
    for ib in range(8):
        ls1, ls2 = int(blk[74 + ib]) & 0xF, int(blk[74 + ib]) >> 4
        s = [0, 0]
        for l in range(4):
            idx = int(blk[2 + 4 * ib + l]) | ((int(blk[66 + ib]) << (8 - 2 * l)) & 0x300)
            s[l // 2] += _signed_grid_dot(_grid_bytes(grid, idx, 8), int(blk[34 + 4 * ib + l]), q8[32 * ib + 8 * l:])
        total += _f(f16_at(blk, 0)) * _f(d8[ib]) * 0.25 * ((0.5 + ls1) * s[0] + (0.5 + ls2) * s[1])
    return total


def dot_iq3_xxs(blk, q8, d8, s8, path):  # vecdotq.cuh:1622-1647
    grid, ks = grids.iq3xxs_grid(), grids.ksigns_iq2xs()
    total = 0.0
    for ib in range(8):
        aux = u16_at(blk, 66 + 4 * ib) | (u16_at(blk, 68 + 4 * ib) << 16)
        sumi = 0
        for l in range(4):
            g = _grid_bytes(grid, int(blk[2 + 8 * ib + 2 * l]), 4) + _grid_bytes(grid, int(blk[2 + 8 * ib + 2 * l + 1]), 4)
            sumi += _signed_grid_dot(g, int(ks[(aux >> (7 * l)) & 127]), q8[32 * ib + 8 * l:])
        total += _f(f16_at(blk, 0)) * (0.5 + (aux >> 28)) * _f(d8[ib]) * 0.5 * sumi
    return total


def dot_iq3_s(blk, q8, d8, s8, path):  # vecdotq.cuh:1649-1672
    grid = grids.iq3xs_grid()
    total = 0.0
    for ib in range(8):
        qh = int(blk[66 + ib])
        sumi = 0
        for l in range(4):
            i1 = int(blk[2 + 8 * ib + 2 * l]) | ((qh << (8 - 2 * l)) & 256)
            i2 = int(blk[2 + 8 * ib + 2 * l + 1]) | ((qh << (7 - 2 * l)) & 256)
            g = _grid_bytes(grid, i1, 4) + _grid_bytes(grid, i2, 4)
            sumi += _signed_grid_dot(g, int(blk[74 + 4 * ib + l]), q8[32 * ib + 8 * l:])
        ls = (int(blk[106 + ib // 2]) >> (4 * (ib % 2))) & 0xF
        total += _f(f16_at(blk, 0)) * (0.5 + ls) * _f(d8[ib]) * 0.5 * sumi
    return total


def dot_iq1_s(blk, q8, d8, s8, path):  # vecdotq.cuh:1674-1704: delta multiplies the stored block sum
    grid = grids.iq1s_grid_gpu()
    total = 0.0
    for ib in range(8):
        qh = u16_at(blk, 34 + 2 * ib)
        sumi = 0
        for l in range(4):
            q = _iq1_q(int(grid[int(blk[2 + 4 * ib + l]) | (((qh >> (3 * l)) & 7) << 8)]))
            sumi += dp4a(q, q8[32 * ib + 8 * l:][:8])
        d1q = _f(f16_at(blk, 0)) * (((qh >> 11) & 0x0E) + 1)
        delta = -1.0 + 0.125 - (qh & 0x8000) * (2.0 * 0.125 / 0x8000)
        total += d1q * (_f(d8[ib]) * sumi + _f(s8[ib]) * delta)
    return total


def dot_iq1_m(blk, q8, d8, s8, path):  # vecdotq.cuh:1706-1750: delta multiplies sums of eight quants
    grid = grids.iq1s_grid_gpu()
    dh, sc = _iq1m_scale(blk)
    total = 0.0
    for ib in range(8):
        sumi, sumf = [0, 0], [0.0, 0.0]
        for l in range(4):
            qhl = int(blk[32 + 2 * ib + l // 2]) >> (4 * (l % 2))
            q = _iq1_q(int(grid[int(blk[4 * ib + l]) | ((qhl & 7) << 8)]))
            u = q8[32 * ib + 8 * l:][:8]
            sumi[l // 2] += dp4a(q, u)
            delta = -1.0 + 0.125 - (qhl & 0x08) * (2.0 * 0.125 / 0x08)
            sumf[l // 2] += delta * int(u.astype(int).sum())
        tmp = sc[ib // 2] >> (6 * (ib % 2))
        sc0, sc1 = 2 * (tmp & 7) + 1, 2 * ((tmp >> 3) & 7) + 1
        total += _f(dh) * _f(d8[ib]) * ((sumi[0] + sumf[0]) * sc0 + (sumi[1] + sumf[1]) * sc1)
    return total


def dot_q2_k_mmq(blk, q8, d8, s8, path):  # vecdotq.cuh:232-263: integer sums per 16, one d8 per 32-block
    scales, qs = blk[0:16], blk[16:80]
    d, dmin = _f(f16_at(blk, 80)), _f(f16_at(blk, 82))
    codes = np.zeros(256, int)
    for n in range(2):
        for s in range(4):
            codes[128 * n + 32 * s:128 * n + 32 * s + 32] = (qs[32 * n:32 * n + 32] >> (2 * s)) & 3
    total = 0.0
    for b in range(8):
        sumi_d = sumi_m = 0
        for h in range(2):
            sc = int(scales[2 * b + h])
            u = q8[32 * b + 16 * h:32 * b + 16 * h + 16]
            sumi_d += dp4a(codes[32 * b + 16 * h:][:16], u) * (sc & 0xF)
            sumi_m += dp4a([sc >> 4] * 16, u)
        total += _f(d8[b]) * (d * sumi_d - dmin * sumi_m)
    return total


DOT = {
    o.Q4_1: dot_q4_1, o.Q5_0: dot_q5_0, o.Q5_1: dot_q5_1, o.IQ4_NL: dot_iq4_nl, o.Q2_K: dot_q2_k, o.Q3_K: dot_q3_k,
    o.Q5_K: dot_q5_k, o.IQ2_XS: dot_iq2_xs, o.IQ2_S: dot_iq2_s, o.IQ3_XXS: dot_iq3_xxs, o.IQ3_S: dot_iq3_s,
    o.IQ1_S: dot_iq1_s, o.IQ1_M: dot_iq1_m,
}
MMQ_FORMATS = [o.Q4_1, o.Q5_0, o.Q5_1, o.Q2_K, o.Q3_K, o.Q5_K]   # the reference has MMQ tiles for these (gguf_kernel.cu:236-287)


def _scalar_matmul(w, x, qtype, n, path, table):
    qk, bs = o.QUANT_SIZES[qtype]
    m, k = x.shape
    q, d8, s8 = o.quantize_q8_1(x)
    wb = w.reshape(n, k // qk, bs)
    r = qk // 32
    y = np.zeros((m, n))
    for mi in range(m):
        for ni in range(n):
            for b in range(k // qk):
                qq = q[mi, b * qk:(b + 1) * qk]
                if r == 1:
                    y[mi, ni] += table[qtype](wb[ni, b], qq, d8[mi, b], s8[mi, b], path)
                else:
                    y[mi, ni] += table[qtype](wb[ni, b], qq, d8[mi, b * r:(b + 1) * r], s8[mi, b * r:(b + 1) * r], path)
    return y


@pytest.mark.parametrize("qtype", sorted(DOT))
def test_mmvq_semantics_against_thread_form(qtype):
    rng = np.random.default_rng(4000 + qtype)
    n, k, m = 3, 768, 2      # K is not a multiple of 512: padded q8_1 columns must not matter
    w = o.make_weights(rng, qtype, n, k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    assert np.allclose(o.mul_mat_a8(w, x, qtype, n, "mmvq"), _scalar_matmul(w, x, qtype, n, "mmvq", DOT), rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("qtype", MMQ_FORMATS)
def test_mmq_semantics_against_thread_form(qtype):
    rng = np.random.default_rng(5000 + qtype)
    n, k, m = 3, 768, 2
    w = o.make_weights(rng, qtype, n, k)
    x = rng.standard_normal((m, k)).astype(np.float16)
    table = dict(DOT)
    table[o.Q2_K] = dot_q2_k_mmq
    assert np.allclose(o.mul_mat_a8(w, x, qtype, n, "mmq"), _scalar_matmul(w, x, qtype, n, "mmq", table), rtol=1e-10, atol=1e-12)
