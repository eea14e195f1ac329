"""CPU oracle for the GGUF quantized-matmul hot path.  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product never does.

It restates, in numpy, the algorithms of the reference's native extension, read
as text (paths relative to ``vllm_gguf_plugin/csrc/gguf/``):

* block layouts and codebooks ........ ``ggml-common.h:17-191`` / ``:193-1060``
* ``quantize_q8_1`` .................. ``gguf_kernel.cu:32-69``
* ``dequantize_*`` ................... ``dequantize.cuh:3-78`` and ``:101-435``
* per-format a8 dot products ......... ``vecdotq.cuh`` ``*_impl`` functions
* MMVQ / MMQ / MoE indexing .......... ``mmvq.cuh:2-41``, ``mmq.cuh:2-104``,
  ``moe.cuh:5-129``, ``moe_vec.cuh:3-53``
* MoE pipeline ....................... ``quantization/fused_moe.py:34-133``

Two dequantisation flavours exist because "bit-exact" depends on the arithmetic:

``dequantize(..., flavour="ref")``
    the rounding sequence of the reference kernels as hipcc builds them for
    gfx950: half-precision ops for standard and K quants (mul followed by
    add/sub contracts to one half ``fma``), fp32 for i-quants.
``dequantize(..., flavour="f32")``
    plain fp32 math with one final rounding (gguf-py / Triton style).

How each function is pinned (see tests/test_oracle_*.py): table hashes against
tests/golden/table_sha256.json; hand-built blocks with closed-form answers;
exhaustive sweeps of index/sign/scale spaces against direct bit descriptions;
q8_1 properties; fp64 brute force loops on tiny shapes for the matmuls and MoE;
for every format, thread-by-thread scalar restatements of the reference's
dequantize kernel and of its vec_dot function (MMVQ and MMQ semantics), written
without this module's helpers, that the vectorised code must match bit for bit
(dequantize) or to fp64 round-off (dot products).
Agreement with the third-party ``gguf.dequantize`` (gguf-py >= 0.17.0, absent
here) and with vLLM's ``moe_align_block_size`` ordering is PARITY UNPINNED.
"""
from __future__ import annotations

import numpy as np

from vllm_gguf_plugin_prism_amd.tables import grids as _g

# ggml type ids (gguf_kernel.cu:119-215) -> (elements per block, bytes per block)
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 = 2, 3, 6, 7, 8, 9
Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 10, 11, 12, 13, 14
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ4_NL, IQ3_S, IQ2_S, IQ4_XS, IQ1_M = 16, 17, 18, 19, 20, 21, 22, 23, 29

QUANT_SIZES = {
    Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34), Q8_1: (32, 36),
    Q2_K: (256, 84), Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210),
    IQ2_XXS: (256, 66), IQ2_XS: (256, 74), IQ3_XXS: (256, 98), IQ1_S: (256, 50), IQ4_NL: (32, 18),
    IQ3_S: (256, 110), IQ2_S: (256, 82), IQ4_XS: (256, 136), IQ1_M: (256, 56),
}
TYPE_NAMES = {
    Q4_0: "Q4_0", Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q8_0: "Q8_0", Q2_K: "Q2_K", Q3_K: "Q3_K",
    Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", IQ2_XXS: "IQ2_XXS", IQ2_XS: "IQ2_XS", IQ3_XXS: "IQ3_XXS",
    IQ1_S: "IQ1_S", IQ4_NL: "IQ4_NL", IQ3_S: "IQ3_S", IQ2_S: "IQ2_S", IQ4_XS: "IQ4_XS", IQ1_M: "IQ1_M",
}
HALF_MATH_TYPES = {Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K}
IQ1_DELTA = 0.125


# ----------------------------------------------------------------------------
# small helpers
# ----------------------------------------------------------------------------
def _blocks(w: np.ndarray, qtype: int) -> np.ndarray:
    bs = QUANT_SIZES[qtype][1]
    b = np.ascontiguousarray(w, dtype=np.uint8).reshape(-1)
    assert b.size % bs == 0, (b.size, bs)
    return b.reshape(-1, bs)


def _f16(b: np.ndarray, off: int) -> np.ndarray:
    """fp16 field at byte offset ``off`` of every block, as float16."""
    return np.ascontiguousarray(b[:, off:off + 2]).view("<f2").reshape(-1)


def _u16(b: np.ndarray, off: int, n: int) -> np.ndarray:
    return np.ascontiguousarray(b[:, off:off + 2 * n]).view("<u2").reshape(-1, n)


def _h(x) -> np.ndarray:
    return np.asarray(x).astype(np.float16)


def _hmul(a, b):
    # 11-bit x 11-bit products are exact in fp32, so one rounding happens.
    return (a.astype(np.float32) * b.astype(np.float32)).astype(np.float16)


def _hsub(a, b):
    return (a.astype(np.float64) - b.astype(np.float64)).astype(np.float16)


def _hadd(a, b):
    return (a.astype(np.float64) + b.astype(np.float64)).astype(np.float16)


def _hfma(a, b, c):
    # a*b is exact in fp64; the sum is exact in fp64 for all practically
    # reachable exponents, so the single rounding to half is the fma rounding.
    return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float16)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit pattern (uint16); NaN kept quiet."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = np.isnan(x)
    return np.where(nan, np.uint16(0x7FC0), rounded)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << 16).view(np.float32)


def get_scale_min_k4(scales: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """6-bit (scale, min) pairs of a K-quant 12-byte field (dequantize.cuh:156-163).

    ``scales`` is u8[nb, 12]; returns two u8[nb, 8] arrays.
    """
    q = scales.astype(np.uint8)
    sc = np.empty(q.shape[:-1] + (8,), dtype=np.uint8)
    mn = np.empty_like(sc)
    for j in range(8):
        if j < 4:
            sc[..., j] = q[..., j] & 63
            mn[..., j] = q[..., j + 4] & 63
        else:
            sc[..., j] = (q[..., j + 4] & 0xF) | ((q[..., j - 4] >> 6) << 4)
            mn[..., j] = (q[..., j + 4] >> 4) | ((q[..., j] >> 6) << 4)
    return sc, mn


# ----------------------------------------------------------------------------
# integer unpacking: every format -> (wi, ws, wmin)
#   value[k] = ws[k // group] * wi[k] - wmin[k // 32]     (exact in fp64)
# ----------------------------------------------------------------------------
def unpack(w: np.ndarray, qtype: int):
    """Return ``(wi, ws, wmin, group)`` for the packed blocks ``w``.

    ``wi``   int32[nb, qk]       integer code of every element
    ``ws``   float64[nb, qk/group] exact scale of every ``group`` elements
    ``wmin`` float64[nb, qk/32] or None, exact offset subtracted per 32 elements
    """
    b = _blocks(w, qtype)
    nb = b.shape[0]
    if qtype == Q4_0:  # ggml-common.h:17-23, dequantize.cuh:3-15
        d = _f16(b, 0).astype(np.float64)
        qs = b[:, 2:18]
        wi = np.concatenate([qs & 0xF, qs >> 4], axis=1).astype(np.int32) - 8
        return wi, d[:, None], None, 32
    if qtype == Q4_1:  # ggml-common.h:25-31, dequantize.cuh:17-30
        d = _f16(b, 0).astype(np.float64)
        m = _f16(b, 2).astype(np.float64)
        qs = b[:, 4:20]
        wi = np.concatenate([qs & 0xF, qs >> 4], axis=1).astype(np.int32)
        return wi, d[:, None], -m[:, None], 32
    if qtype in (Q5_0, Q5_1):  # ggml-common.h:33-49, dequantize.cuh:32-67
        off = 2 if qtype == Q5_0 else 4
        d = _f16(b, 0).astype(np.float64)
        qh = np.ascontiguousarray(b[:, off:off + 4]).view("<u4").reshape(-1)
        qs = b[:, off + 4:off + 20]
        j = np.arange(16, dtype=np.uint32)
        h0 = ((qh[:, None] >> j) & 1).astype(np.int32) << 4
        h1 = ((qh[:, None] >> (j + 16)) & 1).astype(np.int32) << 4
        wi = np.concatenate([(qs & 0xF).astype(np.int32) | h0, (qs >> 4).astype(np.int32) | h1], axis=1)
        if qtype == Q5_0:
            return wi - 16, d[:, None], None, 32
        m = _f16(b, 2).astype(np.float64)
        return wi, d[:, None], -m[:, None], 32
    if qtype == Q8_0:  # ggml-common.h:51-57, dequantize.cuh:69-78
        d = _f16(b, 0).astype(np.float64)
        wi = b[:, 2:34].view(np.int8).astype(np.int32)
        return wi, d[:, None], None, 32
    if qtype == Q2_K:  # ggml-common.h:67-73, dequantize.cuh:101-121
        scales = b[:, 0:16]
        qs = b[:, 16:80]
        d = _f16(b, 80).astype(np.float64)
        dmin = _f16(b, 82).astype(np.float64)
        wi = np.empty((nb, 256), dtype=np.int32)
        for n in range(2):
            for sh in range(4):
                wi[:, 128 * n + 32 * sh:128 * n + 32 * sh + 32] = (qs[:, 32 * n:32 * n + 32] >> (2 * sh)) & 3
        ws = d[:, None] * (scales & 0xF).astype(np.float64)          # per 16
        wmin16 = dmin[:, None] * (scales >> 4).astype(np.float64)    # per 16
        return wi, ws, wmin16, 16
    if qtype == Q3_K:  # ggml-common.h:75-82, dequantize.cuh:123-154
        hm = b[:, 0:32]
        qs = b[:, 32:96]
        sc = b[:, 96:108].astype(np.int32)
        d = _f16(b, 108).astype(np.float64)
        us = np.empty((nb, 16), dtype=np.int32)
        for i in range(16):
            if i < 4:
                us[:, i] = (sc[:, i] & 0xF) | (((sc[:, i + 8] >> 0) & 3) << 4)
            elif i < 8:
                us[:, i] = (sc[:, i] & 0xF) | (((sc[:, i + 4] >> 2) & 3) << 4)
            elif i < 12:
                us[:, i] = (sc[:, i - 8] >> 4) | (((sc[:, i] >> 4) & 3) << 4)
            else:
                us[:, i] = (sc[:, i - 8] >> 4) | (((sc[:, i - 4] >> 6) & 3) << 4)
        wi = np.empty((nb, 256), dtype=np.int32)
        for n in range(2):
            for j in range(4):
                low = ((qs[:, 32 * n:32 * n + 32] >> (2 * j)) & 3).astype(np.int32)
                hb = (hm >> (4 * n + j)) & 1
                wi[:, 128 * n + 32 * j:128 * n + 32 * j + 32] = low - np.where(hb != 0, 0, 4)
        return wi, d[:, None] * (us - 32).astype(np.float64), None, 16
    if qtype in (Q4_K, Q5_K):  # ggml-common.h:84-99, dequantize.cuh:165-230
        d = _f16(b, 0).astype(np.float64)
        dmin = _f16(b, 2).astype(np.float64)
        sc, mn = get_scale_min_k4(b[:, 4:16])
        if qtype == Q4_K:
            qs = b[:, 16:144]
            qh = None
        else:
            qh = b[:, 16:48]
            qs = b[:, 48:176]
        wi = np.empty((nb, 256), dtype=np.int32)
        for g in range(4):
            chunk = qs[:, 32 * g:32 * g + 32]
            lo = (chunk & 0xF).astype(np.int32)
            hi = (chunk >> 4).astype(np.int32)
            if qh is not None:
                lo += (((qh >> (2 * g)) & 1).astype(np.int32)) << 4
                hi += (((qh >> (2 * g + 1)) & 1).astype(np.int32)) << 4
            wi[:, 64 * g:64 * g + 32] = lo
            wi[:, 64 * g + 32:64 * g + 64] = hi
        return wi, d[:, None] * sc.astype(np.float64), dmin[:, None] * mn.astype(np.float64), 32
    if qtype == Q6_K:  # ggml-common.h:101-108, dequantize.cuh:232-256
        ql = b[:, 0:128]
        qh = b[:, 128:192]
        sc = b[:, 192:208].view(np.int8).astype(np.float64)
        d = _f16(b, 208).astype(np.float64)
        wi = np.empty((nb, 256), dtype=np.int32)
        for h in range(2):
            l0 = ql[:, 64 * h:64 * h + 32]
            l1 = ql[:, 64 * h + 32:64 * h + 64]
            hh = qh[:, 32 * h:32 * h + 32]
            base = 128 * h
            wi[:, base + 0:base + 32] = ((l0 & 0xF) | (((hh >> 0) & 3) << 4)).astype(np.int32) - 32
            wi[:, base + 32:base + 64] = ((l1 & 0xF) | (((hh >> 2) & 3) << 4)).astype(np.int32) - 32
            wi[:, base + 64:base + 96] = ((l0 >> 4) | (((hh >> 4) & 3) << 4)).astype(np.int32) - 32
            wi[:, base + 96:base + 128] = ((l1 >> 4) | (((hh >> 6) & 3) << 4)).astype(np.int32) - 32
        return wi, d[:, None] * sc, None, 16
    if qtype == IQ4_NL:  # ggml-common.h:176-182, dequantize.cuh:401-418
        d = _f16(b, 0).astype(np.float64)
        qs = b[:, 2:18]
        kv = _g.kvalues_iq4nl().astype(np.int32)
        wi = np.concatenate([kv[qs & 0xF], kv[qs >> 4]], axis=1)
        return wi, d[:, None], None, 32
    if qtype == IQ4_XS:  # ggml-common.h:184-191, dequantize.cuh:420-435
        d = _f16(b, 0).astype(np.float64)
        sh = _u16(b, 2, 1)[:, 0].astype(np.int32)
        sl = b[:, 4:8].astype(np.int32)
        qs = b[:, 8:136]
        kv = _g.kvalues_iq4nl().astype(np.int32)
        wi = np.empty((nb, 256), dtype=np.int32)
        ls = np.empty((nb, 8), dtype=np.int32)
        for ib in range(8):
            ls[:, ib] = ((sl[:, ib // 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4)
            chunk = qs[:, 16 * ib:16 * ib + 16]
            wi[:, 32 * ib:32 * ib + 16] = kv[chunk & 0xF]
            wi[:, 32 * ib + 16:32 * ib + 32] = kv[chunk >> 4]
        return wi, d[:, None] * (ls - 32).astype(np.float64), None, 32
    if qtype in (IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S, IQ1_S, IQ1_M):
        return _unpack_grid_quants(b, qtype)
    raise ValueError(f"unsupported ggml type {qtype}")


def _signs8(sign_bytes: np.ndarray) -> np.ndarray:
    """u8[...] -> int32[..., 8] of +1/-1 (bit j set -> -1), kmask_iq2xs = 1<<j."""
    j = np.arange(8, dtype=np.uint8)
    return 1 - 2 * ((sign_bytes[..., None] >> j) & 1).astype(np.int32)


def _unpack_grid_quants(b: np.ndarray, qtype: int):
    nb = b.shape[0]
    d = _f16(b, 0).astype(np.float64)
    wi = np.empty((nb, 256), dtype=np.int32)
    if qtype == IQ2_XXS:  # ggml-common.h:110-115, dequantize.cuh:258-275
        grid = _g.grid_bytes(_g.iq2xxs_grid()).astype(np.int32)
        ks = _g.ksigns_iq2xs()
        q2 = b[:, 2:66].reshape(nb, 8, 8)
        aux = np.ascontiguousarray(q2[:, :, 4:8]).view("<u4").reshape(nb, 8)
        ws = d[:, None] * (0.5 + (aux >> 28).astype(np.float64)) * 0.25
        for l in range(4):
            g8 = grid[q2[:, :, l]]                                  # [nb, 8, 8]
            s8 = _signs8(ks[(aux >> (7 * l)) & 127])
            wi.reshape(nb, 8, 32)[:, :, 8 * l:8 * l + 8] = g8 * s8
        return wi, ws, None, 32
    if qtype == IQ2_XS:  # ggml-common.h:117-123, dequantize.cuh:277-293
        grid = _g.grid_bytes(_g.iq2xs_grid()).astype(np.int32)
        ks = _g.ksigns_iq2xs()
        q2 = _u16(b, 2, 32).reshape(nb, 8, 4)
        scales = b[:, 66:74]
        ws = np.empty((nb, 16), dtype=np.float64)
        for l in range(4):
            wi.reshape(nb, 8, 32)[:, :, 8 * l:8 * l + 8] = grid[q2[:, :, l] & 511] * _signs8(ks[q2[:, :, l] >> 9])
        ws[:, 0::2] = d[:, None] * (0.5 + (scales & 0xF).astype(np.float64)) * 0.25
        ws[:, 1::2] = d[:, None] * (0.5 + (scales >> 4).astype(np.float64)) * 0.25
        return wi, ws, None, 16
    if qtype == IQ2_S:  # ggml-common.h:125-132, dequantize.cuh:295-309
        grid = _g.grid_bytes(_g.iq2s_grid()).astype(np.int32)
        qs = b[:, 2:34].reshape(nb, 8, 4).astype(np.int32)
        signs = b[:, 34:66].reshape(nb, 8, 4)
        qh = b[:, 66:74].astype(np.int32)
        scales = b[:, 74:82]
        ws = np.empty((nb, 16), dtype=np.float64)
        for l in range(4):
            idx = qs[:, :, l] | ((qh << (8 - 2 * l)) & 0x300)
            wi.reshape(nb, 8, 32)[:, :, 8 * l:8 * l + 8] = grid[idx] * _signs8(signs[:, :, l])
        ws[:, 0::2] = d[:, None] * (0.5 + (scales & 0xF).astype(np.float64)) * 0.25
        ws[:, 1::2] = d[:, None] * (0.5 + (scales >> 4).astype(np.float64)) * 0.25
        return wi, ws, None, 16
    if qtype == IQ3_XXS:  # ggml-common.h:134-139, dequantize.cuh:311-332
        grid = _g.grid_bytes(_g.iq3xxs_grid()).astype(np.int32)
        ks = _g.ksigns_iq2xs()
        q3 = b[:, 2:66].reshape(nb, 8, 8)
        aux = np.ascontiguousarray(b[:, 66:98]).view("<u4").reshape(nb, 8)
        ws = d[:, None] * (0.5 + (aux >> 28).astype(np.float64)) * 0.5
        for l in range(4):
            s8 = _signs8(ks[(aux >> (7 * l)) & 127])
            g8 = np.concatenate([grid[q3[:, :, 2 * l]], grid[q3[:, :, 2 * l + 1]]], axis=-1)
            wi.reshape(nb, 8, 32)[:, :, 8 * l:8 * l + 8] = g8 * s8
        return wi, ws, None, 32
    if qtype == IQ3_S:  # ggml-common.h:141-150, dequantize.cuh:334-353
        grid = _g.grid_bytes(_g.iq3xs_grid()).astype(np.int32)
        qs = b[:, 2:66].reshape(nb, 8, 8).astype(np.int32)
        qh = b[:, 66:74].astype(np.int32)
        signs = b[:, 74:106].reshape(nb, 8, 4)
        scales = b[:, 106:110]
        ls = np.empty((nb, 8), dtype=np.float64)
        for ib in range(8):
            ls[:, ib] = (scales[:, ib // 2] >> (4 * (ib % 2))) & 0xF
        ws = d[:, None] * (0.5 + ls) * 0.5
        for l in range(4):
            i1 = qs[:, :, 2 * l] | ((qh << (8 - 2 * l)) & 256)
            i2 = qs[:, :, 2 * l + 1] | ((qh << (7 - 2 * l)) & 256)
            g8 = np.concatenate([grid[i1], grid[i2]], axis=-1)
            wi.reshape(nb, 8, 32)[:, :, 8 * l:8 * l + 8] = g8 * _signs8(signs[:, :, l])
        return wi, ws, None, 32
    raise ValueError(f"ggml type {qtype}: delta-shifted 1-bit grids have no integer form; use dequantize()")


# ----------------------------------------------------------------------------
# dequantize
# ----------------------------------------------------------------------------
def dequant_exact(w: np.ndarray, qtype: int) -> np.ndarray:
    """Exact (unrounded) block values as float64[nb*qk]."""
    if qtype in (IQ1_S, IQ1_M):
        return _dequant_iq1(_blocks(w, qtype), qtype).astype(np.float64).reshape(-1)
    wi, ws, wmin, group = unpack(w, qtype)
    v = np.repeat(ws, group, axis=1) * wi
    if wmin is not None:
        v = v - np.repeat(wmin, wi.shape[1] // wmin.shape[1], axis=1)
    return v.reshape(-1)


def _dequant_iq1(b: np.ndarray, qtype: int) -> np.ndarray:
    """IQ1_S / IQ1_M in the reference's fp32 op order (dequantize.cuh:355-399)."""
    nb = b.shape[0]
    grid = _g.iq1s_grid_gpu().astype(np.uint32)
    out = np.empty((nb, 8, 4, 8), dtype=np.float32)
    if qtype == IQ1_S:  # ggml-common.h:153-159
        dd = _f16(b, 0).astype(np.float32)
        qs = b[:, 2:34].reshape(nb, 8, 4).astype(np.uint32)
        qh = _u16(b, 34, 8).astype(np.uint32)
        delta = np.where((qh & 0x8000) != 0, np.float32(-1 - IQ1_DELTA), np.float32(-1 + IQ1_DELTA))
        dl = dd[:, None] * (2 * ((qh >> 12) & 7) + 1).astype(np.float32)
        for il in range(4):
            gi = grid[qs[:, :, il] | (((qh >> (3 * il)) & 7) << 8)]
            lo = gi & 0x0F0F0F0F
            hi = (gi >> 4) & 0x0F0F0F0F
            for j in range(4):
                out[:, :, il, j] = dl * (((lo >> (8 * j)) & 0xFF).astype(np.float32) + delta)
                out[:, :, il, 4 + j] = dl * (((hi >> (8 * j)) & 0xFF).astype(np.float32) + delta)
        return out.reshape(nb, 256)
    # IQ1_M, ggml-common.h:162-174
    qs = b[:, 0:32].reshape(nb, 8, 4).astype(np.uint32)
    qh = b[:, 32:48].astype(np.uint32)
    sc = _u16(b, 48, 4).astype(np.uint32)
    scale_bits = ((sc[:, 0] >> 12) | ((sc[:, 1] >> 8) & 0x00F0) | ((sc[:, 2] >> 4) & 0x0F00) | (sc[:, 3] & 0xF000)).astype(np.uint16)
    dd = scale_bits.view(np.float16).astype(np.float32)
    for ib in range(8):
        for il in range(4):
            ib16 = 2 * ib + il // 2
            dl = dd * (2 * ((sc[:, ib16 // 4] >> (3 * (ib16 % 4))) & 7) + 1).astype(np.float32)
            qhb = qh[:, 2 * ib + il // 2]
            delta = np.where((qhb & (0x08 << (4 * (il % 2)))) != 0, np.float32(-1 - IQ1_DELTA), np.float32(-1 + IQ1_DELTA))
            gi = grid[qs[:, ib, il] | (((qhb >> (4 * (il % 2))) & 7) << 8)]
            lo = gi & 0x0F0F0F0F
            hi = (gi >> 4) & 0x0F0F0F0F
            for j in range(4):
                out[:, ib, il, j] = dl * (((lo >> (8 * j)) & 0xFF).astype(np.float32) + delta)
                out[:, ib, il, 4 + j] = dl * (((hi >> (8 * j)) & 0xFF).astype(np.float32) + delta)
    return out.reshape(nb, 256)


def _dequant_ref_half(w: np.ndarray, qtype: int, contract: bool) -> np.ndarray:
    """Half-precision op sequences of the standard and K-quant kernels -> float16[nb*qk]."""
    b = _blocks(w, qtype)
    wi, _, _, _ = unpack(w, qtype)
    nb = b.shape[0]
    if qtype in (Q4_0, Q5_0):  # (q - 8|16) in half (exact), then one hmul (dequantize.cuh:13-14,46-47)
        d = _f16(b, 0)
        return _hmul(_h(wi), d[:, None]).reshape(-1)
    if qtype == Q8_0:  # dequantize.cuh:74-77
        d = _f16(b, 0)
        return _hmul(_h(wi), d[:, None]).reshape(-1)
    if qtype in (Q4_1, Q5_1):  # hmul then hadd (dequantize.cuh:28-29,65-66)
        d = _f16(b, 0)[:, None]
        m = _f16(b, 2)[:, None]
        if contract:
            return _hfma(_h(wi), d, m).reshape(-1)
        return _hadd(_hmul(_h(wi), d), m).reshape(-1)
    if qtype == Q2_K:  # dequantize.cuh:115-120: hsub(hmul(dall, half(sc*q)), hmul(dmin, half(m)))
        scales = b[:, 0:16]
        dall = _f16(b, 80)[:, None]
        dmin = _f16(b, 82)[:, None]
        scq = _h(np.repeat((scales & 0xF).astype(np.int32), 16, axis=1) * wi)
        m1 = np.repeat(_hmul(dmin, _h(scales >> 4)), 16, axis=1)
        if contract:
            return _hfma(dall, scq, -m1).reshape(-1)
        return _hsub(_hmul(dall, scq), m1).reshape(-1)
    if qtype == Q3_K:  # dequantize.cuh:144-152: dl = hmul(d, half(us-32)); hmul(dl, half(q))
        d = _f16(b, 108)[:, None]
        sc = b[:, 96:108].astype(np.int32)
        us = np.empty((nb, 16), dtype=np.int32)
        for i in range(16):
            if i < 4:
                us[:, i] = (sc[:, i] & 0xF) | (((sc[:, i + 8] >> 0) & 3) << 4)
            elif i < 8:
                us[:, i] = (sc[:, i] & 0xF) | (((sc[:, i + 4] >> 2) & 3) << 4)
            elif i < 12:
                us[:, i] = (sc[:, i - 8] >> 4) | (((sc[:, i] >> 4) & 3) << 4)
            else:
                us[:, i] = (sc[:, i - 8] >> 4) | (((sc[:, i - 4] >> 6) & 3) << 4)
        dl = np.repeat(_hmul(d, _h(us - 32)), 16, axis=1)
        return _hmul(dl, _h(wi)).reshape(-1)
    if qtype in (Q4_K, Q5_K):  # dequantize.cuh:187-194,220-229
        dall = _f16(b, 0)[:, None]
        dmin = _f16(b, 2)[:, None]
        sc, mn = get_scale_min_k4(b[:, 4:16])
        d1 = np.repeat(_hmul(dall, _h(sc)), 32, axis=1)
        m1 = np.repeat(_hmul(dmin, _h(mn)), 32, axis=1)
        if contract:
            return _hfma(d1, _h(wi), -m1).reshape(-1)
        return _hsub(_hmul(d1, _h(wi)), m1).reshape(-1)
    if qtype == Q6_K:  # dequantize.cuh:252-255: hmul(d, int2half_rn(sc * (q - 32)))
        sc = b[:, 192:208].view(np.int8).astype(np.int32)
        d = _f16(b, 208)[:, None]
        prod = np.repeat(sc, 16, axis=1) * wi
        return _hmul(d, prod.astype(np.float32).astype(np.float16)).reshape(-1)
    raise ValueError(qtype)


def _dequant_ref_f32(w: np.ndarray, qtype: int) -> np.ndarray:
    """fp32 op sequences of the i-quant kernels -> float32[nb*qk] (dequantize.cuh:258-435)."""
    b = _blocks(w, qtype)
    if qtype in (IQ1_S, IQ1_M):
        return _dequant_iq1(b, qtype).reshape(-1)
    wi, _, _, _ = unpack(w, qtype)
    nb = b.shape[0]
    d = _f16(b, 0).astype(np.float32)[:, None]
    one = np.float32
    if qtype == IQ4_NL:
        return (d * wi.astype(np.float32)).reshape(-1)
    if qtype == IQ4_XS:
        sh = _u16(b, 2, 1)[:, 0].astype(np.int32)
        sl = b[:, 4:8].astype(np.int32)
        ls = np.stack([((sl[:, ib // 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4) for ib in range(8)], axis=1)
        dl = d * (ls - 32).astype(np.float32)
        return (np.repeat(dl, 32, axis=1) * wi.astype(np.float32)).reshape(-1)
    if qtype in (IQ2_XXS, IQ3_XXS):
        if qtype == IQ2_XXS:
            q2 = b[:, 2:66].reshape(nb, 8, 8)
            aux = np.ascontiguousarray(q2[:, :, 4:8]).view("<u4").reshape(nb, 8)
            fac = one(0.25)
        else:
            aux = np.ascontiguousarray(b[:, 66:98]).view("<u4").reshape(nb, 8)
            fac = one(0.5)
        db = d * (one(0.5) + (aux >> 28).astype(np.float32)) * fac
        # y = d * grid * sign: magnitude and sign folded in wi; |wi| small so products are exact
        return (np.repeat(db, 32, axis=1) * wi.astype(np.float32)).reshape(-1)
    if qtype in (IQ2_XS, IQ2_S):
        scales = b[:, 66:74] if qtype == IQ2_XS else b[:, 74:82]
        db = np.empty((nb, 16), dtype=np.float32)
        db[:, 0::2] = d * (one(0.5) + (scales & 0xF).astype(np.float32)) * one(0.25)
        db[:, 1::2] = d * (one(0.5) + (scales >> 4).astype(np.float32)) * one(0.25)
        return (np.repeat(db, 16, axis=1) * wi.astype(np.float32)).reshape(-1)
    if qtype == IQ3_S:
        scales = b[:, 106:110]
        ls = np.stack([(scales[:, ib // 2] >> (4 * (ib % 2))) & 0xF for ib in range(8)], axis=1)
        db = d * (one(0.5) + ls.astype(np.float32)) * one(0.5)
        return (np.repeat(db, 32, axis=1) * wi.astype(np.float32)).reshape(-1)
    raise ValueError(qtype)


def dequantize(w: np.ndarray, qtype: int, out_dtype: str = "f16", flavour: str = "ref", contract: bool = True) -> np.ndarray:
    """Dense values of the packed tensor ``w``.

    ``out_dtype``: "f16" -> float16, "f32" -> float32, "bf16" -> uint16 bit patterns.
    ``flavour``:   "ref" (reference rounding sequence) or "f32" (one rounding from exact).
    ``contract``:  for "ref", whether mul+add/sub chains round once (hipcc's default).
    """
    if flavour == "f32":
        v32 = dequant_exact(w, qtype).astype(np.float32) if qtype not in (IQ1_S, IQ1_M) else _dequant_ref_f32(w, qtype)
        if out_dtype == "f32":
            return v32
        if out_dtype == "f16":
            return dequant_exact(w, qtype).astype(np.float16) if qtype not in (IQ1_S, IQ1_M) else v32.astype(np.float16)
        return f32_to_bf16_bits(v32)
    if qtype in HALF_MATH_TYPES:
        h = _dequant_ref_half(w, qtype, contract)
        if out_dtype == "f16":
            return h
        if out_dtype == "f32":
            return h.astype(np.float32)
        return f32_to_bf16_bits(h.astype(np.float32))
    v = _dequant_ref_f32(w, qtype)
    if out_dtype == "f32":
        return v
    if out_dtype == "f16":
        return v.astype(np.float16)
    return f32_to_bf16_bits(v)


# ----------------------------------------------------------------------------
# q8_1 activation quantizer (gguf_kernel.cu:32-69)
# ----------------------------------------------------------------------------
def quantize_q8_1(x: np.ndarray):
    """Quantize rows of ``x`` ([M, K] float16/float32, or bf16 given as float32).

    Returns ``(q, d, s)``: int8[M, Kp], float16[M, Kp/32] scales, float16[M, Kp/32]
    block sums, with Kp = K rounded up to 512 and columns [K, Kp) treated as zero.
    """
    x = np.asarray(x)
    m, k = x.shape
    kp = (k + 511) // 512 * 512
    xf = np.zeros((m, kp), dtype=np.float32)
    xf[:, :k] = x.astype(np.float32)
    blk = xf.reshape(m, kp // 32, 32)
    amax = np.abs(blk).max(axis=2)
    s = blk.copy()
    idx = np.arange(32)
    for mask in (16, 8, 4, 2, 1):  # xor butterfly: every lane ends with the same fp32 tree sum
        s = s + s[:, :, idx ^ mask]
    ssum = s[:, :, 0]
    d = (amax / np.float32(127)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = (blk / d[:, :, None]).astype(np.float32)
    t = np.trunc(v)
    r = t + np.copysign(np.float32(1), v) * (np.abs(v - t) >= np.float32(0.5))  # roundf: ties away from zero
    q = np.where(amax[:, :, None] == 0, 0, r).astype(np.int8)
    return q.reshape(m, kp), d.astype(np.float16), ssum.astype(np.float16)


def dequant_q8_1(q: np.ndarray, d: np.ndarray) -> np.ndarray:
    """Exact float64 values d*q of quantized activations."""
    m, kp = q.shape
    return (q.reshape(m, kp // 32, 32).astype(np.float64) * d.astype(np.float64)[:, :, None]).reshape(m, kp)


# ----------------------------------------------------------------------------
# a8 matmuls: per-format reference formula evaluated in fp64
# ----------------------------------------------------------------------------
def _iq1_dot_terms(w: np.ndarray, qtype: int, n: int, k: int):
    """IQ1_S / IQ1_M as (integer grid part, per-8 delta part) (vecdotq.cuh:1674-1750)."""
    b = _blocks(w, qtype)
    nb = b.shape[0]
    grid = _g.iq1s_grid_gpu().astype(np.uint32)
    gq = np.empty((nb, 8, 4, 8), dtype=np.float64)
    if qtype == IQ1_S:
        dd = _f16(b, 0).astype(np.float64)
        qs = b[:, 2:34].reshape(nb, 8, 4).astype(np.uint32)
        qh = _u16(b, 34, 8).astype(np.uint32)
        scale32 = dd[:, None] * (2 * ((qh >> 12) & 7) + 1).astype(np.float64)      # [nb, 8] per 32
        delta32 = np.where((qh & 0x8000) != 0, -1 - IQ1_DELTA, -1 + IQ1_DELTA).astype(np.float64)
        for il in range(4):
            gi = grid[qs[:, :, il] | (((qh >> (3 * il)) & 7) << 8)]
            for j in range(4):
                gq[:, :, il, j] = ((gi >> (8 * j)) & 0xF)
                gq[:, :, il, 4 + j] = ((gi >> (8 * j + 4)) & 0xF)
        scale8 = np.repeat(scale32, 4, axis=1)
        delta8 = np.repeat(delta32, 4, axis=1)
    else:
        qs = b[:, 0:32].reshape(nb, 8, 4).astype(np.uint32)
        qh = b[:, 32:48].astype(np.uint32)
        sc = _u16(b, 48, 4).astype(np.uint32)
        bits = ((sc[:, 0] >> 12) | ((sc[:, 1] >> 8) & 0x00F0) | ((sc[:, 2] >> 4) & 0x0F00) | (sc[:, 3] & 0xF000)).astype(np.uint16)
        dd = bits.view(np.float16).astype(np.float64)
        scale8 = np.empty((nb, 32), dtype=np.float64)
        delta8 = np.empty((nb, 32), dtype=np.float64)
        for ib in range(8):
            for il in range(4):
                ib16 = 2 * ib + il // 2
                scale8[:, 4 * ib + il] = dd * (2 * ((sc[:, ib16 // 4] >> (3 * (ib16 % 4))) & 7) + 1)
                qhb = qh[:, 2 * ib + il // 2]
                delta8[:, 4 * ib + il] = np.where((qhb & (0x08 << (4 * (il % 2)))) != 0, -1 - IQ1_DELTA, -1 + IQ1_DELTA)
                gi = grid[qs[:, ib, il] | (((qhb >> (4 * (il % 2))) & 7) << 8)]
                for j in range(4):
                    gq[:, ib, il, j] = ((gi >> (8 * j)) & 0xF)
                    gq[:, ib, il, 4 + j] = ((gi >> (8 * j + 4)) & 0xF)
    wgrid = (gq.reshape(nb, 32, 8) * scale8[:, :, None]).reshape(n, k)
    return wgrid, (scale8 * delta8).reshape(n, k // 8), scale8.reshape(n, k // 8)


def mul_mat_a8(w: np.ndarray, x: np.ndarray, qtype: int, n: int, path: str = "mmvq") -> np.ndarray:
    """``Y[m, n] = W[n, :] . q8_1(X[m, :])`` in fp64, per-format reference formula.

    ``path`` selects which block "sum" the offset term uses where the two
    reference paths differ (vecdotq.cuh:328-351 vs :353-379): "mmvq" or "mmq".
    """
    assert path in ("mmvq", "mmq")
    x = np.asarray(x)
    m, k = x.shape
    q, d8, s8 = quantize_q8_1(x)
    xh = dequant_q8_1(q, d8)[:, :k]
    nb32 = k // 32
    d8f = d8.astype(np.float64)[:, :nb32]
    s8f = s8.astype(np.float64)[:, :nb32]
    usum = q.reshape(m, -1, 32).astype(np.float64).sum(axis=2)[:, :nb32]

    if qtype in (IQ1_S, IQ1_M):
        wgrid, sdelta, scale8 = _iq1_dot_terms(w, qtype, n, k)
        y = xh @ wgrid.T
        if qtype == IQ1_S:
            # d1q * (ds.x*sumi + ds.y*delta): the delta term uses the stored half block sum
            sd32 = sdelta.reshape(n, nb32, 4)[:, :, 0]
            return y + s8f @ sd32.T
        # IQ1_M: delta * sum(u) computed from the quants, per 8 elements
        u8 = q.reshape(m, -1, 8).astype(np.float64).sum(axis=2)[:, :k // 8] * np.repeat(d8f, 4, axis=1)
        return y + u8 @ sdelta.T

    wi, ws, wmin, group = unpack(w, qtype)
    wv = (np.repeat(ws, group, axis=1) * wi).reshape(n, k)
    if qtype == Q4_0 or (qtype == Q5_0 and path == "mmvq"):
        # d*(sumi*d8 - (8|16)*s8): integer part uses the unsigned code (vecdotq.cuh:46-66,98-125).
        # The Q5_0 MMQ tiles subtract 16 from the codes instead (vecdotq.cuh:700,709,747).
        off = 8 if qtype == Q4_0 else 16
        wv_u = (np.repeat(ws, group, axis=1) * (wi + off)).reshape(n, k)
        return xh @ wv_u.T - off * (s8f @ ws.reshape(n, nb32).T)
    y = xh @ wv.T
    if wmin is None:
        return y
    if qtype in (Q4_1, Q5_1):
        # sumi*d*d8 + m*s8 with hmul2(dm, ds8): both products rounded to half (vecdotq.cuh:86-91)
        b = _blocks(w, qtype)
        dh = _f16(b, 0).reshape(n, nb32)
        mh = _f16(b, 2).reshape(n, nb32)
        wi_mat = wi.reshape(n, nb32, 32).astype(np.float64)
        qb = q[:, :k].reshape(m, nb32, 32).astype(np.float64)
        sumi = np.einsum("mbk,nbk->mnb", qb, wi_mat)
        d4d8 = _hmul(np.broadcast_to(dh[None], (m, n, nb32)), np.broadcast_to(d8[:, None, :nb32], (m, n, nb32))).astype(np.float64)
        m4s8 = _hmul(np.broadcast_to(mh[None], (m, n, nb32)), np.broadcast_to(s8[:, None, :nb32], (m, n, nb32))).astype(np.float64)
        return (sumi * d4d8 + m4s8).sum(axis=2)
    per = wmin.shape[1] * 32 // wi.shape[1]  # wmin entries per 32 elements (1, or 2 for Q2_K)
    if per == 1:
        wm = wmin.reshape(n, nb32)
        if path == "mmq":  # Q4_K / Q5_K MMQ: dmin * m * s8 (vecdotq.cuh:369-372)
            return y - s8f @ wm.T
        return y - (d8f * usum) @ wm.T
    # Q2_K: mins per 16 elements, sum(u) over each 16 (vecdotq.cuh:204-263)
    u16 = q.reshape(m, -1, 16).astype(np.float64).sum(axis=2)[:, :k // 16] * np.repeat(d8f, 2, axis=1)
    return y - u16 @ wmin.reshape(n, k // 16).T


def mul_mat_f32(w: np.ndarray, x: np.ndarray, qtype: int, n: int) -> np.ndarray:
    """Unquantized-activation oracle: fp32 dequant, then an fp32 matmul accumulated in fp64."""
    k = x.shape[1]
    wd = dequantize(w, qtype, "f32", flavour="f32").reshape(n, k)
    return np.asarray(x, dtype=np.float64) @ wd.astype(np.float64).T


# ----------------------------------------------------------------------------
# MoE
# ----------------------------------------------------------------------------
def moe_align_block_size(topk_ids: np.ndarray, block_size: int, num_experts: int):
    """Restatement of vLLM's ``moe_align_block_size`` contract (not in the reference tree).

    Returns ``(sorted_token_ids, expert_ids, num_tokens_post_padded)`` as int32
    arrays: flat pair indices grouped by expert, every group padded to a
    multiple of ``block_size`` with the sentinel ``topk_ids.size``; one expert id
    per block; and the padded total.  The order inside a group is ascending
    pair index (any order is valid for the consumer).
    """
    flat = np.asarray(topk_ids, dtype=np.int64).reshape(-1)
    numel = flat.size
    max_padded = numel + num_experts * (block_size - 1)
    max_padded = (max_padded + block_size - 1) // block_size * block_size
    sorted_ids = np.full(max_padded, numel, dtype=np.int32)
    expert_ids = np.full(max_padded // block_size, -1, dtype=np.int32)
    pos = 0
    for e in range(num_experts):
        idx = np.nonzero(flat == e)[0]
        if idx.size == 0:
            continue
        sorted_ids[pos:pos + idx.size] = idx
        padded = (idx.size + block_size - 1) // block_size * block_size
        expert_ids[pos // block_size:(pos + padded) // block_size] = e
        pos += padded
    return sorted_ids, expert_ids, np.array([pos], dtype=np.int32)


def moe_a8(x, w, sorted_token_ids, expert_ids, num_tokens_post_padded, qtype, n, top_k, tokens, block_size):
    """Grouped a8 matmul (moe.cuh:5-129): ``Y[p, :] = W[e] . q8_1(X[p // top_k])`` for every
    non-padding slot p of every block below the padded count; untouched rows stay zero."""
    x = np.asarray(x)
    wflat = w.reshape(w.shape[0], -1)
    y = np.zeros((tokens * top_k, n), dtype=np.float64)
    npost = int(num_tokens_post_padded[0])
    cache: dict[int, list[int]] = {}
    for blk in range(len(sorted_token_ids) // block_size):
        if blk * block_size >= npost:
            continue
        e = int(expert_ids[blk])
        if e < 0 or e > 255:
            continue
        for s in sorted_token_ids[blk * block_size:(blk + 1) * block_size]:
            if s < tokens * top_k:
                cache.setdefault(e, []).append(int(s))
    for e, pairs in cache.items():
        rows = np.array(pairs) // top_k
        y[pairs] = mul_mat_a8(wflat[e], x[rows], qtype, n, path="mmq")
    return y


def moe_a8_vec(x, w, topk_ids, top_k, qtype, n, tokens):
    """Per-pair a8 GEMV (moe_vec.cuh:3-53): ``Y[z, :] = W[topk_ids[z]] . q8_1(X[z // top_k])``."""
    x = np.asarray(x)
    wflat = w.reshape(w.shape[0], -1)
    flat = np.asarray(topk_ids).reshape(-1)
    y = np.zeros((tokens * top_k, n), dtype=np.float64)
    for e in np.unique(flat):
        pairs = np.nonzero(flat == e)[0]
        y[pairs] = mul_mat_a8(wflat[int(e)], x[pairs // top_k], qtype, n, path="mmvq")
    return y


def silu_and_mul(x: np.ndarray, stored=None) -> np.ndarray:
    """SiLU(x[:, :d]) * x[:, d:] in fp64.

    With ``stored`` (np.float16) the result is what the layer holds between its two expert GEMMs
    (quantization/fused_moe.py:44-51,80: the activation kernel rounds act(gate) to the tensor's dtype and multiplies in
    that dtype): ``T(T(silu(gate)) * up)``, two roundings; the product of two halves is exact in fp32."""
    d = x.shape[-1] // 2
    a = x[..., :d].astype(np.float64)
    act = a / (1.0 + np.exp(-a))
    if stored is None:
        return act * x[..., d:].astype(np.float64)
    assert stored == np.float16
    return (act.astype(np.float16).astype(np.float32) * x[..., d:].astype(np.float16).astype(np.float32)).astype(np.float16)


# ----------------------------------------------------------------------------
# seeded synthetic tensors live with the package (harness code shared with bench.py)
# ----------------------------------------------------------------------------
from vllm_gguf_plugin_prism_amd.synth import (  # noqa: E402,F401
    QUANTIZERS, make_weights, quantize_q4_0, quantize_q4_k, quantize_q6_k, quantize_q8_0, random_blocks,
)


def rel_l2(a: np.ndarray, b: np.ndarray) -> float:
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / den) if den > 0 else float(np.linalg.norm(a - b))
