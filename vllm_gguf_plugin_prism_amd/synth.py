"""Seeded synthetic GGUF tensors for tests and benchmarks (harness only, not on the hot path).

Weights are drawn N(0, std) and quantized with simple valid quantizers for Q8_0, Q4_0,
Q4_K and Q6_K; other formats get random raw block bytes with the fp16 super-scale
overwritten by U(1e-4, 1e-2) (every byte pattern is a valid block for them).  Parity
is always checked on whatever bytes result, so the quantizers need not be optimal.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1 = 2, 3, 6, 7, 8, 9
Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 10, 11, 12, 13, 14
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ4_NL, IQ3_S, IQ2_S, IQ4_XS, IQ1_M = 16, 17, 18, 19, 20, 21, 22, 23, 29

# ggml type id -> (elements per block, bytes per block)
QUANT_SIZES = {
    Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34), Q8_1: (32, 36),
    Q2_K: (256, 84), Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210),
    IQ2_XXS: (256, 66), IQ2_XS: (256, 74), IQ3_XXS: (256, 98), IQ1_S: (256, 50), IQ4_NL: (32, 18),
    IQ3_S: (256, 110), IQ2_S: (256, 82), IQ4_XS: (256, 136), IQ1_M: (256, 56),
}


def _half_bytes(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a.astype("<f2")).view(np.uint8).reshape(a.shape + (2,))


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    n, k = w.shape
    blk = w.reshape(n, k // 32, 32).astype(np.float32)
    d = (np.abs(blk).max(axis=2) / 127).astype(np.float16)
    df = d.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(df[:, :, None] == 0, 0, np.rint(blk / df[:, :, None]))
    q = np.clip(q, -127, 127).astype(np.int8)
    out = np.empty((n, k // 32, 34), dtype=np.uint8)
    out[:, :, 0:2] = _half_bytes(d)
    out[:, :, 2:] = q.view(np.uint8)
    return out.reshape(n, -1)


def quantize_q4_0(w: np.ndarray) -> np.ndarray:
    n, k = w.shape
    blk = w.reshape(n, k // 32, 32).astype(np.float32)
    imax = np.abs(blk).argmax(axis=2)
    vmax = np.take_along_axis(blk, imax[:, :, None], axis=2)[:, :, 0]
    d = (vmax / -8).astype(np.float16)
    df = d.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(df[:, :, None] == 0, 8, np.trunc(blk / df[:, :, None] + 8.5))
    q = np.clip(q, 0, 15).astype(np.uint8)
    out = np.empty((n, k // 32, 18), dtype=np.uint8)
    out[:, :, 0:2] = _half_bytes(d)
    out[:, :, 2:] = q[:, :, :16] | (q[:, :, 16:] << 4)
    return out.reshape(n, -1)


def quantize_q4_k(w: np.ndarray) -> np.ndarray:
    n, k = w.shape
    sb = w.reshape(n, k // 256, 8, 32).astype(np.float32)
    mn0 = np.minimum(sb.min(axis=3), 0)
    scale = (sb.max(axis=3) - mn0) / 15
    d = (scale.max(axis=2) / 63).astype(np.float16)
    dmin = ((-mn0).max(axis=2) / 63).astype(np.float16)
    df = d.astype(np.float32)[:, :, None]
    dmf = dmin.astype(np.float32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.clip(np.where(df == 0, 0, np.rint(scale / df)), 0, 63).astype(np.uint8)
        mm = np.clip(np.where(dmf == 0, 0, np.rint(-mn0 / dmf)), 0, 63).astype(np.uint8)
        den = df * sc
        q = np.where(den[..., None] == 0, 0, np.rint((sb + (dmf * mm)[..., None]) / den[..., None]))
    q = np.clip(q, 0, 15).astype(np.uint8)
    out = np.empty((n, k // 256, 144), dtype=np.uint8)
    out[:, :, 0:2] = _half_bytes(d)
    out[:, :, 2:4] = _half_bytes(dmin)
    s12 = np.zeros((n, k // 256, 12), dtype=np.uint8)
    for j in range(4):
        s12[:, :, j] = (sc[:, :, j] & 63) | ((sc[:, :, j + 4] >> 4) << 6)
        s12[:, :, j + 4] = (mm[:, :, j] & 63) | ((mm[:, :, j + 4] >> 4) << 6)
        s12[:, :, j + 8] = (sc[:, :, j + 4] & 0xF) | ((mm[:, :, j + 4] & 0xF) << 4)
    out[:, :, 4:16] = s12
    for g in range(4):
        out[:, :, 16 + 32 * g:48 + 32 * g] = q[:, :, 2 * g] | (q[:, :, 2 * g + 1] << 4)
    return out.reshape(n, -1)


def quantize_q6_k(w: np.ndarray) -> np.ndarray:
    n, k = w.shape
    sb = w.reshape(n, k // 256, 16, 16).astype(np.float32)
    imax = np.abs(sb).argmax(axis=3)
    s = np.take_along_axis(sb, imax[..., None], axis=3)[..., 0] / -32  # signed, llama.cpp style
    d = (np.abs(s).max(axis=2) / 127).astype(np.float16)
    df = d.astype(np.float32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.clip(np.where(df == 0, 0, np.rint(s / df)), -128, 127).astype(np.int8)
        den = df * sc
        q = np.where(den[..., None] == 0, 0, np.rint(sb / den[..., None]))
    q = (np.clip(q, -32, 31) + 32).astype(np.uint8).reshape(n, k // 256, 256)
    out = np.empty((n, k // 256, 210), dtype=np.uint8)
    for h in range(2):
        e = q[:, :, 128 * h:128 * h + 128]
        out[:, :, 64 * h:64 * h + 32] = (e[:, :, 0:32] & 0xF) | ((e[:, :, 64:96] & 0xF) << 4)
        out[:, :, 64 * h + 32:64 * h + 64] = (e[:, :, 32:64] & 0xF) | ((e[:, :, 96:128] & 0xF) << 4)
        out[:, :, 128 + 32 * h:160 + 32 * h] = (
            (e[:, :, 0:32] >> 4) | ((e[:, :, 32:64] >> 4) << 2) | ((e[:, :, 64:96] >> 4) << 4) | ((e[:, :, 96:128] >> 4) << 6)
        )
    out[:, :, 192:208] = sc.view(np.uint8)
    out[:, :, 208:210] = _half_bytes(d)
    return out.reshape(n, -1)


def random_blocks(rng: np.random.Generator, qtype: int, n: int, k: int, d_lo: float = 1e-4, d_hi: float = 1e-2) -> np.ndarray:
    """Seeded random *raw* block bytes with the fp16 super-scale(s) overwritten by U(d_lo, d_hi).

    Every byte pattern is a valid block for the formats this is used with.
    """
    qk, bs = QUANT_SIZES[qtype]
    nb = n * k // qk
    raw = rng.integers(0, 256, size=(nb, bs), dtype=np.uint8)
    d = rng.uniform(d_lo, d_hi, size=nb).astype(np.float16)
    d_off = {Q2_K: (80, 82), Q3_K: (108,), Q6_K: (208,), Q4_K: (0, 2), Q5_K: (0, 2), Q4_1: (0, 2), Q5_1: (0, 2), IQ1_M: ()}.get(qtype, (0,))
    for o in d_off:
        raw[:, o:o + 2] = _half_bytes(d if o == d_off[0] else (d * np.float16(0.5)).astype(np.float16))
    if qtype == IQ1_M:  # fp16 scale scattered over the top nibbles of scales[1::2] pairs
        bits = d.view(np.uint16)
        sc = np.ascontiguousarray(raw[:, 48:56]).view("<u2")
        sc[:, 0] = (sc[:, 0] & 0x0FFF) | ((bits & 0x000F) << 12)
        sc[:, 1] = (sc[:, 1] & 0x0FFF) | ((bits & 0x00F0) << 8)
        sc[:, 2] = (sc[:, 2] & 0x0FFF) | ((bits & 0x0F00) << 4)
        sc[:, 3] = (sc[:, 3] & 0x0FFF) | (bits & 0xF000)
        raw[:, 48:56] = sc.view(np.uint8)
    return raw.reshape(n, -1)


QUANTIZERS = {Q8_0: quantize_q8_0, Q4_0: quantize_q4_0, Q4_K: quantize_q4_k, Q6_K: quantize_q6_k}


def make_weights(rng: np.random.Generator, qtype: int, n: int, k: int, std: float = 0.02) -> np.ndarray:
    """Seeded weights: N(0, std) quantized where a quantizer exists, random raw blocks otherwise."""
    if qtype in QUANTIZERS:
        return QUANTIZERS[qtype](rng.standard_normal((n, k), dtype=np.float32) * np.float32(std))
    return random_blocks(rng, qtype, n, k)
