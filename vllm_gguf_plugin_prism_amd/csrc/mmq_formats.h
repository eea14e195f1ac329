// Weight-format policies of the prefill GEMMs: how one 32-element block of one packed GGUF weight row is
// fetched from global memory and decoded to int8 codes plus fp32 scale and offset factors.
#pragma once
#include "gguf_common.h"
#include "grid_codes.h"

namespace gguf {

// The routing of the grouped MoE contraction (reference: csrc/gguf/moe.cuh:5-129), as moe_align_block_size leaves it.
struct MoeArgs {
  const int32_t* sorted_token_ids;
  const int32_t* expert_ids;
  const int32_t* num_tokens_post_padded;
  int64_t expert_stride;  // bytes
  int top_k;
  int num_pairs;          // tokens * top_k
  int gemv_sums;          // offset term of Q4_K / Q5_K: 0 = times the stored block sum (the reference's tile kernels,
                          // vecdotq.cuh:369-372), 1 = times d8 * (sum of the quants) (its GEMV, vecdotq.cuh:328-351)
};

// Expected number of blocks of `block` slots that hold pairs, for pairs spread over the experts at random (the sorted array
// has room for block - 1 padding slots per expert, which gives the expert count).  How many there are is known on the
// device only; launch plans that depend on it take this estimate.
static inline double moe_blocks_estimate(int num_sorted, int num_pairs, int block) {
  const double experts = (double)(num_sorted - num_pairs) / (double)(block - 1);
  if (experts < 1.0) return (double)(num_sorted / block);
  const double lam = (double)num_pairs / experts;
  if (lam > 256.0) return (lam / block + 0.5) * experts;
  double blocks = 0.0, term = exp(-lam), cdf = 0.0;   // sum over j >= 0 of P(pairs of an expert > block * j)
  for (int c = 0; c <= 2048 && cdf < 1.0 - 1e-12; ++c) {
    cdf += term;
    if (c % block == 0) blocks += 1.0 - cdf;
    term *= lam / (c + 1);
  }
  return blocks * experts;
}

// The first expert GEMM of a layer with its seam.  The weight rows are [gate | up], inner features each, and a tile's
// columns are the SAME features of both halves (the first half of the columns gate, the second up); the workgroup that
// has both finishes them -- y = T(sum), h = T(T(act(gate)) up), the q8_1 blocks of h -- and writes them into the pair's
// row of a second activation workspace, which the second expert GEMM reads as it is (no [pairs][2 inner] tensor, no
// quantize launch).
struct Gate16 {
  char* rows;             // q8_1 rows of h, one per pair
  int64_t row_bytes;
  int inner, kp, act;     // features of each half; q8_kp(inner); ACT_SILU / ACT_GELU
};

// --------------------------------------------------------------------------------------------
// Format policies: unpack one 32-element block of one weight row to int8 (8 dwords, element order)
// plus fp32 scale(s) and, where the format has one, the fp32 offset factor multiplied by the
// activation block's stored sum (the MMQ semantics, vecdotq.cuh:369-372, 61-64).
// --------------------------------------------------------------------------------------------
// fetch() only issues the global loads of one (row, 32-block) pair into raw registers, unpack() decodes
// them; the two are split so that the loads of the next K step can be in flight during the MFMA phase.
struct MQ4_0 {  // vecdotq.cuh:46-66, 511-571
  static constexpr int QK = 32, BS = 18, G = 32;
  static constexpr bool HAS_MIN = true;
  static constexpr bool LIGHT = true;  // packed block small enough to hold a step of them in registers
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint16_t d; uint4 q; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const uint8_t* b = row + (int64_t)kb * BS;
    Raw r; r.d = ld<uint16_t>(b); r.q = ld<uint4>(b + 2); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = w[i] & 0x0F0F0F0Fu; q[4 + i] = (w[i] >> 4) & 0x0F0F0F0Fu; }
    s0 = (float)__builtin_bit_cast(_Float16, r.d); s1 = s0; mn = 8.0f * s0;
  }
  // per 32-block of the group 8*b8 .. 8*b8+7 of a row: C * scale and C * scale - offset factor, C = 8 the centre the
  // half-MFMA engine subtracts from the codes (0 past the row's end).  Here the two cancel: d * (q - 8) is the weight.
  static constexpr int CENTRE = 8;
  static __device__ __forceinline__ void offs8(const uint8_t* row, int b8, int nkb, float (&cs)[8], float (&cm)[8]) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int b = 8 * b8 + e;
      cs[e] = b < nkb ? 8.0f * ld_f16(row + (int64_t)b * BS) : 0.0f;
      cm[e] = 0.0f;
    }
  }
};

struct MQ8_0 {  // vecdotq.cuh:165-177, 869-921
  static constexpr int QK = 32, BS = 34, G = 32;
  static constexpr bool HAS_MIN = false;
  static constexpr bool LIGHT = true;  // packed block small enough to hold a step of them in registers
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint16_t d; uint4 q0, q1; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const uint8_t* b = row + (int64_t)kb * BS;
    Raw r; r.d = ld<uint16_t>(b); r.q0 = ld<uint4>(b + 2); r.q1 = ld<uint4>(b + 18); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    q[0] = r.q0.x; q[1] = r.q0.y; q[2] = r.q0.z; q[3] = r.q0.w; q[4] = r.q1.x; q[5] = r.q1.y; q[6] = r.q1.z; q[7] = r.q1.w;
    s0 = (float)__builtin_bit_cast(_Float16, r.d); s1 = s0; mn = 0.0f;
  }
};

// Q4_K / Q5_K: for the eight sub-blocks of super-block b8, C * d * sc_j and C * d * sc_j - dmin * m_j from the
// 16-byte block header (6-bit packing: dequantize.cuh:156-163); C is the centre subtracted from the codes
__device__ __forceinline__ void k4_offs8(const uint8_t* row, int bs, int b8, int nkb, float c, float (&cs)[8], float (&cm)[8]) {
  // past the row's end: re-read the last super-block and scale it to nothing (no early return: a branch around the
  // stores to cs / cm would move the two arrays to scratch memory)
  const bool in = 8 * b8 < nkb;
  const uint4 hdr = ld<uint4>(row + (int64_t)min(b8, max(nkb / 8 - 1, 0)) * bs);
  const float d = in ? (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x & 0xFFFF)) : 0.0f;
  const float dmin = in ? (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x >> 16)) : 0.0f;
  const uint32_t lo = hdr.y, mid = hdr.z, hi = hdr.w;  // scale bytes 0..3, 4..7, 8..11
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint32_t b_lo = (lo >> (8 * j)) & 0xFF, b_mid = (mid >> (8 * j)) & 0xFF, b_hi = (hi >> (8 * j)) & 0xFF;
    cs[j] = c * d * (float)(b_lo & 63);
    cm[j] = cs[j] - dmin * (float)(b_mid & 63);
    cs[4 + j] = c * d * (float)((b_hi & 0xF) | ((b_lo >> 6) << 4));
    cm[4 + j] = cs[4 + j] - dmin * (float)((b_hi >> 4) | ((b_mid >> 6) << 4));
  }
}

struct MQ4_K {  // vecdotq.cuh:353-379, 1204-1277
  static constexpr int QK = 256, BS = 144, G = 32;
  static constexpr bool HAS_MIN = true;
  static constexpr bool LIGHT = false;  // packed block small enough to hold a step of them in registers
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint4 hdr, v0, v1; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, j = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r; r.hdr = ld<uint4>(b); r.v0 = ld<uint4>(b + 16 + 32 * (j >> 1)); r.v1 = ld<uint4>(b + 32 + 32 * (j >> 1)); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const int j = kb & 7;
    const int sh = (j & 1) ? 4 : 0;
    const uint32_t w[8] = {r.v0.x, r.v0.y, r.v0.z, r.v0.w, r.v1.x, r.v1.y, r.v1.z, r.v1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = (w[i] >> sh) & 0x0F0F0F0Fu;
    // 6-bit scale / min of sub-block j out of the 12 packed bytes (dequantize.cuh:156-163)
    const uint64_t lo = ((uint64_t)r.hdr.z << 32) | r.hdr.y;  // bytes 0..7
    const uint32_t hi = r.hdr.w;                                // bytes 8..11
    const int jj = j & 3;
    const uint32_t b_lo = (uint32_t)(lo >> (8 * jj)) & 0xFF;        // byte jj
    const uint32_t b_mid = (uint32_t)(lo >> (8 * jj + 32)) & 0xFF;  // byte jj + 4
    const uint32_t b_hi = (hi >> (8 * jj)) & 0xFF;                  // byte jj + 8
    const int sc = j < 4 ? (int)(b_lo & 63) : (int)((b_hi & 0xF) | ((b_lo >> 6) << 4));
    const int m = j < 4 ? (int)(b_mid & 63) : (int)((b_hi >> 4) | ((b_mid >> 6) << 4));
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.hdr.x >> 16));
    s0 = d * (float)sc; s1 = s0; mn = dmin * (float)m;
  }
  static constexpr int CENTRE = 8;
  static __device__ __forceinline__ void offs8(const uint8_t* row, int b8, int nkb, float (&cs)[8], float (&cm)[8]) { k4_offs8(row, BS, b8, nkb, 8.0f, cs, cm); }
};

struct MQ6_K {  // vecdotq.cuh:467-491, 1443-1529: two int8 sub-scales per q8_1 block
  static constexpr int QK = 256, BS = 210, G = 16;
  static constexpr bool HAS_MIN = false;
  static constexpr bool LIGHT = false;  // packed block small enough to hold a step of them in registers
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint4 l0, l1, h0, h1; uint32_t sc, d; };  // 16-bit fields as dwords: two shorts in one struct get packed into one register, which ties their loads together
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, h = (kb >> 2) & 1, t = kb & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint8_t* pl = b + 64 * h + 32 * (t & 1);
    const uint8_t* ph = b + 128 + 32 * h;
    Raw r;
    r.l0 = ld<uint4>(pl); r.l1 = ld<uint4>(pl + 16); r.h0 = ld<uint4>(ph); r.h1 = ld<uint4>(ph + 16);
    r.sc = ld<uint16_t>(b + 192 + 8 * h + 2 * t);
    r.d = ld<uint16_t>(b + 208);
    return r;
  }
  template <bool SIGNED = true>  // false: the codes stay 0..63 and the caller subtracts 32
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const int t = kb & 3;
    const uint32_t lw[8] = {r.l0.x, r.l0.y, r.l0.z, r.l0.w, r.l1.x, r.l1.y, r.l1.z, r.l1.w};
    const uint32_t hw[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
    const int shl = (t >> 1) ? 4 : 0, shh = 2 * t;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t v = ((lw[i] >> shl) & 0x0F0F0F0Fu) | (((hw[i] >> shh) & 0x03030303u) << 4);
      q[i] = SIGNED ? ((v | 0x80808080u) - 0x20202020u) ^ 0x80808080u : v;  // every byte minus 32, no borrow between bytes
    }
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)r.d);
    s0 = d * (float)(int8_t)(r.sc & 0xFF);
    s1 = d * (float)(int8_t)(r.sc >> 8);
    mn = 0.0f;
  }
};

// bits 0..3 of b -> bit 0 of bytes 0..3
__device__ __forceinline__ uint32_t spread4q(uint32_t b) { return ((b & 0xFu) * 0x00204081u) & 0x01010101u; }
// every byte of v (each below 128) minus c, with no borrow between bytes
__device__ __forceinline__ uint32_t sub_bytes(uint32_t v, uint32_t c4) { return ((v | 0x80808080u) - c4) ^ 0x80808080u; }

// Q4_1 and Q5_1 keep the reference's half-precision scale products: S * half(d*d8) + half(m*s8)
// (vecdotq.cuh:71-93, 179-198, 591-646, 771-850).
struct MQ4_1 {
  static constexpr int QK = 32, BS = 20, G = 32;
  static constexpr bool HAS_MIN = true;
  static constexpr bool LIGHT = false;
  static constexpr bool HALFPROD = true, MIN16 = false;
  struct Raw { uint32_t dm; uint4 q; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const uint8_t* b = row + (int64_t)kb * BS;
    Raw r; r.dm = ld<uint32_t>(b); r.q = ld<uint4>(b + 4); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = w[i] & 0x0F0F0F0Fu; q[4 + i] = (w[i] >> 4) & 0x0F0F0F0Fu; }
    s0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.dm & 0xFFFF)); s1 = s0;
    mn = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.dm >> 16)); mn1 = mn;
  }
};

template <bool HAS_M>
struct MQ5 {  // Q5_0: signed codes, no offset term (vecdotq.cuh:668-749); Q5_1: as Q4_1 with a fifth bit
  static constexpr int QK = 32, BS = HAS_M ? 24 : 22, G = 32;
  static constexpr bool HAS_MIN = HAS_M;
  static constexpr bool LIGHT = !HAS_M;
  static constexpr bool HALFPROD = HAS_M, MIN16 = false;
  struct Raw { uint32_t dm, qh; uint4 q; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const uint8_t* b = row + (int64_t)kb * BS;
    Raw r;
    if (HAS_M) { r.dm = ld<uint32_t>(b); r.qh = ld<uint32_t>(b + 4); r.q = ld<uint4>(b + 8); }
    else { r.dm = ld<uint16_t>(b); r.qh = ld<uint32_t>(b + 2); r.q = ld<uint4>(b + 6); }
    return r;
  }
  template <bool SIGNED = true>  // false: Q5_0 codes stay 0..31 and the caller subtracts 16
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q[i] = (w[i] & 0x0F0F0F0Fu) | (spread4q(r.qh >> (4 * i)) << 4);
      q[4 + i] = ((w[i] >> 4) & 0x0F0F0F0Fu) | (spread4q(r.qh >> (16 + 4 * i)) << 4);
      if (!HAS_M && SIGNED) { q[i] = sub_bytes(q[i], 0x10101010u); q[4 + i] = sub_bytes(q[4 + i], 0x10101010u); }
    }
    s0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.dm & 0xFFFF)); s1 = s0;
    mn = HAS_M ? (float)__builtin_bit_cast(_Float16, (uint16_t)(r.dm >> 16)) : 0.0f; mn1 = mn;
  }
};
typedef MQ5<false> MQ5_0;
typedef MQ5<true> MQ5_1;

struct MQ2_K {  // vecdotq.cuh:232-263, 946-1022: per 16 elements a 4-bit scale and a 4-bit min; the min term
                // multiplies the sum of the activation quants of those 16 elements, not the stored block sum
  static constexpr int QK = 256, BS = 84, G = 16;
  static constexpr bool HAS_MIN = true;
  static constexpr bool LIGHT = false;
  static constexpr bool HALFPROD = false, MIN16 = true;
  struct Raw { uint4 v0, v1; uint32_t dm; uint16_t sc; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, n = (kb >> 2) & 1, t = kb & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r;
    r.v0 = ld<uint4>(b + 16 + 32 * n); r.v1 = ld<uint4>(b + 32 + 32 * n);
    r.sc = ld<uint16_t>(b + 8 * n + 2 * t); r.dm = ld<uint32_t>(b + 80);
    return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const int t = kb & 3;
    const uint32_t w[8] = {r.v0.x, r.v0.y, r.v0.z, r.v0.w, r.v1.x, r.v1.y, r.v1.z, r.v1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = (w[i] >> (2 * t)) & 0x03030303u;
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.dm & 0xFFFF));
    const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.dm >> 16));
    s0 = d * (float)(r.sc & 0xF); s1 = d * (float)((r.sc >> 8) & 0xF);
    mn = dmin * (float)((r.sc >> 4) & 0xF); mn1 = dmin * (float)(r.sc >> 12);
  }
};

struct MQ3_K {  // vecdotq.cuh:298-322, 1051-1157: codes -4..3, a signed 6-bit scale per 16 elements
  static constexpr int QK = 256, BS = 110, G = 16;
  static constexpr bool HAS_MIN = false;
  static constexpr bool LIGHT = false;
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint4 v0, v1, h0, h1; uint2 sc01; uint32_t sc2; uint16_t d; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, n = (kb >> 2) & 1;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r;
    r.v0 = ld<uint4>(b + 32 + 32 * n); r.v1 = ld<uint4>(b + 48 + 32 * n); r.h0 = ld<uint4>(b); r.h1 = ld<uint4>(b + 16);
    r.sc01 = ld<uint2>(b + 96); r.sc2 = ld<uint32_t>(b + 104); r.d = ld<uint16_t>(b + 108);
    return r;
  }
  template <bool SIGNED = true>  // false: the codes stay 0..7 and the caller subtracts 4
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const int n = (kb >> 2) & 1, t = kb & 3;
    const uint32_t w[8] = {r.v0.x, r.v0.y, r.v0.z, r.v0.w, r.v1.x, r.v1.y, r.v1.z, r.v1.w};
    const uint32_t h[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t v = ((w[i] >> (2 * t)) & 0x03030303u) | (((h[i] >> (4 * n + t)) & 0x01010101u) << 2);
      q[i] = SIGNED ? sub_bytes(v, 0x04040404u) : v;
    }
    const uint64_t lo64 = ((uint64_t)r.sc01.y << 32) | r.sc01.x;
    const float d = (float)__builtin_bit_cast(_Float16, r.d);
    int us[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {  // 6-bit scale of 16-element group is = 8n + 2t + e (dequantize.cuh:137-140)
      const int g = 2 * t + e, is = 8 * n + g;
      us[e] = (int)((lo64 >> (8 * g + 4 * n)) & 0xF) | (int)(((r.sc2 >> (8 * (is & 3) + 2 * (is >> 2))) & 3) << 4);
    }
    s0 = d * (float)(us[0] - 32); s1 = d * (float)(us[1] - 32); mn = 0.0f; mn1 = 0.0f;
  }
};

struct MQ5_K {  // vecdotq.cuh:415-441, 1325-1415: Q4_K with a fifth bit, bit j of qh[l] for sub-block j
  static constexpr int QK = 256, BS = 176, G = 32;
  static constexpr bool HAS_MIN = true;
  static constexpr bool LIGHT = false;
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint4 hdr, v0, v1, h0, h1; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, j = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r;
    r.hdr = ld<uint4>(b); r.h0 = ld<uint4>(b + 16); r.h1 = ld<uint4>(b + 32);
    r.v0 = ld<uint4>(b + 48 + 32 * (j >> 1)); r.v1 = ld<uint4>(b + 64 + 32 * (j >> 1));
    return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const int j = kb & 7;
    const int sh = (j & 1) ? 4 : 0;
    const uint32_t w[8] = {r.v0.x, r.v0.y, r.v0.z, r.v0.w, r.v1.x, r.v1.y, r.v1.z, r.v1.w};
    const uint32_t h[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = ((w[i] >> sh) & 0x0F0F0F0Fu) | (((h[i] >> j) & 0x01010101u) << 4);
    const uint64_t lo = ((uint64_t)r.hdr.z << 32) | r.hdr.y;
    const uint32_t hi = r.hdr.w;
    const int jj = j & 3;
    const uint32_t b_lo = (uint32_t)(lo >> (8 * jj)) & 0xFF;
    const uint32_t b_mid = (uint32_t)(lo >> (8 * jj + 32)) & 0xFF;
    const uint32_t b_hi = (hi >> (8 * jj)) & 0xFF;
    const int sc = j < 4 ? (int)(b_lo & 63) : (int)((b_hi & 0xF) | ((b_lo >> 6) << 4));
    const int m = j < 4 ? (int)(b_mid & 63) : (int)((b_hi >> 4) | ((b_mid >> 6) << 4));
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.hdr.x & 0xFFFF));
    const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.hdr.x >> 16));
    s0 = d * (float)sc; s1 = s0; mn = dmin * (float)m; mn1 = mn;
  }
  static constexpr int CENTRE = 16;
  static __device__ __forceinline__ void offs8(const uint8_t* row, int b8, int nkb, float (&cs)[8], float (&cm)[8]) { k4_offs8(row, BS, b8, nkb, 16.0f, cs, cm); }
};

// kvalues_iq4nl lookup of the four 4-bit indices that the bytes of w hold at bit SH (0 or 4): byte permutes pick out of
// either half of the table by bits 0-2, a third takes byte i of the half that bit 3 of index i names
template <int SH>
__device__ __forceinline__ int lut16q(uint32_t w) {
  constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
  const uint32_t sel = (SH ? w >> SH : w) & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(T3, T2, sel);
  const uint32_t pick = ((w >> (SH + 1)) & 0x04040404u) | 0x03020100u;
  return (int)__builtin_amdgcn_perm(hi, lo, pick);
}

struct MIQ4_XS {  // extension: the reference has no MMQ tiles for i-quants (gguf_kernel.cu:236-287)
  static constexpr int QK = 256, BS = 136, G = 32;
  static constexpr bool HAS_MIN = false;
  static constexpr bool LIGHT = true;  // packed block small enough to hold a step of them in registers
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint2 hdr; uint4 v; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, ib = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r; r.hdr = ld<uint2>(b); r.v = ld<uint4>(b + 8 + 16 * ib); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    const int ib = kb & 7;
    const uint32_t w[4] = {r.v.x, r.v.y, r.v.z, r.v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = (uint32_t)lut16q<0>(w[i]); q[4 + i] = (uint32_t)lut16q<4>(w[i]); }
    const int ls = (int)(((r.hdr.y >> (4 * ib)) & 0xF) | ((((r.hdr.x >> 16) >> (2 * ib)) & 3) << 4));
    s0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.hdr.x & 0xFFFF)) * (float)(ls - 32);
    s1 = s0; mn = 0.0f;
  }
};

struct MIQ2_XXS {  // extension, see MIQ4_XS
  static constexpr int QK = 256, BS = 66, G = 32;
  static constexpr bool HAS_MIN = false;
  static constexpr bool LIGHT = false;  // packed block small enough to hold a step of them in registers
  static constexpr bool HALFPROD = false, MIN16 = false;
  struct Raw { uint16_t d; uint2 g; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, ib = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r; r.d = ld<uint16_t>(b); r.g = ld<uint2>(b + 2 + 8 * ib); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t code = k_iq2xxs_grid_codes[(r.g.x >> (8 * l)) & 0xFF];
      const uint32_t s7 = (r.g.y >> (7 * l)) & 127;
      const uint32_t sg = s7 | ((__builtin_popcount(s7) & 1) << 7);
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t c = (code >> (2 * j)) & 3;
        const uint32_t mag = 8 + 17 * c + (c >> 1);
        const uint32_t val = ((sg >> j) & 1) ? (0u - mag) & 0xFFu : mag;
        w[j >> 2] |= val << (8 * (j & 3));
      }
      q[2 * l] = w[0]; q[2 * l + 1] = w[1];
    }
    s0 = (float)__builtin_bit_cast(_Float16, r.d) * (0.5f + (float)(r.g.y >> 28)) * 0.25f;
    s1 = s0; mn = 0.0f;
  }
};

}  // namespace gguf
