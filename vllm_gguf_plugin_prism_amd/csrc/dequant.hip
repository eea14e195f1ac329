// GGUF block dequantisation for gfx950: packed blocks -> dense fp16 / bf16 / fp32.
//
// The kernels are write-bound (the dense output is 2-8x the packed input), so the
// work split is by OUTPUT: every thread produces eight consecutive elements and
// stores them with one (fp16/bf16) or two (fp32) 128-bit writes; consecutive
// threads write consecutive 16-byte segments.
//
// Rounding follows the reference kernels (csrc/gguf/dequantize.cuh) as hipcc
// builds them for gfx950: standard and K quants compute in half precision, with
// a mul feeding an add/sub evaluated as ONE half fma; i-quants compute in fp32.
// fp contraction is switched off for the file and every fused op is spelled out,
// so the choice does not depend on the optimiser.
#include "gguf_common.h"
#include "grid_codes.h"

#pragma clang fp contract(off)

namespace gguf {

typedef _Float16 h16;

// ---- eight dense values starting at element e0 (a multiple of 8) --------------------------------

// Q4_0: dequantize.cuh:3-15.  (q - 8) is exact in half, then one multiply.
__device__ __forceinline__ void dq8_q4_0(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 5) * 18;
  const int pos = (int)(e0 & 31);
  const h16 d = ld_h(blk);
  const uint2 q = ld<uint2>(blk + 2 + (pos & 15));
  const int sh = pos >> 4 ? 4 : 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    const int v = (int)((word >> (8 * (i & 3) + sh)) & 0xF);
    o[i] = (h16)(v - 8) * d;
  }
}

// Q8_0: dequantize.cuh:69-78.
__device__ __forceinline__ void dq8_q8_0(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 5) * 34;
  const int pos = (int)(e0 & 31);
  const h16 d = ld_h(blk);
  const uint2 q = ld<uint2>(blk + 2 + pos);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    const int v = (int)(int8_t)(word >> (8 * (i & 3)));
    o[i] = (h16)v * d;
  }
}

// 6-bit scale and min of sub-block j from the 12 packed bytes, given as the three dwords that hold bytes 0-3, 4-7 and
// 8-11 (dequantize.cuh:156-163).  Shifts only: indexing the bytes through a pointer would put them in scratch memory.
__device__ __forceinline__ void scale_min_k4(uint32_t b03, uint32_t b47, uint32_t b8b, int j, int& sc, int& mn) {
  const int sh = 8 * (j & 3);
  const uint32_t lo = (b03 >> sh) & 0xFF, mid = (b47 >> sh) & 0xFF, hi = (b8b >> sh) & 0xFF;
  // both forms are computed and one is selected: a branch here would make the compiler hold back the loads behind it
  const int sc_lo = (int)(lo & 63), mn_lo = (int)(mid & 63);
  const int sc_hi = (int)((hi & 0xF) | ((lo >> 6) << 4)), mn_hi = (int)((hi >> 4) | ((mid >> 6) << 4));
  sc = j < 4 ? sc_lo : sc_hi;
  mn = j < 4 ? mn_lo : mn_hi;
}

// Q4_K: dequantize.cuh:165-196.  d1 = d*sc, m1 = dmin*m (each rounded), y = fma(d1, q, -m1).
__device__ __forceinline__ void dq8_q4_k(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 144;
  const int r = (int)(e0 & 255);
  const int j = r >> 5, pos = r & 31;
  const uint4 hdr = *(const uint4*)blk;  // 144-byte blocks keep 16-byte alignment
  const uint2 q = *(const uint2*)(blk + 16 + 32 * (j >> 1) + pos);   // both loads are in flight before either is used
  const h16 dall = __builtin_bit_cast(h16, (uint16_t)(hdr.x & 0xFFFF));
  const h16 dmin = __builtin_bit_cast(h16, (uint16_t)(hdr.x >> 16));
  int sc, mn;
  scale_min_k4(hdr.y, hdr.z, hdr.w, j, sc, mn);
  const h16 d1 = dall * (h16)sc;
  const h16 m1 = dmin * (h16)mn;
  const int sh = (j & 1) ? 4 : 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    const int v = (int)((word >> (8 * (i & 3) + sh)) & 0xF);
    o[i] = __builtin_fmaf16(d1, (h16)v, -m1);
  }
}

// Q6_K: dequantize.cuh:232-256.  y = d * half_rn(sc * (q - 32)).
__device__ __forceinline__ void dq8_q6_k(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 210;
  const int r = (int)(e0 & 255);
  const int h = r >> 7, t = (r >> 5) & 3, l0 = r & 31;  // element = 128h + 32t + l
  const uint2 ql = ld<uint2>(blk + 64 * h + 32 * (t & 1) + l0);
  const uint2 qh = ld<uint2>(blk + 128 + 32 * h + l0);
  const int sc = (int)(int8_t)blk[192 + 8 * h + 2 * t + (l0 >> 4)];
  const h16 d = ld_h(blk + 208);
  const int shl = (t >> 1) ? 4 : 0, shh = 2 * t;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t lw = i < 4 ? ql.x : ql.y, hw = i < 4 ? qh.x : qh.y;
    const int lo = (int)((lw >> (8 * (i & 3) + shl)) & 0xF);
    const int hi = (int)((hw >> (8 * (i & 3) + shh)) & 3);
    const int v = sc * ((lo | (hi << 4)) - 32);
    o[i] = d * (h16)v;  // int -> half rounds to nearest even above 2048
  }
}

// kvalues_iq4nl (ggml-common.h:1060) of four 4-bit codes held one per byte, as four signed bytes: the table sits
// in four registers and v_perm picks from it, instead of eight byte loads from memory per thread.
__device__ __forceinline__ int kvalues_iq4nl4(uint32_t idx) {
  constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;  // -127 -104 -83 -65 | ... | 53 69 89 113
  const uint32_t sel = idx & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(T3, T2, sel);
  const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
  return (int)((hi & m) | (lo & ~m));
}

// IQ4_XS: dequantize.cuh:420-435 (fp32).
__device__ __forceinline__ void dq8_iq4_xs(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 136;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, pos = r & 31;
  const uint32_t sh = ld<uint16_t>(blk + 2);
  const int ls = ((blk[4 + (ib >> 1)] >> (4 * (ib & 1))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4);
  const float d = ld_f16(blk) * (float)(ls - 32);
  const uint2 q = ld<uint2>(blk + 8 + 16 * ib + (pos & 15));
  const int shq = pos >> 4 ? 4 : 0;
  const int v0 = kvalues_iq4nl4((q.x >> shq) & 0x0F0F0F0Fu), v1 = kvalues_iq4nl4((q.y >> shq) & 0x0F0F0F0Fu);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = d * (float)(int8_t)((i < 4 ? v0 : v1) >> (8 * (i & 3)));
}

// IQ2_XXS: dequantize.cuh:258-275 (fp32).  Grid magnitudes are decoded from the 16-bit code word.
__device__ __forceinline__ void dq8_iq2_xxs(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 66;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, l = (r >> 3) & 3;
  const uint8_t* g = blk + 2 + 8 * ib;
  const uint32_t aux = ld<uint16_t>(g + 4) | ((uint32_t)ld<uint16_t>(g + 6) << 16);
  const float d = ld_f16(blk) * (0.5f + (float)(aux >> 28)) * 0.25f;
  const uint32_t s7 = (aux >> (7 * l)) & 127;
  const uint32_t signs = s7 | ((__builtin_popcount(s7) & 1) << 7);
  const uint32_t code = k_iq2xxs_grid_codes[g[l]];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int c = (code >> (2 * j)) & 3;
    const float mag = (float)(8 + 17 * c + (c >> 1));
    o[j] = d * mag * ((signs >> j) & 1 ? -1.0f : 1.0f);
  }
}


// ---- the remaining standard and K formats (half arithmetic, as above) ------------------------------------------

// Q4_1: dequantize.cuh:17-30.  q * d + m, the multiply feeding the add rounds once.
__device__ __forceinline__ void dq8_q4_1(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 5) * 20;
  const int pos = (int)(e0 & 31);
  const h16 d = ld_h(blk), m = ld_h(blk + 2);
  const uint2 q = ld<uint2>(blk + 4 + (pos & 15));
  const int sh = pos >> 4 ? 4 : 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    o[i] = __builtin_fmaf16((h16)(int)((word >> (8 * (i & 3) + sh)) & 0xF), d, m);
  }
}

// Q5_0 / Q5_1: dequantize.cuh:32-67.  Bit j of qh is the fifth bit of element j.
template <bool HAS_M>
__device__ __forceinline__ void dq8_q5(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  constexpr int BS = HAS_M ? 24 : 22, OFF = HAS_M ? 4 : 2;
  const uint8_t* blk = w + (e0 >> 5) * BS;
  const int pos = (int)(e0 & 31);
  const h16 d = ld_h(blk);
  const uint32_t qh = ld<uint32_t>(blk + OFF) >> pos;
  const uint2 q = ld<uint2>(blk + OFF + 4 + (pos & 15));
  const int sh = pos >> 4 ? 4 : 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    const int v = (int)((word >> (8 * (i & 3) + sh)) & 0xF) | (int)(((qh >> i) & 1) << 4);
    if constexpr (HAS_M) o[i] = __builtin_fmaf16((h16)v, d, ld_h(blk + 2));
    else o[i] = (h16)(v - 16) * d;
  }
}

// Q2_K: dequantize.cuh:101-121.  fma(dall, half(sc*q), -(dmin*half(m))): the offset product rounds on its own.
__device__ __forceinline__ void dq8_q2_k(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 84;
  const int r = (int)(e0 & 255);
  const int n = r >> 7, sft = 2 * ((r >> 5) & 3), l0 = r & 31;
  const int scm = blk[r >> 4];
  const h16 dall = ld_h(blk + 80), dmin = ld_h(blk + 82);
  const h16 m1 = dmin * (h16)(scm >> 4);
  const int sc = scm & 0xF;
  const uint2 q = ld<uint2>(blk + 16 + 32 * n + l0);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    const int v = (int)((word >> (8 * (i & 3) + sft)) & 3);
    o[i] = __builtin_fmaf16(dall, (h16)(sc * v), -m1);
  }
}

// 6-bit scale `is` of a Q3_K block, minus nothing (dequantize.cuh:137-140); s points at the 12 scale bytes.
__device__ __forceinline__ int q3k_scale(const uint8_t* __restrict__ s, int is) {
  // the twelve bytes as three dwords, fields by shifts: byte loads at computed offsets behind a branch would be
  // issued one after the other
  const uint32_t s0 = ld<uint32_t>(s), s1 = ld<uint32_t>(s + 4), s2 = ld<uint32_t>(s + 8);
  const uint32_t lo8 = ((is & 4) ? s1 : s0) >> (8 * (is & 3));        // byte is % 8
  const int lo = (int)((lo8 >> (is < 8 ? 0 : 4)) & 0xF);
  const int hi = (int)((s2 >> (8 * (is & 3) + 2 * (is >> 2))) & 3);
  return lo | (hi << 4);
}

// Q3_K: dequantize.cuh:123-154.  dl = d * half(us - 32), then dl * half(q - 4*(1 - hbit)).
__device__ __forceinline__ void dq8_q3_k(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 110;
  const int r = (int)(e0 & 255);
  const int n = r >> 7, j = (r >> 5) & 3, l0 = r & 31;
  const uint2 q = ld<uint2>(blk + 32 + 32 * n + l0);
  const uint2 hm = ld<uint2>(blk + l0);
  const h16 dl = ld_h(blk + 108) * (h16)(q3k_scale(blk + 96, r >> 4) - 32);
  const int hb = 4 * n + j;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t qw = i < 4 ? q.x : q.y, hw = i < 4 ? hm.x : hm.y;
    const int v = (int)((qw >> (8 * (i & 3) + 2 * j)) & 3) - (((hw >> (8 * (i & 3) + hb)) & 1) ? 0 : 4);
    o[i] = dl * (h16)v;
  }
}

// Q5_K: dequantize.cuh:198-230.  As Q4_K with a fifth bit from qh.
__device__ __forceinline__ void dq8_q5_k(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 176;
  const int r = (int)(e0 & 255);
  const int j = r >> 5, pos = r & 31;
  const uint4 hdr = *(const uint4*)blk;  // 176-byte blocks keep 16-byte alignment
  const uint2 q = *(const uint2*)(blk + 48 + 32 * (j >> 1) + pos);
  const uint2 qh = *(const uint2*)(blk + 16 + pos);
  const h16 dall = __builtin_bit_cast(h16, (uint16_t)(hdr.x & 0xFFFF));
  const h16 dmin = __builtin_bit_cast(h16, (uint16_t)(hdr.x >> 16));
  int sc, mn;
  scale_min_k4(hdr.y, hdr.z, hdr.w, j, sc, mn);
  const h16 d1 = dall * (h16)sc;
  const h16 m1 = dmin * (h16)mn;
  const int sh = (j & 1) ? 4 : 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y, hw = i < 4 ? qh.x : qh.y;
    const int v = (int)((word >> (8 * (i & 3) + sh)) & 0xF) + (int)(((hw >> (8 * (i & 3) + j)) & 1) << 4);
    o[i] = __builtin_fmaf16(d1, (h16)v, -m1);
  }
}

// ---- the remaining i-quants (fp32; every product below is exact, so the only rounding is the final convert) -----

__device__ __forceinline__ uint32_t sign_byte(uint32_t s7) { return s7 | ((__builtin_popcount(s7) & 1) << 7); }
__device__ __forceinline__ float mag2(uint32_t code, int j) {  // {8, 25, 43}
  const int c = (code >> (2 * j)) & 3;
  return (float)(8 + 17 * c + (c >> 1));
}
__device__ __forceinline__ float signed_f(float v, uint32_t signs, int j) { return (signs >> j) & 1 ? -v : v; }

// IQ2_XS: dequantize.cuh:277-293.
__device__ __forceinline__ void dq8_iq2_xs(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 74;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, il = (r >> 3) & 3;
  const uint32_t q2 = ld<uint16_t>(blk + 2 + 2 * (4 * ib + il));
  const float d = ld_f16(blk) * (0.5f + (float)((blk[66 + ib] >> (4 * (il >> 1))) & 0xF)) * 0.25f;
  const uint32_t code = k_iq2xs_grid_codes[q2 & 511];
  const uint32_t signs = sign_byte(q2 >> 9);
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = signed_f(d * mag2(code, j), signs, j);
}

// IQ2_S: dequantize.cuh:295-309.
__device__ __forceinline__ void dq8_iq2_s(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 82;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, il = (r >> 3) & 3;
  const uint32_t idx = blk[2 + 4 * ib + il] | (((uint32_t)blk[66 + ib] << (8 - 2 * il)) & 0x300);
  const float d = ld_f16(blk) * (0.5f + (float)((blk[74 + ib] >> (4 * (il >> 1))) & 0xF)) * 0.25f;
  const uint32_t code = k_iq2s_grid_codes[idx];
  const uint32_t signs = blk[34 + 4 * ib + il];
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = signed_f(d * mag2(code, j), signs, j);
}

__device__ __forceinline__ float mag3xxs(uint32_t code, int j) {  // {4, 12, ..., 52, 62}
  const int c = (code >> (3 * j)) & 7;
  return (float)(4 + 8 * c + 2 * ((c + 1) >> 3));
}
__device__ __forceinline__ float mag3xs(uint32_t code, int j) {  // {4, 12, ..., 60}
  return (float)(4 + 8 * ((code >> (3 * j)) & 7));
}

// IQ3_XXS: dequantize.cuh:311-332.
__device__ __forceinline__ void dq8_iq3_xxs(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 98;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, il = (r >> 3) & 3;
  const uint8_t* q3 = blk + 2 + 8 * ib;
  const uint32_t aux = ld<uint16_t>(blk + 66 + 4 * ib) | ((uint32_t)ld<uint16_t>(blk + 68 + 4 * ib) << 16);
  const float d = ld_f16(blk) * (0.5f + (float)(aux >> 28)) * 0.5f;
  const uint32_t signs = sign_byte((aux >> (7 * il)) & 127);
  const uint32_t c1 = k_iq3xxs_grid_codes[q3[2 * il]], c2 = k_iq3xxs_grid_codes[q3[2 * il + 1]];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    o[j] = signed_f(d * mag3xxs(c1, j), signs, j);
    o[4 + j] = signed_f(d * mag3xxs(c2, j), signs, 4 + j);
  }
}

// IQ3_S: dequantize.cuh:334-353.
__device__ __forceinline__ void dq8_iq3_s(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 110;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, il = (r >> 3) & 3;
  const uint8_t* qs = blk + 2 + 8 * ib;
  const uint32_t qh = blk[66 + ib];
  const uint32_t i1 = qs[2 * il] | ((qh << (8 - 2 * il)) & 256), i2 = qs[2 * il + 1] | ((qh << (7 - 2 * il)) & 256);
  const float d = ld_f16(blk) * (0.5f + (float)((blk[106 + (ib >> 1)] >> (4 * (ib & 1))) & 0xF)) * 0.5f;
  const uint32_t signs = blk[74 + 4 * ib + il];
  const uint32_t c1 = k_iq3xs_grid_codes[i1], c2 = k_iq3xs_grid_codes[i2];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    o[j] = signed_f(d * mag3xs(c1, j), signs, j);
    o[4 + j] = signed_f(d * mag3xs(c2, j), signs, 4 + j);
  }
}

// Eight values {0,1,2} of one 1-bit grid entry in output order: the table packs value j in nibble j, and the
// reference reads the even nibbles first (dequantize.cuh:368-370).
__device__ __forceinline__ float iq1_val(uint32_t code, int j) {
  const int nib = j < 4 ? 2 * j : 2 * (j - 4) + 1;
  return (float)((code >> (2 * nib)) & 3);
}

// IQ1_S: dequantize.cuh:355-374.  y = d * (q + delta), delta = -1 -/+ 0.125.
__device__ __forceinline__ void dq8_iq1_s(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 50;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, il = (r >> 3) & 3;
  const uint32_t qh = ld<uint16_t>(blk + 34 + 2 * ib);
  const float delta = qh & 0x8000 ? -1.0f - 0.125f : -1.0f + 0.125f;
  const float d = ld_f16(blk) * (float)(2 * ((qh >> 12) & 7) + 1);
  const uint32_t code = k_iq1s_grid_gpu_codes[blk[2 + 4 * ib + il] | (((qh >> (3 * il)) & 7) << 8)];
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = d * (iq1_val(code, j) + delta);
}

// IQ1_M: dequantize.cuh:376-399.  The fp16 super-scale is scattered over the top nibbles of four 16-bit words.
__device__ __forceinline__ void dq8_iq1_m(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 56;
  const int r = (int)(e0 & 255);
  const int ib = r >> 5, il = (r >> 3) & 3;
  const uint32_t s0 = ld<uint16_t>(blk + 48), s1 = ld<uint16_t>(blk + 50), s2 = ld<uint16_t>(blk + 52), s3 = ld<uint16_t>(blk + 54);
  const uint16_t sbits = (uint16_t)((s0 >> 12) | ((s1 >> 8) & 0x00F0) | ((s2 >> 4) & 0x0F00) | (s3 & 0xF000));
  const int ib16 = 2 * ib + (il >> 1);
  const uint32_t scw = ld<uint16_t>(blk + 48 + 2 * (ib16 >> 2));
  const float d = (float)__builtin_bit_cast(h16, sbits) * (float)(2 * ((scw >> (3 * (ib16 & 3))) & 7) + 1);
  const uint32_t qh = blk[32 + 2 * ib + (il >> 1)];
  const float delta = qh & (0x08u << (4 * (il & 1))) ? -1.0f - 0.125f : -1.0f + 0.125f;
  const uint32_t code = k_iq1s_grid_gpu_codes[blk[4 * ib + il] | (((qh >> (4 * (il & 1))) & 7) << 8)];
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = d * (iq1_val(code, j) + delta);
}

// IQ4_NL: dequantize.cuh:401-418.  The Q4_0 layout with the non-linear code table.
__device__ __forceinline__ void dq8_iq4_nl(const uint8_t* __restrict__ w, int64_t e0, float (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 5) * 18;
  const int pos = (int)(e0 & 31);
  const float d = ld_f16(blk);
  const uint2 q = ld<uint2>(blk + 2 + (pos & 15));
  const int sh = pos >> 4 ? 4 : 0;
  const int v0 = kvalues_iq4nl4((q.x >> sh) & 0x0F0F0F0Fu), v1 = kvalues_iq4nl4((q.y >> sh) & 0x0F0F0F0Fu);
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = d * (float)(int8_t)((i < 4 ? v0 : v1) >> (8 * (i & 3)));
}

template <typename OutT>
__device__ __forceinline__ void store8(OutT* __restrict__ y, const OutT (&v)[8]) {
  if constexpr (sizeof(OutT) == 2) {
    *(uint4*)y = *(const uint4*)v;
  } else {
    ((uint4*)y)[0] = ((const uint4*)v)[0];
    ((uint4*)y)[1] = ((const uint4*)v)[1];
  }
}

// eight dense values of packed elements [e0, e0 + 8) of `w`
template <int TYPE, typename OutT>
__device__ __forceinline__ void dequant8_values(const uint8_t* __restrict__ w, int64_t e0, OutT (&out)[8]) {
  constexpr bool F32_MATH = TYPE == T_IQ4_XS || TYPE == T_IQ2_XXS || TYPE == T_IQ2_XS || TYPE == T_IQ2_S || TYPE == T_IQ3_XXS ||
                            TYPE == T_IQ3_S || TYPE == T_IQ1_S || TYPE == T_IQ1_M || TYPE == T_IQ4_NL;
  if constexpr (F32_MATH) {
    float f[8];
    if constexpr (TYPE == T_IQ4_XS) dq8_iq4_xs(w, e0, f);
    if constexpr (TYPE == T_IQ2_XXS) dq8_iq2_xxs(w, e0, f);
    if constexpr (TYPE == T_IQ2_XS) dq8_iq2_xs(w, e0, f);
    if constexpr (TYPE == T_IQ2_S) dq8_iq2_s(w, e0, f);
    if constexpr (TYPE == T_IQ3_XXS) dq8_iq3_xxs(w, e0, f);
    if constexpr (TYPE == T_IQ3_S) dq8_iq3_s(w, e0, f);
    if constexpr (TYPE == T_IQ1_S) dq8_iq1_s(w, e0, f);
    if constexpr (TYPE == T_IQ1_M) dq8_iq1_m(w, e0, f);
    if constexpr (TYPE == T_IQ4_NL) dq8_iq4_nl(w, e0, f);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = from_f32<OutT>(f[i]);
  } else {
    h16 h[8];
    if constexpr (TYPE == T_Q4_0) dq8_q4_0(w, e0, h);
    if constexpr (TYPE == T_Q4_1) dq8_q4_1(w, e0, h);
    if constexpr (TYPE == T_Q5_0) dq8_q5<false>(w, e0, h);
    if constexpr (TYPE == T_Q5_1) dq8_q5<true>(w, e0, h);
    if constexpr (TYPE == T_Q8_0) dq8_q8_0(w, e0, h);
    if constexpr (TYPE == T_Q2_K) dq8_q2_k(w, e0, h);
    if constexpr (TYPE == T_Q3_K) dq8_q3_k(w, e0, h);
    if constexpr (TYPE == T_Q4_K) dq8_q4_k(w, e0, h);
    if constexpr (TYPE == T_Q5_K) dq8_q5_k(w, e0, h);
    if constexpr (TYPE == T_Q6_K) dq8_q6_k(w, e0, h);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = from_half<OutT>(h[i]);
  }
}

// the same, stored at `dst`
template <int TYPE, typename OutT>
__device__ __forceinline__ void dequant8(const uint8_t* __restrict__ w, int64_t e0, OutT* __restrict__ dst) {
  alignas(16) OutT out[8];
  dequant8_values<TYPE, OutT>(w, e0, out);
  store8<OutT>(dst, out);
}

// A workgroup covers 4096 consecutive elements; every thread produces two groups of eight, 2048 elements apart, and
// decodes both before it stores either, so that the loads of the two groups (and, for the codebook formats, their
// dependent table lookups) are in flight together.  Groups past the end are computed on the last group and not stored.
template <int TYPE, typename OutT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ w, OutT* __restrict__ y, int64_t nelem) {
  const int64_t e0 = (int64_t)blockIdx.x * 4096 + threadIdx.x * 8, e1 = e0 + 2048;
  const int64_t last = nelem - 8;
  alignas(16) OutT a[8], b[8];
  dequant8_values<TYPE, OutT>(w, e0 < last ? e0 : last, a);
  dequant8_values<TYPE, OutT>(w, e1 < last ? e1 : last, b);
  if (e0 < nelem) store8<OutT>(y + e0, a);
  if (e1 < nelem) store8<OutT>(y + e1, b);
}

// Row gather fused with dequantisation: Y[i, :] = dense(W[ids[i], :]).  A row whose id is outside [0, n_rows) is
// written as zeros.  blockIdx.y walks the requested rows, blockIdx.x the K / 2048 column chunks.
template <int TYPE, typename OutT>
__global__ __launch_bounds__(256) void dequant_rows_kernel(const uint8_t* __restrict__ w, const int64_t* __restrict__ ids,
                                                            int64_t n_ids, int64_t n_rows, int64_t K, OutT* __restrict__ y) {
  const int64_t c0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (c0 >= K) return;
  for (int64_t i = blockIdx.y; i < n_ids; i += gridDim.y) {
    const int64_t row = ids[i];
    OutT* dst = y + i * K + c0;
    if (row < 0 || row >= n_rows) {
      alignas(16) OutT zero[8] = {};
      store8<OutT>(dst, zero);
    } else {
      dequant8<TYPE, OutT>(w, row * K + c0, dst);
    }
  }
}

template <int TYPE>
static int launch_dequant(const void* w, void* y, int ydtype, int64_t nelem, hipStream_t stream) {
  const unsigned grid = (unsigned)((nelem + 4095) / 4096);
  GGUF_DISPATCH_DTYPE(ydtype, hipLaunchKernelGGL((dequant_kernel<TYPE, scalar_t>), dim3(grid), dim3(256), 0, stream,
                                                 (const uint8_t*)w, (scalar_t*)y, nelem));
  return launch_status();
}

template <int TYPE>
static int launch_dequant_rows(const void* w, const int64_t* ids, int64_t n_ids, int64_t n_rows, int64_t K, void* y,
                               int ydtype, hipStream_t stream) {
  const dim3 grid((unsigned)((K / 8 + 255) / 256), (unsigned)(n_ids < 32768 ? n_ids : 32768));
  GGUF_DISPATCH_DTYPE(ydtype, hipLaunchKernelGGL((dequant_rows_kernel<TYPE, scalar_t>), grid, dim3(256), 0, stream,
                                                 (const uint8_t*)w, ids, n_ids, n_rows, K, (scalar_t*)y));
  return launch_status();
}

}  // namespace gguf

extern "C" int gguf_dequantize_rows(const void* W, int type, const int64_t* row_ids, int64_t n_ids, int64_t n_rows, int64_t K,
                                    void* Y, int ydtype, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (n_ids < 0 || n_rows < 0 || K <= 0 || K % qk != 0 || K / 8 / 256 > 0x7FFFFFFFLL) return GGUF_ERR_SHAPE;
  if (ydtype < 0 || ydtype > 2) return GGUF_ERR_DTYPE;
  if (n_ids == 0) return GGUF_OK;
  if (!W || !row_ids || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (type) {
    case T_Q4_0: return launch_dequant_rows<T_Q4_0>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q4_1: return launch_dequant_rows<T_Q4_1>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q5_0: return launch_dequant_rows<T_Q5_0>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q5_1: return launch_dequant_rows<T_Q5_1>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q8_0: return launch_dequant_rows<T_Q8_0>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q2_K: return launch_dequant_rows<T_Q2_K>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q3_K: return launch_dequant_rows<T_Q3_K>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q4_K: return launch_dequant_rows<T_Q4_K>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q5_K: return launch_dequant_rows<T_Q5_K>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_Q6_K: return launch_dequant_rows<T_Q6_K>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ2_XXS: return launch_dequant_rows<T_IQ2_XXS>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ2_XS: return launch_dequant_rows<T_IQ2_XS>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ3_XXS: return launch_dequant_rows<T_IQ3_XXS>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ1_S: return launch_dequant_rows<T_IQ1_S>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ4_NL: return launch_dequant_rows<T_IQ4_NL>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ3_S: return launch_dequant_rows<T_IQ3_S>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ2_S: return launch_dequant_rows<T_IQ2_S>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ4_XS: return launch_dequant_rows<T_IQ4_XS>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    case T_IQ1_M: return launch_dequant_rows<T_IQ1_M>(W, row_ids, n_ids, n_rows, K, Y, ydtype, s);
    default: return GGUF_ERR_TYPE;
  }
}

extern "C" int gguf_dequantize(const void* W, int type, void* Y, int ydtype, int64_t nelem, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (nelem < 0 || nelem % qk != 0 || nelem / 8 / 256 > 0x7FFFFFFFLL) return GGUF_ERR_SHAPE;
  if (ydtype < 0 || ydtype > 2) return GGUF_ERR_DTYPE;
  if (nelem == 0) return GGUF_OK;
  if (!W || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (type) {
    case T_Q4_0: return launch_dequant<T_Q4_0>(W, Y, ydtype, nelem, s);
    case T_Q4_1: return launch_dequant<T_Q4_1>(W, Y, ydtype, nelem, s);
    case T_Q5_0: return launch_dequant<T_Q5_0>(W, Y, ydtype, nelem, s);
    case T_Q5_1: return launch_dequant<T_Q5_1>(W, Y, ydtype, nelem, s);
    case T_Q8_0: return launch_dequant<T_Q8_0>(W, Y, ydtype, nelem, s);
    case T_Q2_K: return launch_dequant<T_Q2_K>(W, Y, ydtype, nelem, s);
    case T_Q3_K: return launch_dequant<T_Q3_K>(W, Y, ydtype, nelem, s);
    case T_Q4_K: return launch_dequant<T_Q4_K>(W, Y, ydtype, nelem, s);
    case T_Q5_K: return launch_dequant<T_Q5_K>(W, Y, ydtype, nelem, s);
    case T_Q6_K: return launch_dequant<T_Q6_K>(W, Y, ydtype, nelem, s);
    case T_IQ2_XXS: return launch_dequant<T_IQ2_XXS>(W, Y, ydtype, nelem, s);
    case T_IQ2_XS: return launch_dequant<T_IQ2_XS>(W, Y, ydtype, nelem, s);
    case T_IQ3_XXS: return launch_dequant<T_IQ3_XXS>(W, Y, ydtype, nelem, s);
    case T_IQ1_S: return launch_dequant<T_IQ1_S>(W, Y, ydtype, nelem, s);
    case T_IQ4_NL: return launch_dequant<T_IQ4_NL>(W, Y, ydtype, nelem, s);
    case T_IQ3_S: return launch_dequant<T_IQ3_S>(W, Y, ydtype, nelem, s);
    case T_IQ2_S: return launch_dequant<T_IQ2_S>(W, Y, ydtype, nelem, s);
    case T_IQ4_XS: return launch_dequant<T_IQ4_XS>(W, Y, ydtype, nelem, s);
    case T_IQ1_M: return launch_dequant<T_IQ1_M>(W, Y, ydtype, nelem, s);
    default: return GGUF_ERR_TYPE;
  }
}
