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

__device__ __forceinline__ void scale_min_k4(const uint8_t* __restrict__ s, int j, int& sc, int& mn) {
  if (j < 4) {
    sc = s[j] & 63;
    mn = s[j + 4] & 63;
  } else {
    sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4);
    mn = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
  }
}

// Q4_K: dequantize.cuh:165-196.  d1 = d*sc, m1 = dmin*m (each rounded), y = fma(d1, q, -m1).
__device__ __forceinline__ void dq8_q4_k(const uint8_t* __restrict__ w, int64_t e0, h16 (&o)[8]) {
  const uint8_t* blk = w + (e0 >> 8) * 144;
  const int r = (int)(e0 & 255);
  const int j = r >> 5, pos = r & 31;
  const uint4 hdr = *(const uint4*)blk;  // 144-byte blocks keep 16-byte alignment
  const h16 dall = __builtin_bit_cast(h16, (uint16_t)(hdr.x & 0xFFFF));
  const h16 dmin = __builtin_bit_cast(h16, (uint16_t)(hdr.x >> 16));
  const uint32_t sw[3] = {hdr.y, hdr.z, hdr.w};
  int sc, mn;
  scale_min_k4((const uint8_t*)sw, j, sc, mn);
  const h16 d1 = dall * (h16)sc;
  const h16 m1 = dmin * (h16)mn;
  const uint2 q = *(const uint2*)(blk + 16 + 32 * (j >> 1) + pos);
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
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t word = i < 4 ? q.x : q.y;
    o[i] = d * (float)k_kvalues_iq4nl[(word >> (8 * (i & 3) + shq)) & 0xF];
  }
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

template <typename OutT>
__device__ __forceinline__ void store8(OutT* __restrict__ y, const OutT (&v)[8]) {
  if constexpr (sizeof(OutT) == 2) {
    *(uint4*)y = *(const uint4*)v;
  } else {
    ((uint4*)y)[0] = ((const uint4*)v)[0];
    ((uint4*)y)[1] = ((const uint4*)v)[1];
  }
}

template <int TYPE, typename OutT>
__global__ __launch_bounds__(256) void dequant_kernel(const uint8_t* __restrict__ w, OutT* __restrict__ y, int64_t nelem) {
  const int64_t e0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (e0 >= nelem) return;
  alignas(16) OutT out[8];
  if constexpr (TYPE == T_IQ4_XS || TYPE == T_IQ2_XXS) {
    float f[8];
    if constexpr (TYPE == T_IQ4_XS) dq8_iq4_xs(w, e0, f);
    if constexpr (TYPE == T_IQ2_XXS) dq8_iq2_xxs(w, e0, f);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = from_f32<OutT>(f[i]);
  } else {
    h16 h[8];
    if constexpr (TYPE == T_Q4_0) dq8_q4_0(w, e0, h);
    if constexpr (TYPE == T_Q8_0) dq8_q8_0(w, e0, h);
    if constexpr (TYPE == T_Q4_K) dq8_q4_k(w, e0, h);
    if constexpr (TYPE == T_Q6_K) dq8_q6_k(w, e0, h);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = from_half<OutT>(h[i]);
  }
  store8<OutT>(y + e0, out);
}

template <int TYPE>
static int launch_dequant(const void* w, void* y, int ydtype, int64_t nelem, hipStream_t stream) {
  const int64_t threads = nelem / 8;
  const unsigned grid = (unsigned)((threads + 255) / 256);
  GGUF_DISPATCH_DTYPE(ydtype, hipLaunchKernelGGL((dequant_kernel<TYPE, scalar_t>), dim3(grid), dim3(256), 0, stream,
                                                 (const uint8_t*)w, (scalar_t*)y, nelem));
  return launch_status();
}

}  // namespace gguf

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
    case T_Q8_0: return launch_dequant<T_Q8_0>(W, Y, ydtype, nelem, s);
    case T_Q4_K: return launch_dequant<T_Q4_K>(W, Y, ydtype, nelem, s);
    case T_Q6_K: return launch_dequant<T_Q6_K>(W, Y, ydtype, nelem, s);
    case T_IQ4_XS: return launch_dequant<T_IQ4_XS>(W, Y, ydtype, nelem, s);
    case T_IQ2_XXS: return launch_dequant<T_IQ2_XXS>(W, Y, ydtype, nelem, s);
    default: return GGUF_ERR_TYPE;
  }
}
