// Prefill-path GEMM on packed GGUF weights with q8_1 activations, on gfx950 int8 MFMA.
//
//   Y[m, n] = sum_kb  d8[m, kb] * dw[n, kb] * S[m, n, kb]  ( - offset terms )
//   S[m, n, kb] = sum over the 32 (or 16) elements of block kb of  xq[m, k] * wq[n, k]      (int32)
//
// The reference computes S with dp4a on the vector ALU from re-packed LDS tiles
// (csrc/gguf/mmq.cuh:2-104, vecdotq.cuh load_tiles_* / vec_dot_*_mul_mat).  Here S is
// one v_mfma_i32_32x32x32_i8 per 32x32 output tile and 32-element block (two
// v_mfma_i32_32x32x16_i8 for formats whose weight scale changes every 16 elements), and
// the vector ALU only rescales: convert, multiply by the activation scale, fused
// multiply-add with the weight scale into an fp32 accumulator.
//
// Work split: a workgroup of four waves owns an (M_T x N_T) output tile and walks K in
// steps of 128 elements.  Per step it stages the q8_1 activations (int8 + block scales)
// and unpacks the GGUF blocks of its N_T weight rows to plain int8 + per-block fp32
// scales in LDS; every wave then owns a (32*TM x 32*TN) sub-tile.  MFMA operands:
// A = activations (rows = tokens), B = weights (columns = output features), so a lane
// holds one output feature n and 16 token rows, the weight scale is a per-lane scalar
// and stores to Y are contiguous across lanes.
//
// The same kernel runs the grouped MoE contraction (reference: csrc/gguf/moe.cuh:5-129):
// token rows are gathered through sorted_token_ids, the weight base moves to the block's
// expert, and results scatter to the rows the slots name.
#include "gguf_common.h"
#include "grid_codes.h"

namespace gguf {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// The element is taken by value first: a bit cast applied directly to a vector element expression reads
// element 0 with this compiler.
__device__ __forceinline__ float carrier_to_float(int bits) { return __int_as_float(bits) - 12582912.0f; }

constexpr int KS = 128;     // K elements per step
// LDS row pitch in bytes.  K=32 operands are read 16 bytes per lane: a 16-byte skew (144) spreads 8 consecutive rows
// over all banks.  K=16 operands are read 8 bytes per lane: an 8-byte skew (136) spreads 16 consecutive rows.
template <int G> struct Pitch { static constexpr int value = G == 32 ? KS + 16 : KS + 8; };

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
  struct Raw { uint16_t d; uint4 q; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const uint8_t* b = row + (int64_t)kb * BS;
    Raw r; r.d = ld<uint16_t>(b); r.q = ld<uint4>(b + 2); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const uint32_t w[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = w[i] & 0x0F0F0F0Fu; q[4 + i] = (w[i] >> 4) & 0x0F0F0F0Fu; }
    s0 = (float)__builtin_bit_cast(_Float16, r.d); s1 = s0; mn = 8.0f * s0;
  }
};

struct MQ8_0 {  // vecdotq.cuh:165-177, 869-921
  static constexpr int QK = 32, BS = 34, G = 32;
  static constexpr bool HAS_MIN = false;
  struct Raw { uint16_t d; uint4 q0, q1; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const uint8_t* b = row + (int64_t)kb * BS;
    Raw r; r.d = ld<uint16_t>(b); r.q0 = ld<uint4>(b + 2); r.q1 = ld<uint4>(b + 18); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    q[0] = r.q0.x; q[1] = r.q0.y; q[2] = r.q0.z; q[3] = r.q0.w; q[4] = r.q1.x; q[5] = r.q1.y; q[6] = r.q1.z; q[7] = r.q1.w;
    s0 = (float)__builtin_bit_cast(_Float16, r.d); s1 = s0; mn = 0.0f;
  }
};

struct MQ4_K {  // vecdotq.cuh:353-379, 1204-1277
  static constexpr int QK = 256, BS = 144, G = 32;
  static constexpr bool HAS_MIN = true;
  struct Raw { uint4 hdr, v0, v1; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, j = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r; r.hdr = ld<uint4>(b); r.v0 = ld<uint4>(b + 16 + 32 * (j >> 1)); r.v1 = ld<uint4>(b + 32 + 32 * (j >> 1)); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
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
};

struct MQ6_K {  // vecdotq.cuh:467-491, 1443-1529: two int8 sub-scales per q8_1 block
  static constexpr int QK = 256, BS = 210, G = 16;
  static constexpr bool HAS_MIN = false;
  struct Raw { uint4 l0, l1, h0, h1; uint16_t sc, d; };
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
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const int t = kb & 3;
    const uint32_t lw[8] = {r.l0.x, r.l0.y, r.l0.z, r.l0.w, r.l1.x, r.l1.y, r.l1.z, r.l1.w};
    const uint32_t hw[8] = {r.h0.x, r.h0.y, r.h0.z, r.h0.w, r.h1.x, r.h1.y, r.h1.z, r.h1.w};
    const int shl = (t >> 1) ? 4 : 0, shh = 2 * t;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t v = ((lw[i] >> shl) & 0x0F0F0F0Fu) | (((hw[i] >> shh) & 0x03030303u) << 4);
      q[i] = ((v | 0x80808080u) - 0x20202020u) ^ 0x80808080u;  // every byte minus 32, no borrow between bytes
    }
    const float d = (float)__builtin_bit_cast(_Float16, r.d);
    s0 = d * (float)(int8_t)(r.sc & 0xFF);
    s1 = d * (float)(int8_t)(r.sc >> 8);
    mn = 0.0f;
  }
};

__device__ __forceinline__ int lut16q(uint32_t idx) {  // kvalues_iq4nl lookup of four indices, one per byte
  constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
  const uint32_t sel = idx & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(T3, T2, sel);
  const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
  return (int)((hi & m) | (lo & ~m));
}

struct MIQ4_XS {  // extension: the reference has no MMQ tiles for i-quants (gguf_kernel.cu:236-287)
  static constexpr int QK = 256, BS = 136, G = 32;
  static constexpr bool HAS_MIN = false;
  struct Raw { uint2 hdr; uint4 v; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, ib = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r; r.hdr = ld<uint2>(b); r.v = ld<uint4>(b + 8 + 16 * ib); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const int ib = kb & 7;
    const uint32_t w[4] = {r.v.x, r.v.y, r.v.z, r.v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = (uint32_t)lut16q(w[i] & 0x0F0F0F0Fu); q[4 + i] = (uint32_t)lut16q((w[i] >> 4) & 0x0F0F0F0Fu); }
    const int ls = (int)(((r.hdr.y >> (4 * ib)) & 0xF) | ((((r.hdr.x >> 16) >> (2 * ib)) & 3) << 4));
    s0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(r.hdr.x & 0xFFFF)) * (float)(ls - 32);
    s1 = s0; mn = 0.0f;
  }
};

struct MIQ2_XXS {  // extension, see MIQ4_XS
  static constexpr int QK = 256, BS = 66, G = 32;
  static constexpr bool HAS_MIN = false;
  struct Raw { uint16_t d; uint2 g; };
  static __device__ __forceinline__ Raw fetch(const uint8_t* row, int kb) {
    const int sb = kb >> 3, ib = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Raw r; r.d = ld<uint16_t>(b); r.g = ld<uint2>(b + 2 + 8 * ib); return r;
  }
  static __device__ __forceinline__ void unpack(const Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
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

// --------------------------------------------------------------------------------------------
struct MoeArgs {
  const int32_t* sorted_token_ids;
  const int32_t* expert_ids;
  const int32_t* num_tokens_post_padded;
  int64_t expert_stride;  // bytes
  int top_k;
  int num_pairs;          // tokens * top_k
};

template <class F, int WM, int WN, int TM, int TN, typename T, bool MOE>
__global__ __launch_bounds__(64 * WM * WN, 2) void mmq_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                       T* __restrict__ Y, int M, int N, int K, int64_t ws_row_bytes,
                                                       MoeArgs moe) {
  constexpr int NT = 64 * WM * WN;       // threads per workgroup
  constexpr int LDK = Pitch<F::G>::value;
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  constexpr int NG = KS / F::G;          // weight scales per row per step
  constexpr int AQ = (M_T * 8 + NT - 1) / NT;  // 8-byte/16-byte activation granules per thread and step
  constexpr int AS = (M_T * 4 + NT - 1) / NT;  // activation block scales per thread and step
  constexpr int WP = (N_T * 4 + NT - 1) / NT;  // (weight row, 32-block) pairs per thread and step
  extern __shared__ __align__(16) char smem[];
  int8_t* xq = (int8_t*)smem;                       // [M_T][LDK]
  int8_t* wq = xq + M_T * LDK;                      // [N_T][LDK]
  float* xd = (float*)(wq + N_T * LDK);             // [4][M_T]   q8_1 block scales
  float* xa = xd + 4 * M_T;                         // [4][M_T]   q8_1 block sums (HAS_MIN)
  float* wsc = xa + (F::HAS_MIN ? 4 * M_T : 0);     // [NG][N_T]
  float* wmn = wsc + NG * N_T;                      // [4][N_T]   (HAS_MIN)

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WN, wn = wave % WN;
  const int m_base = blockIdx.y * M_T, n_base = blockIdx.x * N_T;
  const int Kp = (int)q8_kp(K);
  const int64_t rowbytes = (int64_t)(K / F::QK) * F::BS;
  const int nkb_total = K >> 5;

  if (MOE) {
    static_assert(!MOE || M_T == 32, "one expert per 32 sorted slots");
    if (m_base >= moe.num_tokens_post_padded[0]) return;
    const int e = moe.expert_ids[blockIdx.y];
    if (e < 0 || e > 255) return;
    W += (int64_t)e * moe.expert_stride;
  }

  // ---- per-thread staging plan, fixed over K: which rows this thread fetches
  const char* aq_src[AQ];   // activation quants: row base + 16 * granule
  bool aq_ok[AQ];
#pragma unroll
  for (int i = 0; i < AQ; ++i) {
    const int p = tid + NT * i, m = min(p >> 3, M_T - 1), g = p & 7;
    int src = m_base + m;
    bool ok = p < M_T * 8;
    if (MOE) {
      const int pair = moe.sorted_token_ids[src];
      ok = ok && pair < moe.num_pairs;
      src = pair < moe.num_pairs ? pair / moe.top_k : 0;
    } else {
      src = min(src, M - 1);
    }
    aq_src[i] = ws + (int64_t)src * ws_row_bytes + 16 * g;
    aq_ok[i] = ok;
  }
  const float* as_src[AS];  // activation block scales
  bool as_ok[AS];
#pragma unroll
  for (int i = 0; i < AS; ++i) {
    const int p = tid + NT * i, m = min(p >> 2, M_T - 1), kb = p & 3;
    int src = m_base + m;
    bool ok = p < M_T * 4;
    if (MOE) {
      const int pair = moe.sorted_token_ids[src];
      ok = ok && pair < moe.num_pairs;
      src = pair < moe.num_pairs ? pair / moe.top_k : 0;
    } else {
      src = min(src, M - 1);
    }
    as_src[i] = (const float*)(ws + (int64_t)src * ws_row_bytes + Kp) + kb;
    as_ok[i] = ok;
  }
  const uint8_t* w_src[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int p = tid + NT * i, n = min(p >> 2, N_T - 1);
    w_src[i] = W + (int64_t)min(n_base + n, N - 1) * rowbytes;
  }

  uint4 r_aq[AQ];
  float r_ad[AS], r_aa[AS];
  typename F::Raw r_w[WP];

  auto fetch = [&](int k0) {
    const int kb0 = k0 >> 5;
#pragma unroll
    for (int i = 0; i < AQ; ++i) r_aq[i] = *(const uint4*)(aq_src[i] + k0);  // q8 rows are padded to 512, always readable
#pragma unroll
    for (int i = 0; i < AS; ++i) {
      r_ad[i] = as_src[i][kb0];
      if (F::HAS_MIN) r_aa[i] = as_src[i][kb0 + Kp / 32];
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int kb = min(kb0 + ((tid + NT * i) & 3), nkb_total - 1);  // clamped: a step past K re-reads the last block
      r_w[i] = F::fetch(w_src[i], kb);
    }
  };
  auto stash = [&](int k0) {
    const int kb0 = k0 >> 5;
#pragma unroll
    for (int i = 0; i < AQ; ++i) {
      const int p = tid + NT * i, m = p >> 3, g = p & 7;
      if (p < M_T * 8) {
        const bool ok = aq_ok[i] && kb0 + (g >> 1) < nkb_total;
        const uint4 v = ok ? r_aq[i] : make_uint4(0, 0, 0, 0);
        if (LDK % 16 == 0) {
          *(uint4*)(xq + m * LDK + 16 * g) = v;
        } else {
          *(uint2*)(xq + m * LDK + 16 * g) = make_uint2(v.x, v.y);
          *(uint2*)(xq + m * LDK + 16 * g + 8) = make_uint2(v.z, v.w);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < AS; ++i) {
      const int p = tid + NT * i, m = p >> 2, kb = p & 3;
      if (p < M_T * 4) {
        const bool ok = as_ok[i] && kb0 + kb < nkb_total;
        xd[kb * M_T + m] = ok ? r_ad[i] : 0.0f;
        if (F::HAS_MIN) xa[kb * M_T + m] = ok ? r_aa[i] : 0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + NT * i, n = p >> 2, kb = p & 3;
      if (p >= N_T * 4) continue;
      uint32_t q[8];
      float s0, s1, mn;
      F::unpack(r_w[i], kb0 + kb, q, s0, s1, mn);
      if (kb0 + kb >= nkb_total) {
#pragma unroll
        for (int t = 0; t < 8; ++t) q[t] = 0;
        s0 = s1 = mn = 0.0f;
      }
      if (LDK % 16 == 0) {
        *(uint4*)(wq + n * LDK + 32 * kb) = make_uint4(q[0], q[1], q[2], q[3]);
        *(uint4*)(wq + n * LDK + 32 * kb + 16) = make_uint4(q[4], q[5], q[6], q[7]);
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) *(uint2*)(wq + n * LDK + 32 * kb + 8 * t) = make_uint2(q[2 * t], q[2 * t + 1]);
      }
      if (F::G == 32) {
        wsc[kb * N_T + n] = s0;
      } else {
        wsc[(2 * kb) * N_T + n] = s0;
        wsc[(2 * kb + 1) * N_T + n] = s1;
      }
      if (F::HAS_MIN) wmn[kb * N_T + n] = mn;
    }
  };

  float acc[TM][TN][16];
#pragma unroll
  for (int j = 0; j < TM; ++j)
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][i][r] = 0.0f;

  const int lrow = lane & 31, lhalf = lane >> 5;

  // int32 -> fp32 without a convert: the MFMA accumulates onto 0x4B400000 in every element, so the integer
  // result S (|S| < 2^22 for 32 products of int8) comes out as the bit pattern of the float 12582912 + S,
  // and one exact fp32 subtraction recovers S.  v_cvt_f32_i32 issues at half the rate of v_sub_f32 here.
  v16i carrier;
#pragma unroll
  for (int r = 0; r < 16; ++r) carrier[r] = 0x4B400000;

  fetch(0);
  stash(0);
  __syncthreads();

  for (int k0 = 0; k0 < K; k0 += KS) {
    const bool more = k0 + KS < K;
#ifdef GGUF_DBG_NOFETCH
    if (more && K < 0) fetch(k0 + KS);
#else
    if (more) fetch(k0 + KS);  // next step's global loads fly during this step's MFMA phase
#endif

    // ---- contract this step from LDS
#ifdef GGUF_DBG_NOCOMPUTE
    if (K < 0)
#endif
#pragma unroll 1
    for (int kb = 0; kb < 4; ++kb) {
      float d8[TM][16];
      float a8[TM][16];
      v4i af[TM];
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const int mrow = 32 * (wm * TM + j);
        if (F::G == 32) af[j] = *(const v4i*)(xq + (mrow + lrow) * LDK + 32 * kb + 16 * lhalf);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float4 v = *(const float4*)(xd + kb * M_T + mrow + 8 * g + 4 * lhalf);
          d8[j][4 * g] = v.x; d8[j][4 * g + 1] = v.y; d8[j][4 * g + 2] = v.z; d8[j][4 * g + 3] = v.w;
          if (F::HAS_MIN) {
            const float4 u = *(const float4*)(xa + kb * M_T + mrow + 8 * g + 4 * lhalf);
            a8[j][4 * g] = u.x; a8[j][4 * g + 1] = u.y; a8[j][4 * g + 2] = u.z; a8[j][4 * g + 3] = u.w;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int ncol = 32 * (wn * TN + i) + lrow;
        if (F::G == 32) {
          const v4i bf = *(const v4i*)(wq + ncol * LDK + 32 * kb + 16 * lhalf);
          const float dw = wsc[kb * N_T + ncol];
          const float mw = F::HAS_MIN ? wmn[kb * N_T + ncol] : 0.0f;
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            const v16i s = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[j], bf, carrier, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float f = carrier_to_float(s[r]);  // exact int -> float
              acc[j][i][r] = __builtin_fmaf(f * dw, d8[j][r], acc[j][i][r]);
              if (F::HAS_MIN) acc[j][i][r] = __builtin_fmaf(-a8[j][r], mw, acc[j][i][r]);
            }
          }
        } else {
          // weight scale changes every 16 elements: one K=16 MFMA per half block.  In the 16-byte operand a lane
          // already holds, half h of the block is bytes [8h, 8h+8) of lane half 0 and of lane half 1; the K=16
          // shape wants 8 consecutive k per lane half, so the operands are re-read with that addressing.
          const float dwa = wsc[(2 * kb) * N_T + ncol], dwb = wsc[(2 * kb + 1) * N_T + ncol];
          const long b0 = *(const long*)(wq + ncol * LDK + 32 * kb + 8 * lhalf);
          const long b1 = *(const long*)(wq + ncol * LDK + 32 * kb + 16 + 8 * lhalf);
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            const int mrow = 32 * (wm * TM + j);
            const long a0 = *(const long*)(xq + (mrow + lrow) * LDK + 32 * kb + 8 * lhalf);
            const long a1 = *(const long*)(xq + (mrow + lrow) * LDK + 32 * kb + 16 + 8 * lhalf);
            const v16i sa = __builtin_amdgcn_mfma_i32_32x32x16_i8(a0, b0, carrier, 0, 0, 0);
            const v16i sb2 = __builtin_amdgcn_mfma_i32_32x32x16_i8(a1, b1, carrier, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float fa = carrier_to_float(sa[r]);
              const float fb = carrier_to_float(sb2[r]);
              const float t = __builtin_fmaf(fb, dwb, fa * dwa);
              acc[j][i][r] = __builtin_fmaf(t, d8[j][r], acc[j][i][r]);
            }
          }
        }
      }
    }
    __syncthreads();
#ifdef GGUF_DBG_NOSTASH
    if (more && K < 0) {
#else
    if (more) {
#endif
      stash(k0 + KS);
      __syncthreads();
    }
  }

  // ---- store: lane = one output feature, 16 token rows per tile
#pragma unroll
  for (int j = 0; j < TM; ++j) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int mt = m_base + 32 * (wm * TM + j) + 8 * (r >> 2) + 4 * lhalf + (r & 3);
      int64_t dst;
      bool ok;
      if (MOE) {
        const int pair = moe.sorted_token_ids[mt];
        ok = pair < moe.num_pairs;
        dst = pair;
      } else {
        ok = mt < M;
        dst = mt;
      }
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int n = n_base + 32 * (wn * TN + i) + lrow;
        if (ok && n < N) Y[dst * N + n] = from_f32<T>(acc[j][i][r]);
      }
    }
  }
}

template <class F, int WM, int WN, int TM, int TN, bool MOE>
static constexpr size_t mmq_lds_bytes() {
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  return (size_t)(M_T + N_T) * Pitch<F::G>::value + (size_t)4 * M_T * 4 * (F::HAS_MIN ? 2 : 1) +
         (size_t)(KS / F::G) * N_T * 4 + (F::HAS_MIN ? (size_t)4 * N_T * 4 : 0);
}

template <class F, int WM, int WN, int TM, int TN, typename T, bool MOE>
static void launch_mmq(const void* W, const void* ws, void* Y, int M, int N, int K, int m_tiles, const MoeArgs& moe,
                       hipStream_t stream) {
  constexpr int N_T = 32 * WN * TN;
  constexpr size_t lds = mmq_lds_bytes<F, WM, WN, TM, TN, MOE>();
  auto kern = mmq_kernel<F, WM, WN, TM, TN, T, MOE>;
  static bool configured = false;  // opt in to > 64 KB of dynamic LDS once per instantiation
  if (!configured) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3((N + N_T - 1) / N_T, m_tiles), dim3(64 * WM * WN), lds, stream, (const uint8_t*)W, (const char*)ws,
                     (T*)Y, M, N, K, q8_row_bytes(K), moe);
}

int quantize_q8_1(const void* x, int xdtype, void* ws, int64_t M, int64_t K, hipStream_t stream);

template <class F, typename T>
static int mmq_typed(const void* W, const void* ws, void* Y, int M, int N, int K, hipStream_t stream) {
  MoeArgs none = {};
  if (M <= 64) {
    launch_mmq<F, 2, 2, 1, 2, T, false>(W, ws, Y, M, N, K, (M + 63) / 64, none, stream);      // 64 x 128
  } else {
    launch_mmq<F, 4, 2, 1, 2, T, false>(W, ws, Y, M, N, K, (M + 127) / 128, none, stream);    // 128 x 128, 8 waves
  }
  return launch_status();
}

template <class F>
static int mmq_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (mmq_typed<F, scalar_t>(W, ws, Y, M, N, K, s)));
  return GGUF_ERR_DTYPE;
}

template <class F, typename T>
static int moe_typed(const void* W, const void* ws, void* Y, int N, int K, int num_sorted, const MoeArgs& moe,
                     hipStream_t stream) {
  launch_mmq<F, 1, 4, 1, 2, T, true>(W, ws, Y, 0, N, K, num_sorted / 32, moe, stream);  // 32 slots x 256
  return launch_status();
}

template <class F>
static int moe_fmt(const void* W, const void* ws, void* Y, int dtype, int N, int K, int num_sorted, const MoeArgs& moe,
                   hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_typed<F, scalar_t>(W, ws, Y, N, K, num_sorted, moe, s)));
  return GGUF_ERR_DTYPE;
}

__global__ void zero_rows_kernel(uint4* __restrict__ p, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) p[i] = make_uint4(0, 0, 0, 0);
}

static bool mmq_type_ok(int type) {
  switch (type) {
    case T_Q4_0: case T_Q8_0: case T_Q4_K: case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: return true;
    default: return false;
  }
}

}  // namespace gguf

extern "C" int gguf_mmq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N,
                        int64_t K, int64_t M, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0 || !mmq_type_ok(type)) return GGUF_ERR_TYPE;
  if (N < 0 || M < 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL || M > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || M == 0) return GGUF_OK;
  if (!W || !x || !q8_workspace || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const int rc = quantize_q8_1(x, xdtype, q8_workspace, M, K, s);
  if (rc != GGUF_OK) return rc;
  switch (type) {
    case T_Q4_0: return mmq_fmt<MQ4_0>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_Q8_0: return mmq_fmt<MQ8_0>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_Q4_K: return mmq_fmt<MQ4_K>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_Q6_K: return mmq_fmt<MQ6_K>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_IQ4_XS: return mmq_fmt<MIQ4_XS>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_IQ2_XXS: return mmq_fmt<MIQ2_XXS>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
  }
  return GGUF_ERR_TYPE;
}

extern "C" int gguf_moe_block_size(int type) { return gguf::block_elems(type) ? 32 : 0; }

extern "C" int gguf_moe_mmq(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                            const int32_t* sorted_token_ids, const int32_t* expert_ids,
                            const int32_t* num_tokens_post_padded, int64_t num_sorted, void* Y, int type, int64_t N,
                            int64_t K, int64_t top_k, int64_t tokens, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0 || !mmq_type_ok(type)) return GGUF_ERR_TYPE;
  if (N < 0 || tokens < 0 || top_k <= 0 || num_sorted < 0 || K <= 0 || K % qk != 0 || expert_stride_bytes < 0 ||
      tokens * top_k > 0x7FFFFFF0LL || N > 0x7FFFFFF0LL)
    return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || tokens == 0) return GGUF_OK;
  if (!X || !q8_workspace || !W || !sorted_token_ids || !expert_ids || !num_tokens_post_padded || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  // rows that no slot names stay zero, as with the reference's zero-filled output (gguf_kernel.cu:301-302)
  const int64_t ybytes = tokens * top_k * N * (xdtype == GGUF_DTYPE_F32 ? 4 : 2);
  const int64_t n16 = ybytes / 16;
  if (ybytes % 16 != 0) return GGUF_ERR_SHAPE;
  hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, (uint4*)Y, n16);
  const int rc = quantize_q8_1(X, xdtype, q8_workspace, tokens, K, s);
  if (rc != GGUF_OK) return rc;
  MoeArgs moe = {sorted_token_ids, expert_ids, num_tokens_post_padded, expert_stride_bytes, (int)top_k, (int)(tokens * top_k)};
  const int ns = (int)(num_sorted / 32 * 32);  // a trailing partial block is ignored, like the reference's integer division
  if (ns == 0) return launch_status();
  switch (type) {
    case T_Q4_0: return moe_fmt<MQ4_0>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_Q8_0: return moe_fmt<MQ8_0>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_Q4_K: return moe_fmt<MQ4_K>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_Q6_K: return moe_fmt<MQ6_K>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_IQ4_XS: return moe_fmt<MIQ4_XS>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_IQ2_XXS: return moe_fmt<MIQ2_XXS>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
  }
  return GGUF_ERR_TYPE;
}
