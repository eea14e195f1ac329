// The older integer tile kernel, kept for the grouped MoE contraction on blocks of 32 slots (the dense product of every
// tile format runs on the pipelined kernel of mmq_i_core.h), and the C entry points of the tile operators.
//
//   Y[m, n] = sum_kb  d8[m, kb] * dw[n, kb] * S[m, n, kb]  ( - offset terms )
//   S[m, n, kb] = sum over the 32 (or 16) elements of block kb of  xq[m, k] * wq[n, k]      (int32)
//
// The reference computes S with dp4a on the vector ALU from re-packed LDS tiles
// (csrc/gguf/mmq.cuh:2-104, vecdotq.cuh load_tiles_* / vec_dot_*_mul_mat).  Here S is
// one v_mfma_i32_32x32x32_i8 per 32x32 output tile and 32-element block (two
// v_mfma_i32_32x32x16_i8 for formats whose weight scale changes every 16 elements), and
// the vector ALU only rescales: per result one fused multiply-add with the weight scale
// (which also turns the int32 into fp32, see seeded_times) and one with the activation
// scale into an fp32 accumulator, plus one for formats with an offset term.  On this
// chip an MFMA and vector-ALU work of other waves on the same SIMD do not run at the
// same time, so those two or three instructions per result, not the MFMA, set the pace.
//
// Work split: a workgroup of four or eight waves owns an (M_T x N_T) output tile and walks K in
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
#include "mmq_formats.h"
#include "q8_1_device.h"

namespace gguf {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// int32 MFMA results reach fp32 without a convert instruction.  Every MFMA accumulates onto the bit pattern of
// the float kSeed = 1.5 * 2^23, whose unit in the last place is 1: for |S| < 2^22 (32 products of int8 stay below
// 2^19) the integer sum kSeedBits + S is the bit pattern of the float kSeed + S.  One fused multiply-add then gives
//   fma(kSeed + S, dw, -kSeed * dw) = RN(S * dw)
// exactly, because kSeed * dw is exact in fp32 whenever dw has at most 22 significant bits, and every weight scale
// here is an fp16 value times an integer of at most 8 bits.  v_cvt_f32_i32 issues at half the rate of v_fma_f32.
constexpr float kSeed = 12582912.0f;
constexpr int kSeedBits = 0x4B400000;
// Takes the MFMA element by value: a bit cast applied directly to a vector element expression reads element 0
// with this compiler.
__device__ __forceinline__ float seeded_times(int bits, float dw, float neg_seed_dw) {
  return __builtin_fmaf(__int_as_float(bits), dw, neg_seed_dw);
}

// acc += v[lane (l & ~3) + T] * c : a fused multiply-add whose first factor is taken from lane T of the caller's
// quad by DPP.  In the 32x32 MFMA result layout register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, so when lane l
// holds a per-row factor for row 8*g + 4*(l/32) + l%4, the factor of register 4*g + T sits in lane T of every quad:
// four registers hold what sixteen would, and they cost four 4-byte LDS reads instead of four 16-byte ones.
// The factor registers are written by LDS loads only, so no VALU-write-to-DPP-read wait states are needed.
template <int T>
__device__ __forceinline__ void fmac_quad(float& acc, float v, float c) {
  static_assert(T >= 0 && T < 4, "lane within the quad");
  if constexpr (T == 0) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(v), "v"(c));
  if constexpr (T == 1) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(v), "v"(c));
  if constexpr (T == 2) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(v), "v"(c));
  if constexpr (T == 3) asm("v_fmac_f32_dpp %0, %1, %2 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf" : "+v"(acc) : "v"(v), "v"(c));
}
// v[lane (l & ~3) + T] as a value (a DPP move the compiler can see and schedule)
template <int T>
__device__ __forceinline__ float quad_get(float v) {
  constexpr int ctrl = T | (T << 2) | (T << 4) | (T << 6);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xF, 0xF, true));
}
template <int R>
__device__ __forceinline__ float row_get(const float (&v)[4]) { return quad_get<R & 3>(v[R >> 2]); }

template <int R>
__device__ __forceinline__ void fmac_row(float& acc, const float (&v)[4], float c) { fmac_quad<R & 3>(acc, v[R >> 2], c); }

// acc[r] += v[row of r] * c[r]  and  acc[r] += v[row of r] * c  over the 16 registers of one MFMA result
__device__ __forceinline__ void rescale16(float (&acc)[16], const float (&v)[4], const float (&c)[16]) {
  fmac_row<0>(acc[0], v, c[0]);    fmac_row<1>(acc[1], v, c[1]);    fmac_row<2>(acc[2], v, c[2]);    fmac_row<3>(acc[3], v, c[3]);
  fmac_row<4>(acc[4], v, c[4]);    fmac_row<5>(acc[5], v, c[5]);    fmac_row<6>(acc[6], v, c[6]);    fmac_row<7>(acc[7], v, c[7]);
  fmac_row<8>(acc[8], v, c[8]);    fmac_row<9>(acc[9], v, c[9]);    fmac_row<10>(acc[10], v, c[10]); fmac_row<11>(acc[11], v, c[11]);
  fmac_row<12>(acc[12], v, c[12]); fmac_row<13>(acc[13], v, c[13]); fmac_row<14>(acc[14], v, c[14]); fmac_row<15>(acc[15], v, c[15]);
}
__device__ __forceinline__ void offset16(float (&acc)[16], const float (&v)[4], float c) {
  fmac_row<0>(acc[0], v, c);   fmac_row<1>(acc[1], v, c);   fmac_row<2>(acc[2], v, c);   fmac_row<3>(acc[3], v, c);
  fmac_row<4>(acc[4], v, c);   fmac_row<5>(acc[5], v, c);   fmac_row<6>(acc[6], v, c);   fmac_row<7>(acc[7], v, c);
  fmac_row<8>(acc[8], v, c);   fmac_row<9>(acc[9], v, c);   fmac_row<10>(acc[10], v, c); fmac_row<11>(acc[11], v, c);
  fmac_row<12>(acc[12], v, c); fmac_row<13>(acc[13], v, c); fmac_row<14>(acc[14], v, c); fmac_row<15>(acc[15], v, c);
}


// Q4_1 / Q5_1 (reference: vec_dot_q8_1_q8_1_impl, vecdotq.cuh:179-198): acc += S * half(d * d8) + half(m * s8),
// both scale products rounded to half precision as __hmul2 does; d, d8, m and s8 are fp16 values held in floats.
template <int R>
__device__ __forceinline__ void half_products1(float& acc, int bits, const float (&d8)[4], const float (&s8)[4], float d, float m) {
  const _Float16 dd = (_Float16)d * (_Float16)row_get<R>(d8);
  const _Float16 ms = (_Float16)m * (_Float16)row_get<R>(s8);
  acc += (__int_as_float(bits) - kSeed) * (float)dd + (float)ms;
}
__device__ __forceinline__ void half_products16(float (&acc)[16], const v16i& s, const float (&d8)[4], const float (&s8)[4], float d, float m) {
  half_products1<0>(acc[0], s[0], d8, s8, d, m);    half_products1<1>(acc[1], s[1], d8, s8, d, m);
  half_products1<2>(acc[2], s[2], d8, s8, d, m);    half_products1<3>(acc[3], s[3], d8, s8, d, m);
  half_products1<4>(acc[4], s[4], d8, s8, d, m);    half_products1<5>(acc[5], s[5], d8, s8, d, m);
  half_products1<6>(acc[6], s[6], d8, s8, d, m);    half_products1<7>(acc[7], s[7], d8, s8, d, m);
  half_products1<8>(acc[8], s[8], d8, s8, d, m);    half_products1<9>(acc[9], s[9], d8, s8, d, m);
  half_products1<10>(acc[10], s[10], d8, s8, d, m); half_products1<11>(acc[11], s[11], d8, s8, d, m);
  half_products1<12>(acc[12], s[12], d8, s8, d, m); half_products1<13>(acc[13], s[13], d8, s8, d, m);
  half_products1<14>(acc[14], s[14], d8, s8, d, m); half_products1<15>(acc[15], s[15], d8, s8, d, m);
}

// Q2_K: acc[r] += d8[row] * (ua[row] * nma + ub[row] * nmb)
template <int R>
__device__ __forceinline__ void group_offsets1(float& acc, const float (&d8)[4], const float (&ua)[4], const float (&ub)[4], float nma, float nmb) {
  const float t = __builtin_fmaf(row_get<R>(ub), nmb, row_get<R>(ua) * nma);
  fmac_row<R>(acc, d8, t);
}
__device__ __forceinline__ void group_offsets16(float (&acc)[16], const float (&d8)[4], const float (&ua)[4], const float (&ub)[4], float nma, float nmb) {
  group_offsets1<0>(acc[0], d8, ua, ub, nma, nmb);   group_offsets1<1>(acc[1], d8, ua, ub, nma, nmb);
  group_offsets1<2>(acc[2], d8, ua, ub, nma, nmb);   group_offsets1<3>(acc[3], d8, ua, ub, nma, nmb);
  group_offsets1<4>(acc[4], d8, ua, ub, nma, nmb);   group_offsets1<5>(acc[5], d8, ua, ub, nma, nmb);
  group_offsets1<6>(acc[6], d8, ua, ub, nma, nmb);   group_offsets1<7>(acc[7], d8, ua, ub, nma, nmb);
  group_offsets1<8>(acc[8], d8, ua, ub, nma, nmb);   group_offsets1<9>(acc[9], d8, ua, ub, nma, nmb);
  group_offsets1<10>(acc[10], d8, ua, ub, nma, nmb); group_offsets1<11>(acc[11], d8, ua, ub, nma, nmb);
  group_offsets1<12>(acc[12], d8, ua, ub, nma, nmb); group_offsets1<13>(acc[13], d8, ua, ub, nma, nmb);
  group_offsets1<14>(acc[14], d8, ua, ub, nma, nmb); group_offsets1<15>(acc[15], d8, ua, ub, nma, nmb);
}

// LDS row pitch in bytes.  K=32 operands are read 16 bytes per lane: a 16-byte skew (144) spreads 8 consecutive rows
// over all banks.  K=16 operands are read 8 bytes per lane: an 8-byte skew (136) spreads 16 consecutive rows.
template <int G, int KS> struct Pitch { static constexpr int value = G == 32 ? KS + 16 : KS + 8; };


// --------------------------------------------------------------------------------------------
// LDS bytes of one group's tiles: int8 activations and weights, then their block scales (a multiple of 16).
template <class F, int WM, int WN, int TM, int TN, int KS>
__host__ __device__ constexpr size_t mmq_group_lds_bytes() {
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN, KB = KS / 32;
  constexpr int XA = !F::HAS_MIN ? 0 : F::MIN16 ? 2 * KB : KB;  // per-row offset factors: block sums, or 16-element quant sums
  constexpr int WMN = !F::HAS_MIN ? 0 : F::MIN16 ? KS / F::G : KB;
  return (size_t)(M_T + N_T) * Pitch<F::G, KS>::value + (size_t)(KB + XA) * M_T * 4 + (size_t)(KS / F::G + WMN) * N_T * 4;
}

// MODE selects how staging and contraction overlap:
//   MODE_PREFETCH  the next step's global loads are issued before this step's MFMA phase and held in registers;
//   MODE_PLAIN     load, stage, contract in turn; latency is covered only by other workgroups on the CU;
//   MODE_KSPLIT    MODE_PLAIN with twice the waves: all of them stage the step together, then each half of the
//                  workgroup contracts half of the step's 32-blocks for the same outputs, and the two partial tiles
//                  are added through LDS at the end.  For shapes with too few output tiles to fill the chip.
enum { MODE_PREFETCH = 0, MODE_PLAIN = 1, MODE_KSPLIT = 3 };

template <class F, int WM, int WN, int TM, int TN, int KS, int OCC, int MODE, typename T, bool MOE, bool GATE = false>
__global__ __launch_bounds__(64 * WM * WN * (MODE == MODE_KSPLIT ? 2 : 1), OCC) void mmq_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                         T* __restrict__ Y, int M, int N, int K, int64_t ws_row_bytes,
                                                         MoeArgs moe, int64_t w_pitch, int64_t ldy, const T* __restrict__ bias, Gate16 gate) {
  static_assert(!GATE || (MOE && TM == 1 && WM == 1 && MODE == MODE_PREFETCH), "the gated epilogue is the MoE tile's");
  constexpr int GW = WM * WN;            // waves that share one set of accumulators' tile
  constexpr int KW = MODE == MODE_KSPLIT ? 2 : 1;  // wave sets splitting the 32-blocks of a step
  constexpr int NT = 64 * GW * KW;       // threads that stage one tile: the whole workgroup
  constexpr int KB = KS / 32;            // q8_1 blocks per step
  constexpr int GR = KS / 16;            // 16-byte granules per activation row and step
  constexpr int LDK = Pitch<F::G, KS>::value;
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  constexpr int NG = KS / F::G;          // weight scales per row per step
  constexpr int AQ = (M_T * GR + NT - 1) / NT;  // activation granules per thread and step
  constexpr int AS = (M_T * KB + NT - 1) / NT;  // activation block scales per thread and step
  constexpr int WP = (N_T * KB + NT - 1) / NT;  // (weight row, 32-block) pairs per thread and step
  extern __shared__ __align__(16) char smem[];
  int8_t* xq = (int8_t*)smem;                       // [M_T][LDK]
  int8_t* wq = xq + M_T * LDK;                      // [N_T][LDK]
  float* xd = (float*)(wq + N_T * LDK);             // [KB][M_T]  q8_1 block scales
  float* xa = xd + KB * M_T;                        // [KB][M_T] q8_1 block sums (HAS_MIN), or [2*KB][M_T] quant sums (MIN16)
  float* wsc = xa + (!F::HAS_MIN ? 0 : F::MIN16 ? 2 * KB * M_T : KB * M_T);  // [NG][N_T]
  float* wmn = wsc + NG * N_T;                      // [KB][N_T]  (HAS_MIN)

  const int tid = (int)threadIdx.x, lane = tid & 63;
  const int kgrp = (tid >> 6) / GW, wave = (tid >> 6) % GW;         // wave-uniform
  const int wm = wave / WN, wn = wave % WN;
  constexpr int KB_MINE = (KS / 32) / KW;                            // 32-blocks of a step this wave contracts
  const int m_base = blockIdx.y * M_T;
  const int n_base = blockIdx.x * (GATE ? N_T / 2 : N_T);   // GATE: in features of one half (see Gate16)
  const int Kp = (int)q8_kp(K);
  const int64_t rowbytes = w_pitch;   // bytes between rows of W: the dense row size unless the caller's tensor is padded
  const int nkb_total = K >> 5;

  if (MOE) {
    static_assert(!MOE || M_T == 32, "one expert per 32 sorted slots");
    if (m_base >= moe.num_tokens_post_padded[0]) return;
    const int e = moe.expert_ids[blockIdx.y];
    if (e < 0 || e > 255) return;   // the reference's guard (moe.cuh:33); callers with more experts are turned away in ops.py
    W += (int64_t)e * moe.expert_stride;
  }

  // ---- per-thread staging plan, fixed over K: which rows this thread fetches
  const char* aq_src[AQ];   // activation quants: row base + 16 * granule
  bool aq_ok[AQ];
#pragma unroll
  for (int i = 0; i < AQ; ++i) {
    const int p = tid + NT * i, m = min(p / GR, M_T - 1), g = p % GR;
    int src = m_base + m;
    bool ok = p < M_T * GR;
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
  const int sum_plane = (MOE && moe.gemv_sums ? 2 : 1) * (Kp / 32);  // planes of a workspace row behind d: s8, then d8 * sum(q)
#pragma unroll
  for (int i = 0; i < AS; ++i) {
    const int p = tid + NT * i, m = min(p / KB, M_T - 1), kb = p % KB;
    int src = m_base + m;
    bool ok = p < M_T * KB;
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
    const int p = tid + NT * i, n = min(p / KB, N_T - 1);
    // GATE: the first half of the columns are features n_base .. of the gate half, the second the same features of up
    const int row = GATE ? (n < N_T / 2 ? 0 : gate.inner) + min(n_base + (n & (N_T / 2 - 1)), gate.inner - 1) : min(n_base + n, N - 1);
    w_src[i] = W + (int64_t)row * rowbytes;
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
      if (F::HAS_MIN && !F::MIN16) r_aa[i] = as_src[i][kb0 + sum_plane];
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int kb = min(kb0 + ((tid + NT * i) % KB), nkb_total - 1);  // clamped: a step past K re-reads the last block
      r_w[i] = F::fetch(w_src[i], kb);
    }
  };
  auto stash = [&](int k0) {
    const int kb0 = k0 >> 5;
#pragma unroll
    for (int i = 0; i < AQ; ++i) {
      const int p = tid + NT * i, m = p / GR, g = p % GR;
      if (p < M_T * GR) {
        const bool ok = aq_ok[i] && kb0 + (g >> 1) < nkb_total;
        const uint4 v = ok ? r_aq[i] : make_uint4(0, 0, 0, 0);
        if (F::MIN16)  // this granule is one 16-element group: its quant sum, for the per-group offset term
          xa[g * M_T + m] = (float)dot4(0x01010101, (int)v.x, dot4(0x01010101, (int)v.y, dot4(0x01010101, (int)v.z, dot4(0x01010101, (int)v.w, 0))));
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
      const int p = tid + NT * i, m = p / KB, kb = p % KB;
      if (p < M_T * KB) {
        const bool ok = as_ok[i] && kb0 + kb < nkb_total;
        xd[kb * M_T + m] = ok ? r_ad[i] : 0.0f;
        if (F::HAS_MIN && !F::MIN16) xa[kb * M_T + m] = ok ? r_aa[i] : 0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + NT * i, n = p / KB, kb = p % KB;
      if (p >= N_T * KB) continue;
      uint32_t q[8];
      float s0, s1, mn, mn1;
      F::unpack(r_w[i], kb0 + kb, q, s0, s1, mn, mn1);
      if (kb0 + kb >= nkb_total) {
#pragma unroll
        for (int t = 0; t < 8; ++t) q[t] = 0;
        s0 = s1 = mn = mn1 = 0.0f;
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
      if (F::HAS_MIN && !F::MIN16) wmn[kb * N_T + n] = mn;
      if (F::MIN16) { wmn[(2 * kb) * N_T + n] = mn; wmn[(2 * kb + 1) * N_T + n] = mn1; }
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

  v16i seed;
#pragma unroll
  for (int r = 0; r < 16; ++r) seed[r] = kSeedBits;

  // one 32-element block of the step in LDS -> accumulators
  auto contract = [&](int kb) {
    float d8[TM][4];   // q8_1 scale of row 8*g + 4*lhalf + lane%4 of tile j, one register per g (see fmac_quad)
    float a8[TM][4];   // q8_1 stored sum, same arrangement
    v4i af[TM];
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      const int mrow = 32 * (wm * TM + j);
      if (F::G == 32) af[j] = *(const v4i*)(xq + (mrow + lrow) * LDK + 32 * kb + 16 * lhalf);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        d8[j][g] = xd[kb * M_T + mrow + 8 * g + 4 * lhalf + (lane & 3)];
        if (F::HAS_MIN && !F::MIN16) a8[j][g] = xa[kb * M_T + mrow + 8 * g + 4 * lhalf + (lane & 3)];
      }
    }
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      const int ncol = 32 * (wn * TN + i) + lrow;
      if (F::G == 32) {
        const v4i bf = *(const v4i*)(wq + ncol * LDK + 32 * kb + 16 * lhalf);
        const float dw = wsc[kb * N_T + ncol];
        const float neg_mw = F::HAS_MIN ? -wmn[kb * N_T + ncol] : 0.0f;
        const float neg_seed_dw = -kSeed * dw;
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const v16i s = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[j], bf, seed, 0, 0, 0);
          if constexpr (F::HALFPROD) {
            half_products16(acc[j][i], s, d8[j], a8[j], dw, -neg_mw);
          } else {
            float c[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) c[r] = seeded_times(s[r], dw, neg_seed_dw);  // = RN(S * dw)
            rescale16(acc[j][i], d8[j], c);
            if (F::HAS_MIN) offset16(acc[j][i], a8[j], neg_mw);
          }
        }
      } else {
        // weight scale changes every 16 elements: one K=16 MFMA per half block.  In the 16-byte operand a lane
        // already holds, half h of the block is bytes [8h, 8h+8) of lane half 0 and of lane half 1; the K=16
        // shape wants 8 consecutive k per lane half, so the operands are re-read with that addressing.
        const float dwa = wsc[(2 * kb) * N_T + ncol], dwb = wsc[(2 * kb + 1) * N_T + ncol];
        const float neg_seed_dwa = -kSeed * dwa, neg_seed_dwb = -kSeed * dwb;
        const long b0 = *(const long*)(wq + ncol * LDK + 32 * kb + 8 * lhalf);
        const long b1 = *(const long*)(wq + ncol * LDK + 32 * kb + 16 + 8 * lhalf);
#pragma unroll
        for (int j = 0; j < TM; ++j) {
          const int mrow = 32 * (wm * TM + j);
          const long a0 = *(const long*)(xq + (mrow + lrow) * LDK + 32 * kb + 8 * lhalf);
          const long a1 = *(const long*)(xq + (mrow + lrow) * LDK + 32 * kb + 16 + 8 * lhalf);
          const v16i sa = __builtin_amdgcn_mfma_i32_32x32x16_i8(a0, b0, seed, 0, 0, 0);
          const v16i sb2 = __builtin_amdgcn_mfma_i32_32x32x16_i8(a1, b1, seed, 0, 0, 0);
          float ca[16], cb[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            ca[r] = seeded_times(sa[r], dwa, neg_seed_dwa);
            cb[r] = seeded_times(sb2[r], dwb, neg_seed_dwb);
          }
          rescale16(acc[j][i], d8[j], ca);
          rescale16(acc[j][i], d8[j], cb);
          if constexpr (F::MIN16) {
            // offset term per 16-element group: d8 * (U_a * -min_a + U_b * -min_b), U = sum of the group's quants
            float ua[4], ub[4];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
              ua[g] = xa[(2 * kb) * M_T + mrow + 8 * g + 4 * lhalf + (lane & 3)];
              ub[g] = xa[(2 * kb + 1) * M_T + mrow + 8 * g + 4 * lhalf + (lane & 3)];
            }
            const float nma = -wmn[(2 * kb) * N_T + ncol], nmb = -wmn[(2 * kb + 1) * N_T + ncol];
            group_offsets16(acc[j][i], d8[j], ua, ub, nma, nmb);
          }
        }
      }
    }
  };

  if constexpr (MODE == MODE_PREFETCH) {
    fetch(0);
    stash(0);
    __syncthreads();
    for (int k0 = 0; k0 < K; k0 += KS) {
      const bool more = k0 + KS < K;
      if (more) fetch(k0 + KS);
#pragma unroll 1
      for (int kb = 0; kb < KB; ++kb) contract(kb);
      __syncthreads();
      if (more) {
        stash(k0 + KS);
        __syncthreads();
      }
    }
  } else if constexpr (MODE == MODE_PLAIN || MODE == MODE_KSPLIT) {
    for (int k0 = 0; k0 < K; k0 += KS) {
      fetch(k0);
      stash(k0);
      __syncthreads();
#pragma unroll 1
      for (int kb = kgrp * KB_MINE; kb < (kgrp + 1) * KB_MINE; ++kb) contract(kb);
      __syncthreads();
    }
    if constexpr (KW == 2) {
      // add the second wave set's partial tile to the first's through LDS (the tiles are free after the last barrier)
      float* red = (float*)smem;
      static_assert((size_t)GW * TM * TN * 16 * 64 * 4 <= mmq_group_lds_bytes<F, WM, WN, TM, TN, KS>(), "partial tile fits the staging area");
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float* slot = red + ((((wave * TM + j) * TN + i) * 16 + r) * 64 + lane);
            if (kgrp == 1) *slot = acc[j][i][r];
          }
      __syncthreads();
      if (kgrp == 1) return;
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int i = 0; i < TN; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[j][i][r] += red[(((wave * TM + j) * TN + i) * 16 + r) * 64 + lane];
    }
  }

  if constexpr (GATE) {
    // ---- the tile's sums, rounded as the operator stores them, meet in LDS (the staging area is free: the loop ends on
    // a barrier); then eight features of a slot per thread, both halves, and every four threads form one q8_1 block
    static_assert((size_t)M_T * N_T * 4 <= mmq_group_lds_bytes<F, WM, WN, TM, TN, KS>(), "the tile of sums fits the staging area");
    float* yt = (float*)smem;   // [M_T][N_T]
#pragma unroll
    for (int r = 0; r < 16; ++r)
#pragma unroll
      for (int i = 0; i < TN; ++i)
        yt[(8 * (r >> 2) + 4 * lhalf + (r & 3)) * N_T + 32 * (wn * TN + i) + lrow] = to_f32<T>(from_f32<T>(acc[0][i][r]));
    __syncthreads();
    constexpr int PARTS = N_T / 2 / 8;   // threads per slot (a multiple of 4: quads stay whole)
    static_assert((M_T * PARTS) % NT == 0 && PARTS % 4 == 0, "every thread takes the same number of (slot, part) items");
#pragma unroll
    for (int it = 0; it < M_T * PARTS / NT; ++it) {
      const int item = tid + NT * it, slot = item / PARTS, part = item % PARTS;
      float xv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) xv[i] = gate1<T>(yt[slot * N_T + 8 * part + i], yt[slot * N_T + N_T / 2 + 8 * part + i], gate.act);
      const Q8Quad qq = q8_1_quantize8(xv);
      const int pair = moe.sorted_token_ids[m_base + slot];
      const int f = n_base + 8 * part;
      if (pair < moe.num_pairs && f < gate.inner) {     // (inner is a multiple of 32: blocks are whole)
        char* row = gate.rows + (int64_t)pair * gate.row_bytes;
        *(uint2*)(row + f) = qq.q;
        if ((part & 3) == 0) {
          float* fd = (float*)(row + gate.kp);
          const int b = f >> 5, nbp = gate.kp >> 5;
          fd[b] = qq.d;
          fd[nbp + b] = qq.s;
          fd[2 * nbp + b] = qq.du;
        }
      }
    }
    return;
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
        if (ok && n < N) Y[dst * ldy + n] = finish<T>(acc[j][i][r], bias, n);
      }
    }
  }
}


template <class F, int WM, int WN, int TM, int TN, int KS, int OCC, int MODE, typename T, bool MOE, bool GATE = false>
static void launch_mmq(const void* W, const void* ws, void* Y, int M, int N, int K, int m_tiles, const MoeArgs& moe,
                       hipStream_t stream, const LinearArgs& la = LinearArgs(), const Gate16& gate = Gate16{}) {
  constexpr int KW = MODE == MODE_KSPLIT ? 2 : 1;
  constexpr int N_T = 32 * WN * TN;
  constexpr size_t lds = mmq_group_lds_bytes<F, WM, WN, TM, TN, KS>();
  static_assert(mmq_group_lds_bytes<F, WM, WN, TM, TN, KS>() % 16 == 0, "group tiles keep 16-byte alignment");
  auto kern = mmq_kernel<F, WM, WN, TM, TN, KS, OCC, MODE, T, MOE, GATE>;
  if constexpr (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, lds, done);
  }
  const int n_tiles = GATE ? (gate.inner + N_T / 2 - 1) / (N_T / 2) : (N + N_T - 1) / N_T;
  hipLaunchKernelGGL(kern, dim3(n_tiles, m_tiles), dim3(64 * WM * WN * KW), lds, stream, (const uint8_t*)W, (const char*)ws,
                     (T*)Y, M, N, K, q8_row_bytes(K), moe, la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS,
                     la.ldy ? la.ldy : (int64_t)N, (const T*)la.bias, gate);
}



template <class F, typename T>
static int moe_typed(const void* W, const void* ws, void* Y, int N, int K, int num_sorted, const MoeArgs& moe,
                     hipStream_t stream) {
  // 32 slots x 256 features; x 128 where the blocks that hold pairs (estimated) times the feature tiles would leave CUs
  // idle (12 blocks of an 8-expert layer at 128 tokens x 16 tiles of [4096,14336]: 192 workgroups for 512 places)
  if (moe_blocks_estimate(num_sorted, moe.num_pairs, 32) * ((N + 255) / 256) < 2.0 * num_cus())
    launch_mmq<F, 1, 4, 1, 1, 128, 2, MODE_PREFETCH, T, true>(W, ws, Y, 0, N, K, num_sorted / 32, moe, stream);
  else
    launch_mmq<F, 1, 4, 1, 2, 128, 2, MODE_PREFETCH, T, true>(W, ws, Y, 0, N, K, num_sorted / 32, moe, stream);
  return launch_status();
}

template <class F>
static int moe_fmt(const void* W, const void* ws, void* Y, int dtype, int N, int K, int num_sorted, const MoeArgs& moe,
                   hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_typed<F, scalar_t>(W, ws, Y, N, K, num_sorted, moe, s)));
  return GGUF_ERR_DTYPE;
}

// The first expert GEMM of a layer on blocks of 32 slots with the gated activation and the q8_1 quantisation of its
// result in the epilogue (see Gate16): W is [experts][2 inner][K packed], a tile is 32 slots x 128 features of both halves.
template <class F>
static int moe_gate_fmt(const void* W, const void* ws, void* q8h, int dtype, int inner, int K, int num_sorted, const MoeArgs& moe, int act,
                        hipStream_t s) {
  const Gate16 gate{(char*)q8h, q8_row_bytes(inner), inner, (int)q8_kp(inner), act};
  GGUF_DISPATCH_DTYPE(dtype, (launch_mmq<F, 1, 4, 1, 2, 128, 2, MODE_PREFETCH, scalar_t, true, true>(W, ws, nullptr, 0, 2 * inner, K, num_sorted / 32,
                                                                                                   moe, s, LinearArgs(), gate));
                      return launch_status());
  return GGUF_ERR_DTYPE;
}

// nbytes of zeros from p (16-byte aligned): whole 16-byte words, then the last thread past them clears the odd bytes
__global__ void zero_rows_kernel(uint4* __restrict__ p, int64_t nbytes) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x, n16 = nbytes >> 4;
  if (i < n16) p[i] = make_uint4(0, 0, 0, 0);
  else if (i == n16) for (int64_t b = n16 << 4; b < nbytes; ++b) ((uint8_t*)p)[b] = 0;
}

#define GGUF_MOE32_FORMATS(CASE) \
  CASE(T_Q4_0, MQ4_0) CASE(T_Q4_1, MQ4_1) CASE(T_Q5_0, MQ5_0) CASE(T_Q5_1, MQ5_1) CASE(T_Q8_0, MQ8_0) CASE(T_Q2_K, MQ2_K) \
  CASE(T_Q3_K, MQ3_K) CASE(T_Q4_K, MQ4_K) CASE(T_Q5_K, MQ5_K) CASE(T_Q6_K, MQ6_K) CASE(T_IQ4_XS, MIQ4_XS) CASE(T_IQ2_XXS, MIQ2_XXS)

// the grouped contraction on blocks of 32 slots, and the gated first GEMM of a layer on them
static int moe_tiles32(const void* W, const void* ws, void* Y, int dtype, int type, int N, int K, int num_sorted, const MoeArgs& moe, hipStream_t s) {
  switch (type) {
#define MOE32_CASE(ID, FMT) case ID: return moe_fmt<FMT>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    GGUF_MOE32_FORMATS(MOE32_CASE)
#undef MOE32_CASE
  }
  return GGUF_ERR_TYPE;
}
static int moe_tiles32_gate(const void* W, const void* ws, void* q8h, int dtype, int type, int inner, int K, int num_sorted, const MoeArgs& moe,
                            int act, hipStream_t s) {
  switch (type) {
#define MOE32_CASE(ID, FMT) case ID: return moe_gate_fmt<FMT>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    GGUF_MOE32_FORMATS(MOE32_CASE)
#undef MOE32_CASE
  }
  return GGUF_ERR_TYPE;
}

static bool mmq_type_ok(int type) {
  switch (type) {
    case T_Q4_0: case T_Q4_1: case T_Q5_0: case T_Q5_1: case T_Q8_0: case T_Q2_K: case T_Q3_K: case T_Q4_K: case T_Q5_K:
    case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: return true;
    default: return false;
  }
}

// The per-pair MoE GEMV (ggml_moe_a8_vec, gguf_kernel.cu:395-530) on the grouped tile kernel, for calls in which the
// experts are shared by enough pairs: the rows are quantized once, the routing sort runs in the workspace behind
// them, and every expert block is one pass over the expert's weights on the matrix cores instead of one pass per
// group of pairs on the vector ALUs.  Results keep the GEMV's semantics: Q4_K / Q5_K take their offset term from the
// quant sums (MoeArgs::gemv_sums); Q5_0 is the one tile format whose tile arithmetic differs from its GEMV
// (vecdotq.cuh:98-125 against :668-749) and stays on the vector kernel.
bool moe_vec_tiles_ok(int type, int64_t pairs, int64_t num_experts, int64_t expert_bytes) {
  if (!mmq_type_ok(type) || type == T_Q5_0) return false;
  return num_experts > 0 && num_experts <= 256 && moe_share_pays(pairs, num_experts, expert_bytes);  // the tile kernel takes expert ids 0..255 (moe.cuh:33)
}

int64_t moe_vec_tiles_workspace(int64_t tokens, int64_t top_k, int64_t K, int64_t num_experts) {
  const int64_t sorted_cap = tokens * top_k + num_experts * 31;
  return tokens * q8_row_bytes(K) + (sorted_cap + sorted_cap / 32 + 2) * 4;
}

// moe_tiles16.hip: the same contraction over blocks of 16 slots, for experts with few pairs
bool moe_tiles16_ok(int type);
int moe_tiles16(const void* W, const void* ws, void* Y, int dtype, int type, int N, int K, int num_sorted, const MoeArgs& moe,
                hipStream_t s);

int moe_vec_tiles(const void* X, int xdtype, void* workspace, const void* W, const int32_t* topk_ids, void* Y, int type, int N,
                  int K, int top_k, int tokens, int act, int num_experts, hipStream_t s) {
  const int pairs = tokens * top_k;
  int rc = quantize_q8_1(X, xdtype, workspace, tokens, K, s, act);
  if (rc != GGUF_OK) return rc;
  // Blocks of 16 slots while an expert has 16 pairs or fewer on average (most of a 32-slot block would be padding),
  // blocks of 32 above.  The routing arrays of either fit the room moe_vec_tiles_workspace reports.
  const int blk = pairs <= 16 * num_experts && moe_tiles16_ok(type) ? 16 : 32;
  const int64_t sorted_cap = (int64_t)pairs + (int64_t)num_experts * (blk - 1);
  const int64_t block_cap = sorted_cap / blk + 1;
  int32_t* sorted = (int32_t*)((char*)workspace + (int64_t)tokens * q8_row_bytes(K));  // rows are a multiple of 4 bytes long
  int32_t* experts = sorted + sorted_cap;
  int32_t* post = experts + block_cap;
  rc = gguf_moe_align_block_size(topk_ids, pairs, num_experts, blk, sorted, sorted_cap, experts, block_cap, post, (gguf_stream_t)s);
  if (rc != GGUF_OK) return rc;
  const int64_t stride = (int64_t)N * (K / block_elems(type)) * block_bytes(type);
  MoeArgs moe = {sorted, experts, post, stride, top_k, pairs, type == T_Q4_K || type == T_Q5_K ? 1 : 0};
  if (blk == 16) return moe_tiles16(W, workspace, Y, xdtype, type, N, K, (int)(sorted_cap / 16 * 16), moe, s);
  const int ns = (int)(sorted_cap / 32 * 32);   // blocks past the padded total see expert -1 and leave
  switch (type) {
    case T_Q4_0: return moe_fmt<MQ4_0>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q4_1: return moe_fmt<MQ4_1>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q5_1: return moe_fmt<MQ5_1>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q8_0: return moe_fmt<MQ8_0>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q2_K: return moe_fmt<MQ2_K>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q3_K: return moe_fmt<MQ3_K>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q4_K: return moe_fmt<MQ4_K>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q5_K: return moe_fmt<MQ5_K>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_Q6_K: return moe_fmt<MQ6_K>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_IQ4_XS: return moe_fmt<MIQ4_XS>(W, workspace, Y, xdtype, N, K, ns, moe, s);
    case T_IQ2_XXS: return moe_fmt<MIQ2_XXS>(W, workspace, Y, xdtype, N, K, ns, moe, s);
  }
  return GGUF_ERR_TYPE;
}

// ---- A MoE layer on the tile kernels for experts shared by a few pairs each (blocks of 16 slots): quantize X and sort
// the pairs once (one launch), first expert GEMM with the gated activation and the quantisation of its result in the epilogue, second
// expert GEMM straight from those rows, weighted sum -- four launches where the separate operators take seven
// (quantize, sort, GEMM, quantize with the activation, sort, GEMM, sum).  The arithmetic is the per-pair operator's on
// both GEMMs (offset sums of the GEMV for Q4_K / Q5_K), every intermediate rounded where the separate steps store it.
int moe_tiles16_gate(const void* W, const void* ws, void* q8h, int dtype, int type, int inner, int K, int num_sorted, const MoeArgs& moe,
                     int act, hipStream_t s);
}  // namespace gguf
extern "C" int gguf_moe_weighted_sum(const void* Y, const float* topk_weights, void* out, int dtype, int64_t tokens, int64_t top_k,
                                     int64_t N, gguf_stream_t stream);
namespace gguf {

static inline int64_t up16(int64_t v) { return (v + 15) / 16 * 16; }

// 16: both formats have 16-slot tiles and the experts see at most 16 pairs each on average; 32: the layer runs on blocks of
// 32 slots; 0: not on the tile kernels (a format without tiles; with the per-pair operator's arithmetic also Q5_0, the
// one format whose tile arithmetic differs from its GEMV's)
int moe_tiles_layer_block(int type13, int type2, int64_t pairs, int64_t num_experts, int64_t I, bool vec_sums) {
  if (num_experts <= 0 || num_experts > 256 || I % 32 != 0) return 0;
  if (vec_sums && (type13 == T_Q5_0 || type2 == T_Q5_0)) return 0;
  if (moe_tiles16_ok(type13) && moe_tiles16_ok(type2) && type13 != T_Q5_0 && type2 != T_Q5_0 && pairs <= 16 * num_experts) return 16;
  return mmq_type_ok(type13) && mmq_type_ok(type2) ? 32 : 0;
}

// [q8_1 rows of X][q8_1 rows of h][second GEMM's result, pairs x N_out][sorted ids, expert ids, padded total]
int64_t moe_tiles_layer_workspace(int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out, int64_t num_experts, int elt, int block) {
  const int64_t pairs = tokens * top_k, sorted_cap = pairs + num_experts * (block - 1);
  return up16(tokens * q8_row_bytes(H)) + up16(pairs * q8_row_bytes(I)) + up16(pairs * N_out * elt) + (sorted_cap + sorted_cap / block + 2) * 4;
}

int moe_prepare(const void* X, int xdtype, void* q8x, int tokens, int K, const int32_t* topk_ids, int numel, int num_experts, int block,
                int32_t* sorted_ids, int sorted_capacity, int32_t* expert_ids, int expert_capacity, int32_t* num_post_padded,
                hipStream_t s);   // moe_aux.hip
int moe_weighted_sum_live(const void* Y, const float* topk_weights, const int32_t* topk_ids, int num_experts, void* out, int dtype,
                          int64_t tokens, int64_t top_k, int64_t N, hipStream_t s, const int32_t* slot_of_pair = nullptr);   // moe_aux.hip
int moe_prepare_sorted(const void* X, int xdtype, void* q8x_sorted, int K, const int32_t* topk_ids, int numel, int top_k, int num_experts,
                       int block, int32_t* sorted_ids, int sorted_capacity, int32_t* expert_ids, int expert_capacity,
                       int32_t* num_post_padded, int32_t* slot_of_pair, hipStream_t s);   // moe_aux.hip
int mmq_int_moe(const void* W, const void* ws, void* Y, int dtype, int type, int slots, int N, int K, const int32_t* expert_ids,
                const int32_t* num_tokens_post_padded, int64_t expert_stride, int block, hipStream_t s);   // mmq_i.hip

int moe_tiles_layer(const void* X, int xdtype, void* workspace, const void* W13, int type13, const void* W2, int type2, const int32_t* topk_ids,
                    const float* topk_w, void* out, int H, int I, int N_out, int top_k, int tokens, int act, int num_experts, bool vec_sums,
                    int block, hipStream_t s) {
  const int pairs = tokens * top_k, elt = xdtype == GGUF_DTYPE_F32 ? 4 : 2;
  char* q8x = (char*)workspace;
  char* q8h = q8x + up16((int64_t)tokens * q8_row_bytes(H));
  char* y2 = q8h + up16((int64_t)pairs * q8_row_bytes(I));
  const int64_t sorted_cap = (int64_t)pairs + (int64_t)num_experts * (block - 1), block_cap = sorted_cap / block + 1;
  int32_t* sorted = (int32_t*)(y2 + up16((int64_t)pairs * N_out * elt));
  int32_t* experts = sorted + sorted_cap;
  int32_t* post = experts + block_cap;
  // the rows of X quantized and the routing sorted in one launch (two where the sort's histogram rows outgrow 64 KB of LDS)
  int rc = moe_prepare(X, xdtype, q8x, tokens, H, topk_ids, pairs, num_experts, block, sorted, (int)sorted_cap, experts, (int)block_cap, post, s);
  if (rc == GGUF_NOT_TAKEN) {
    rc = quantize_q8_1(X, xdtype, q8x, tokens, H, s);
    if (rc != GGUF_OK) return rc;
    rc = gguf_moe_align_block_size(topk_ids, pairs, num_experts, block, sorted, sorted_cap, experts, block_cap, post, (gguf_stream_t)s);
  }
  if (rc != GGUF_OK) return rc;
  const int ns = (int)(sorted_cap / block * block);
  // vec_sums: the offset term of Q4_K / Q5_K as the per-pair operator forms it; else as the grouped operator does
  const auto gemv_sums = [&](int type) { return vec_sums && (type == T_Q4_K || type == T_Q5_K) ? 1 : 0; };
  const MoeArgs m1 = {sorted, experts, post, (int64_t)2 * I * (H / block_elems(type13)) * block_bytes(type13), top_k, pairs, gemv_sums(type13)};
  rc = block == 16 ? moe_tiles16_gate(W13, q8x, q8h, xdtype, type13, I, H, ns, m1, act, s)
                   : moe_tiles32_gate(W13, q8x, q8h, xdtype, type13, I, H, ns, m1, act, s);
  if (rc != GGUF_OK) return rc == GGUF_NOT_TAKEN ? GGUF_ERR_TYPE : rc;
  // the second GEMM's rows are the pairs themselves: slot -> pair -> row pair of q8h
  const MoeArgs m2 = {sorted, experts, post, (int64_t)N_out * (I / block_elems(type2)) * block_bytes(type2), 1, pairs, gemv_sums(type2)};
  rc = block == 16 ? moe_tiles16(W2, q8h, y2, xdtype, type2, N_out, I, ns, m2, s) : moe_tiles32(W2, q8h, y2, xdtype, type2, N_out, I, ns, m2, s);
  if (rc != GGUF_OK) return rc == GGUF_NOT_TAKEN ? GGUF_ERR_TYPE : rc;
  // the grouped operator leaves the rows of pairs whose expert id names no expert at zero (the sort drops them): the
  // sum takes them as zero instead of reading rows of y2 that nobody wrote
  return moe_weighted_sum_live(y2, topk_w, vec_sums ? nullptr : topk_ids, num_experts, out, xdtype, tokens, top_k, N_out, s);
}

// ---- A MoE layer whose experts see many pairs each, on the pipelined integer engine: the routing is sorted into blocks of
// `block` slots (64), the rows of X are quantized into slot order, and both expert GEMMs run as the dense product does, a block
// of slots being a run of rows like any other (mmq_i_core.h, MmqiMoe); the intermediate and the result stay in slot
// order and the weighted sum gathers its rows through the inverse of the sort.  Six launches: sort, quantize, GEMM,
// quantize with the activation, GEMM, weighted sum.
// [q8_1 rows of X, slot order][first GEMM's result, slots x 2 I][q8_1 rows of h][second GEMM's result, slots x N_out]
// [sorted ids, expert ids, padded total, slot of every pair]
int64_t moe_sorted_layer_workspace(int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out, int64_t num_experts, int elt,
                                   int block) {
  const int64_t pairs = tokens * top_k, cap = pairs + num_experts * (block - 1), slots = cap / block * block;
  return up16(slots * q8_row_bytes(H)) + up16(slots * 2 * I * elt) + up16(slots * q8_row_bytes(I)) + up16(slots * N_out * elt) +
         (cap + cap / block + 2 + pairs) * 4;
}

int moe_sorted_layer(const void* X, int xdtype, void* workspace, const void* W13, int type13, const void* W2, int type2, const int32_t* topk_ids,
                     const float* topk_w, void* out, int H, int I, int N_out, int top_k, int tokens, int act, int num_experts, int block,
                     hipStream_t s) {
  const int pairs = tokens * top_k, elt = xdtype == GGUF_DTYPE_F32 ? 4 : 2;
  const int64_t cap = (int64_t)pairs + (int64_t)num_experts * (block - 1), slots = cap / block * block, block_cap = cap / block + 1;
  char* q8x = (char*)workspace;
  char* y1 = q8x + up16(slots * q8_row_bytes(H));
  char* q8h = y1 + up16(slots * 2 * I * elt);
  char* y2 = q8h + up16(slots * q8_row_bytes(I));
  int32_t* sorted = (int32_t*)(y2 + up16(slots * N_out * elt));
  int32_t* experts = sorted + cap;
  int32_t* post = experts + block_cap;
  int32_t* slot_of_pair = post + 1;
  int rc = moe_prepare_sorted(X, xdtype, q8x, H, topk_ids, pairs, top_k, num_experts, block, sorted, (int)cap, experts, (int)block_cap, post,
                              slot_of_pair, s);
  if (rc != GGUF_OK) return rc;
  rc = mmq_int_moe(W13, q8x, y1, xdtype, type13, (int)slots, 2 * I, H, experts, post, (int64_t)2 * I * (H / block_elems(type13)) * block_bytes(type13), block, s);
  if (rc != GGUF_OK) return rc == GGUF_NOT_TAKEN ? GGUF_ERR_TYPE : rc;
  rc = quantize_q8_1(y1, xdtype, q8h, slots, I, s, act);     // rows of y1 are [gate | up]: h = T(T(act(gate)) up), quantized
  if (rc != GGUF_OK) return rc;
  rc = mmq_int_moe(W2, q8h, y2, xdtype, type2, (int)slots, N_out, I, experts, post, (int64_t)N_out * (I / block_elems(type2)) * block_bytes(type2), block, s);
  if (rc != GGUF_OK) return rc == GGUF_NOT_TAKEN ? GGUF_ERR_TYPE : rc;
  return moe_weighted_sum_live(y2, topk_w, nullptr, 0, out, xdtype, tokens, top_k, N_out, s, slot_of_pair);
}

// mmvq.hip
int mmvq_any(int type, const void* W, const void* x, void* q8_workspace, void* Y, int xdtype, int64_t N, int64_t K, int64_t M,
             hipStream_t s, const LinearArgs& la);

constexpr int MMQ_ROWS16_MAX = 32;   // up to this many rows of X the integer path runs the 16-row tile kernel

// mmq_h.hip
int mmq_half(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial,
             int64_t partial_bytes, hipStream_t s, const LinearArgs& la);
bool mmq_half_supported(int type);
int64_t mmq_half_partial_bytes(int M, int N, int K);

// moe_tiles16.hip: the 16-row tile kernel for 9 .. 32 rows of X (GGUF_NOT_TAKEN for formats it does not cover)
int mmq_rows16(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial, int64_t partial_bytes,
               hipStream_t s, const LinearArgs& la);
int64_t mmq_rows16_partial_bytes(int M, int N, int K);
// rows16_direct.hip: whether a call with at most 16 rows runs the kernel that reads Q4_K from the packed blocks
bool rows16_direct_takes(const void* W, int64_t w_pitch, int type, int M, int N, int K, int64_t partial_bytes);
bool rows16_direct_pays(int type, int M, int64_t N, int64_t K, bool against_gemv);

// mmq_i.hip
int mmq_int(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial,
            int64_t partial_bytes, hipStream_t s, const LinearArgs& la);
int64_t mmq_int_partial_bytes(int M, int N, int K);

}  // namespace gguf

// Bytes of the row region of a workspace, rounded up so that what follows is aligned: the quantized rows, and for
// the half engine their half-precision copy behind them.
static int64_t mmq_rows_bytes(int64_t M, int64_t K, bool half_plane) {
  return (M * (gguf::q8_row_bytes(K) + (half_plane ? 2 * gguf::q8_half_pitch(K) : 0)) + 255) / 256 * 256;
}

extern "C" int64_t gguf_mmq_workspace_bytes_engine(int64_t M, int64_t N, int64_t K, int engine) {
  if (M <= 0 || N <= 0 || K <= 0 || M > 0x7FFFFFF0LL || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL) return 0;
  if (engine < GGUF_MMQ_AUTO || engine > GGUF_MMQ_HALF) return 0;
  if (engine == GGUF_MMQ_HALF) return mmq_rows_bytes(M, K, true) + gguf::mmq_half_partial_bytes((int)M, (int)N, (int)K);
  const int64_t pi = gguf::mmq_int_partial_bytes((int)M, (int)N, (int)K);
  const int64_t p16 = M <= gguf::MMQ_ROWS16_MAX ? gguf::mmq_rows16_partial_bytes((int)M, (int)N, (int)K) : 0;
  return mmq_rows_bytes(M, K, false) + (pi > p16 ? pi : p16);
}

// room for either engine
extern "C" int64_t gguf_mmq_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  const int64_t a = gguf_mmq_workspace_bytes_engine(M, N, K, GGUF_MMQ_INT8), b = gguf_mmq_workspace_bytes_engine(M, N, K, GGUF_MMQ_HALF);
  return a > b ? a : b;
}

// gguf_mmq_linear with the size of the workspace's row region given by the caller: rows_bytes < 0 stands for the public
// layout (quantized rows, then room for their half-precision copy); the entry point that brings its own workspace
// keeps the quantized rows only and never runs the half engine.
namespace gguf {
int mmq_linear_impl(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                    int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M, int engine,
                    int64_t workspace_bytes, int64_t rows_bytes, gguf_stream_t stream);
}

extern "C" int gguf_mmq_linear(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                               int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M, int engine,
                               int64_t workspace_bytes, gguf_stream_t stream) {
  return gguf::mmq_linear_impl(W, w_row_pitch_bytes, x, xdtype, q8_workspace, Y, y_row_pitch, bias, type, N, K, M, engine,
                               workspace_bytes, -1, stream);
}

int gguf::mmq_linear_impl(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                          int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M, int engine,
                          int64_t workspace_bytes, int64_t rows_bytes, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0 || !mmq_type_ok(type)) return GGUF_ERR_TYPE;
  if (K > 0 && K % qk == 0 && (w_row_pitch_bytes < K / qk * block_bytes(type) || y_row_pitch < N)) return GGUF_ERR_SHAPE;
  LinearArgs la;
  la.w_pitch = w_row_pitch_bytes;
  la.ldy = y_row_pitch;
  la.bias = bias;
  if (N < 0 || M < 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL || M > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (engine < GGUF_MMQ_AUTO || engine > GGUF_MMQ_HALF || workspace_bytes < 0) return GGUF_ERR_SHAPE;
  if (engine == GGUF_MMQ_HALF && !mmq_half_supported(type)) return GGUF_ERR_TYPE;
  if (engine == GGUF_MMQ_HALF && xdtype == GGUF_DTYPE_F32) return GGUF_ERR_DTYPE;
  if (N == 0 || M == 0) return GGUF_OK;
  if (!W || !x || !q8_workspace || !Y) return GGUF_ERR_NULL;
  if (((uintptr_t)W & 1) || (w_row_pitch_bytes & 1)) return GGUF_ERR_SHAPE;  // packed blocks sit at even addresses
  hipStream_t s = (hipStream_t)stream;
  // (the 16-row tile kernel that reads the K-quants straight from the packed blocks takes the same time for 1 .. 16 rows
  // and passes the GEMV, which has one kernel for 5 .. 8 rows, there: Q4_K [14336,4096] 17 against 21 us at 6 rows,
  // against 14 us at 4; see rows16_direct_pays)
  // The row region: the quantized rows, for the half engine also their half-precision copy.  (A caller-given size is
  // that of quantized rows only.)
  if (rows_bytes >= 0 && engine == GGUF_MMQ_HALF) return GGUF_ERR_SHAPE;   // no room for the half-precision rows in that layout
  if (rows_bytes < 0) rows_bytes = mmq_rows_bytes(M, K, engine == GGUF_MMQ_HALF);
  if (workspace_bytes == 0 && engine != GGUF_MMQ_HALF) workspace_bytes = M * q8_row_bytes(K);   // the stated minimum
  if (workspace_bytes < M * (q8_row_bytes(K) + (engine == GGUF_MMQ_HALF ? 2 * q8_half_pitch(K) : 0))) return GGUF_ERR_WORKSPACE;
  const int64_t partial_room = workspace_bytes - rows_bytes;
  const bool tiles_at_5 = M <= 16 && rows16_direct_pays(type, (int)M, N, K, true) && rows16_direct_takes(W, w_row_pitch_bytes, type, (int)M, (int)N, (int)K, partial_room > 0 ? partial_room : 0);
  if (engine == GGUF_MMQ_AUTO && M <= 8 && !tiles_at_5) {
    // a handful of rows: the streaming GEMV kernel with the tile kernels' offset sums reads W once at close to the
    // GEMV's rate and is exact in int8; it declines shapes it does not cover
    LinearArgs lt = la;
    lt.tile_sums = true;
    const int rc = mmvq_any(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, lt);
    if (rc != GGUF_NOT_TAKEN) return rc;
  }
  if (engine == GGUF_MMQ_AUTO) engine = GGUF_MMQ_INT8;   // the reference's arithmetic; the half engine is for callers that ask
  float* partial = (float*)((char*)q8_workspace + rows_bytes);
  const int64_t partial_bytes = workspace_bytes > rows_bytes ? workspace_bytes - rows_bytes : 0;
  if (engine == GGUF_MMQ_HALF) {
    void* half_plane = (char*)q8_workspace + M * q8_row_bytes(K);
    const int rc = quantize_q8_1(x, xdtype, q8_workspace, M, K, s, 0, half_plane);
    if (rc != GGUF_OK) return rc;
    return mmq_half(W, q8_workspace, Y, xdtype, type, (int)M, (int)N, (int)K, partial, partial_bytes, s, la);
  }
  int rc = quantize_q8_1(x, xdtype, q8_workspace, M, K, s);
  if (rc != GGUF_OK) return rc;
  if (M <= MMQ_ROWS16_MAX) {   // a few rows: 16-row tiles, K split over the chip
    rc = mmq_rows16(W, q8_workspace, Y, xdtype, type, (int)M, (int)N, (int)K, partial, partial_bytes, s, la);
    if (rc != GGUF_NOT_TAKEN) return rc;
  }
  rc = mmq_int(W, q8_workspace, Y, xdtype, type, (int)M, (int)N, (int)K, partial, partial_bytes, s, la);   // every tile format
  return rc == GGUF_NOT_TAKEN ? GGUF_ERR_TYPE : rc;
}

extern "C" int gguf_mmq_engine(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N,
                               int64_t K, int64_t M, int engine, int64_t workspace_bytes, gguf_stream_t stream) {
  const int qk = gguf::block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (K <= 0 || K % qk != 0) return GGUF_ERR_SHAPE;
  return gguf_mmq_linear(W, K / qk * gguf::block_bytes(type), x, xdtype, q8_workspace, Y, N, nullptr, type, N, K, M, engine,
                         workspace_bytes, stream);
}

extern "C" int gguf_mmq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N,
                        int64_t K, int64_t M, gguf_stream_t stream) {
  return gguf_mmq_engine(W, x, xdtype, q8_workspace, Y, type, N, K, M, GGUF_MMQ_AUTO, 0, stream);
}

extern "C" int gguf_moe_block_size(int type) { return gguf::block_elems(type) ? 32 : 0; }

extern "C" int gguf_moe_mmq(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                            const int32_t* sorted_token_ids, const int32_t* expert_ids,
                            const int32_t* num_tokens_post_padded, int64_t num_sorted, void* Y, int type, int64_t N,
                            int64_t K, int64_t top_k, int64_t tokens, gguf_stream_t stream) {
  return gguf_moe_mmq_block(X, xdtype, q8_workspace, W, expert_stride_bytes, sorted_token_ids, expert_ids, num_tokens_post_padded,
                            num_sorted, Y, type, N, K, top_k, tokens, 0, 32, 0, stream);
}

extern "C" int gguf_moe_mmq_act(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                                const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                const int32_t* num_tokens_post_padded, int64_t num_sorted, void* Y, int type, int64_t N,
                                int64_t K, int64_t top_k, int64_t tokens, int act, gguf_stream_t stream) {
  return gguf_moe_mmq_block(X, xdtype, q8_workspace, W, expert_stride_bytes, sorted_token_ids, expert_ids, num_tokens_post_padded,
                            num_sorted, Y, type, N, K, top_k, tokens, act, 32, 0, stream);
}

extern "C" int gguf_moe_block_size_for(int type, int64_t pairs, int64_t num_experts) {
  if (!gguf::block_elems(type)) return 0;
  // (the Q4_0 layer of 64 experts [2048,2048] / [2048,1024], top-8: blocks of 16 against 32 at 65 / 96 / 128 / 256 tokens
  //  98 / 111 / 119 / 191 us against 112 / 113 / 113 / 148 us)
  return num_experts > 0 && pairs <= 12 * num_experts && gguf::moe_tiles16_ok(type) ? 16 : 32;
}

extern "C" int gguf_moe_mmq_block(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                                  const int32_t* sorted_token_ids, const int32_t* expert_ids,
                                  const int32_t* num_tokens_post_padded, int64_t num_sorted, void* Y, int type, int64_t N,
                                  int64_t K, int64_t top_k, int64_t tokens, int act, int64_t block, int64_t num_experts,
                                  gguf_stream_t stream) {
  using namespace gguf;
  if (act < 0 || act > 2) return GGUF_ERR_SHAPE;
  const int qk = block_elems(type);
  if (qk == 0 || !mmq_type_ok(type)) return GGUF_ERR_TYPE;
  if (block != 32 && block != 16) return GGUF_ERR_SHAPE;
  if (block == 16 && !moe_tiles16_ok(type)) return GGUF_ERR_TYPE;
  // the kernels keep the reference's guard on expert ids (moe.cuh:33: blocks of experts above 255 are skipped); a
  // caller that says how many experts there are is told so instead of receiving rows of zeros
  if (num_experts < 0 || num_experts > 256) return GGUF_ERR_SHAPE;
  if (N < 0 || tokens < 0 || top_k <= 0 || num_sorted < 0 || K <= 0 || K % qk != 0 || expert_stride_bytes < 0 ||
      tokens * top_k > 0x7FFFFFF0LL || N > 0x7FFFFFF0LL)
    return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || tokens == 0) return GGUF_OK;
  if (!X || !q8_workspace || !W || !sorted_token_ids || !expert_ids || !num_tokens_post_padded || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  // rows that no slot names stay zero, as with the reference's zero-filled output (gguf_kernel.cu:301-302)
  const int64_t ybytes = tokens * top_k * N * (xdtype == GGUF_DTYPE_F32 ? 4 : 2);
  if ((uintptr_t)Y & 15) return GGUF_ERR_SHAPE;
  hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)((ybytes / 16 + 256) / 256)), dim3(256), 0, s, (uint4*)Y, ybytes);
  const int rc = quantize_q8_1(X, xdtype, q8_workspace, tokens, K, s, act);
  if (rc != GGUF_OK) return rc;
  MoeArgs moe = {sorted_token_ids, expert_ids, num_tokens_post_padded, expert_stride_bytes, (int)top_k, (int)(tokens * top_k), 0};
  const int ns = (int)(num_sorted / block * block);  // a trailing partial block is ignored, like the reference's integer division
  if (ns == 0) return launch_status();
  if (block == 16) return moe_tiles16(W, q8_workspace, Y, xdtype, type, (int)N, (int)K, ns, moe, s);
  return moe_tiles32(W, q8_workspace, Y, xdtype, type, (int)N, (int)K, ns, moe, s);
}
