// Prefill-path GEMM on packed GGUF weights, on gfx950 half-precision MFMA: the kernel, shared by the a8 operator
// (mmq_h.hip: q8_1 activations) and the dense-weight operator (dq_gemm.hip: activations as they are).
//
//   Y[m, n] = sum_k  xh[m, k] * wh[n, k]        xh = RN16(d8 * xq)   the q8_1 activations, dequantized
//                                               wh = RN16(RN16(dw) * wq)   the GGUF weights, dequantized
//
// The int8 engine (mmq.hip) keeps the block scales out of the matrix product and pays two to four vector-ALU
// instructions per result and 32-element block for it, which on this chip cannot overlap the MFMAs of the same
// SIMD.  Here both operands carry their scales into the product, so the K loop is MFMA and LDS reads only; the
// vector ALU decodes every weight block once per workgroup and step (about 2.5 instructions per weight), amortised
// over the M_T token rows of the tile.  v_mfma_f32_32x32x16_f16 runs at half the int8 rate, yet the loop is more
// than twice as fast because nothing else is left in it.
//
// Arithmetic: the products of half operands are exact in the MFMA's fp32 accumulation, so the only differences from
// the int8 engine are the roundings of the two operands to half precision (relative 2^-12 each, 2^-11 for the
// weights' two roundings).  That is below the rounding of a half or bfloat16 result; fp32 results stay on the int8 engine.
// Weights are staged times 2^4 and the result scaled back, which keeps small weight scales out of the half
// subnormals; weights of magnitude 4094 and more overflow.
//
// Offset terms: formats whose offset multiplies the sum of the activation quants (Q2_K) fold it into wh.  Formats
// whose offset multiplies the stored block sum of the unquantized activations (Q4_0, Q4_K, Q5_K in the reference's
// MMQ semantics, vecdotq.cuh:61-64,369-372) centre their codes and add the rest in a second, 16 times shorter loop
// over the blocks (see there).
#pragma once
#include <type_traits>

#include "mmq_formats.h"

namespace gguf {

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));   // a plain vector: stays in registers where HIP's uint4 struct may not
typedef u32x4 __attribute__((address_space(1))) global_u32x4;  // a load through an integer address must name its address space

constexpr float HP_SCALE = 16.0f, HP_UNSCALE = 0.0625f;

// How a format's codes reach half precision.  A byte b becomes the half 1024 + b by placing it under the exponent
// byte 0x64, and subtracting 1024 + BIAS leaves the code exactly: formats with unsigned codes (BIAS = the code's
// zero point) skip their own recentring, signed int8 codes are flipped to b = code + 128 first.
template <class F> struct HalfCodes {
  static constexpr bool FLIP = true;
  static constexpr int BIAS = 128;
  static __device__ __forceinline__ void unpack(const typename F::Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    F::unpack(r, kb, q, s0, s1, mn, mn1);
  }
};
template <class F, int B> struct UnsignedCodes {
  static constexpr bool FLIP = false;
  static constexpr int BIAS = B;
  static __device__ __forceinline__ void unpack(const typename F::Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    F::unpack(r, kb, q, s0, s1, mn, mn1);
  }
};
template <class F, int B> struct RecentredCodes {
  static constexpr bool FLIP = false;
  static constexpr int BIAS = B;
  static __device__ __forceinline__ void unpack(const typename F::Raw& r, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn, float& mn1) {
    F::template unpack<false>(r, kb, q, s0, s1, mn, mn1);
  }
};
template <> struct HalfCodes<MQ4_0> : UnsignedCodes<MQ4_0, MQ4_0::CENTRE> {};   // codes centred; the offset pass adds what that leaves
template <> struct HalfCodes<MQ4_K> : UnsignedCodes<MQ4_K, MQ4_K::CENTRE> {};
template <> struct HalfCodes<MQ5_K> : UnsignedCodes<MQ5_K, MQ5_K::CENTRE> {};
template <> struct HalfCodes<MQ2_K> : UnsignedCodes<MQ2_K, 0> {};
template <> struct HalfCodes<MQ6_K> : RecentredCodes<MQ6_K, 32> {};
template <> struct HalfCodes<MQ3_K> : RecentredCodes<MQ3_K, 4> {};
template <> struct HalfCodes<MQ5_0> : RecentredCodes<MQ5_0, 16> {};

// 32 codes (element order, four per dword) -> 32 halfs  (code - BIAS) * s - m, with s and m per 16 elements
template <bool FLIP, int BIAS, bool WITH_MIN>
__device__ __forceinline__ void codes_to_half(const uint32_t (&q)[8], float s0, float s1, float m0, float m1, uint4 (&out)[4]) {
  const _Float16 h0 = (_Float16)(s0 * HP_SCALE), h1 = (_Float16)(s1 * HP_SCALE);
  const _Float16 g0 = (_Float16)(m0 * HP_SCALE), g1 = (_Float16)(m1 * HP_SCALE);
  const v2h bias = {(_Float16)(1024.0f + BIAS), (_Float16)(1024.0f + BIAS)};
  uint32_t w[16];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t u = FLIP ? q[i] ^ 0x80808080u : q[i];
    const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, u, 0x04010400u);
    const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, u, 0x04030402u);
    const _Float16 s = i < 4 ? h0 : h1, m = i < 4 ? g0 : g1;
    const v2h sc = {s, s}, mn = {m, m};
    v2h a = __builtin_bit_cast(v2h, lo) - bias, b = __builtin_bit_cast(v2h, hi) - bias;
    if (WITH_MIN) { a = a * sc - mn; b = b * sc - mn; }
    else { a = a * sc; b = b * sc; }
    w[2 * i] = __builtin_bit_cast(uint32_t, a);
    w[2 * i + 1] = __builtin_bit_cast(uint32_t, b);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) out[i] = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
}

// What the kernel multiplies the activations with.
//   A8Codes<F>  the reference's a8 semantics (vecdotq.cuh): offsets that multiply the stored block sum of the
//               unquantized activations are kept out of the weights (centred codes, offset pass); xh holds the
//               dequantized q8_1 rows.
//   DqCodes<F>  the dense weights themselves, as ggml_dequantize yields them in half precision (dequantize.cuh):
//               offsets are part of the weight; xh holds the activations as they are.  For the standard and K
//               formats the roundings are the reference kernels' own: half(d * sc), half(dmin * m), one fused multiply-add.
template <class F> struct A8Codes : HalfCodes<F> {
  using Fmt = F;
  static constexpr bool WITH_MIN = F::MIN16, PLUS_MIN = false;
  static constexpr bool SUM_PASS = F::HAS_MIN && !F::MIN16;
};
template <class F> struct DqCodes : HalfCodes<F> {
  using Fmt = F;
  static constexpr bool WITH_MIN = F::HAS_MIN, PLUS_MIN = F::HALFPROD;  // Q4_1 / Q5_1 add their m, the K formats subtract dmin * m
  static constexpr bool SUM_PASS = false;
};
template <> struct DqCodes<MQ4_0> : HalfCodes<MQ4_0> {   // d * (q - 8) with the codes centred at 8: no offset left
  using Fmt = MQ4_0;
  static constexpr bool WITH_MIN = false, PLUS_MIN = false, SUM_PASS = false;
};
template <> struct DqCodes<MQ4_K> : UnsignedCodes<MQ4_K, 0> {
  using Fmt = MQ4_K;
  static constexpr bool WITH_MIN = true, PLUS_MIN = false, SUM_PASS = false;
};
template <> struct DqCodes<MQ5_K> : UnsignedCodes<MQ5_K, 0> {
  using Fmt = MQ5_K;
  static constexpr bool WITH_MIN = true, PLUS_MIN = false, SUM_PASS = false;
};
template <> struct DqCodes<MQ4_1> : UnsignedCodes<MQ4_1, 0> {
  using Fmt = MQ4_1;
  static constexpr bool WITH_MIN = true, PLUS_MIN = true, SUM_PASS = false;
};
template <> struct DqCodes<MQ5_1> : UnsignedCodes<MQ5_1, 0> {
  using Fmt = MQ5_1;
  static constexpr bool WITH_MIN = true, PLUS_MIN = true, SUM_PASS = false;
};

template <class C, int WM, int WN, int TM, int TN, int OCC, typename T>
__global__ __launch_bounds__(64 * WM * WN, OCC) void mmqh_kernel(const uint8_t* __restrict__ W, const _Float16* __restrict__ xh,
                                                                  const char* __restrict__ ws, int64_t ws_row_bytes,
                                                                  T* __restrict__ Y, float* __restrict__ partial, int M, int N,
                                                                  int K, int Kp, int tiles_x, int whole_tiles, int shared_tiles, int splits,
                                                                  int64_t w_pitch, int64_t ldy, const T* __restrict__ bias) {
  using F = typename C::Fmt;
  constexpr int NT = 64 * WM * WN;
  constexpr int KS = 64;                 // elements of K per step
  constexpr int KB = KS / 32;            // 32-blocks per step
  constexpr int GR = KS / 8;             // 16-byte granules (8 halfs) per activation row and step
  constexpr int LDH = KS + 8;            // LDS row pitch in halfs: a 16-byte skew spreads 8 consecutive rows over all banks
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  constexpr int PAIRS = N_T * KB;        // (weight row, 32-block) pairs to decode per step, one thread each
  static_assert(NT % PAIRS == 0 && (M_T * GR) % NT == 0, "tile and workgroup sizes must divide evenly");
  static_assert(NT / PAIRS == 2, "the unrolled pipeline below assumes two decode groups");
  constexpr int DG = NT / PAIRS;         // decode groups: group g decodes the steps t with t % DG == g
  constexpr int AQ = M_T * GR / NT;      // activation granules per thread and step
  constexpr int TILE = (M_T + N_T) * LDH;  // halfs per buffer
  extern __shared__ __align__(16) char smem[];
  _Float16* const tiles = (_Float16*)smem;   // two buffers of { activations [M_T][LDH], decoded weights [N_T][LDH] }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int lrow = lane & 31, lhalf = lane >> 5;
  // Workgroup -> work: the first `whole_tiles` workgroups take one output tile each over all of K; behind them every
  // further tile is shared by `splits` workgroups, each taking a stretch of K (see the loop below).
  const int wg = blockIdx.x;
  const int tile = wg < whole_tiles ? wg : whole_tiles + (wg - whole_tiles) % shared_tiles;   // neighbours in launch order walk
  const int split = wg < whole_tiles ? 0 : (wg - whole_tiles) / shared_tiles;                  // the same stretch of K
  const int nsplit = wg < whole_tiles ? 1 : splits;
  const int m_base = (tile / tiles_x) * M_T, n_base = (tile % tiles_x) * N_T;
  const int64_t rowbytes = w_pitch;   // bytes between rows of W: the dense row size unless the caller's tensor is padded
  const int nkb_total = K >> 5;
  const int nsteps = (K + KS - 1) / KS;

  const _Float16* aq_src[AQ];
#pragma unroll
  for (int i = 0; i < AQ; ++i) {
    const int p = tid + NT * i, m = p / GR, g = p % GR;
    aq_src[i] = xh + (int64_t)min(m_base + m, M - 1) * (Kp + 128) + 8 * g;   // rows past M repeat the last row; never stored
  }
  const int grp = tid / PAIRS, n_dec = (tid % PAIRS) / KB, kb_dec = tid % KB;
  const uint8_t* const w_row = W + (int64_t)min(n_base + n_dec, N - 1) * rowbytes;

  // Global loads run two turns ahead of their use: two register stages for the activations (a turn = one step) and two
  // for this thread's weight block (a turn = DG steps), indexed by compile-time constants so that they stay registers.
  u32x4 r_aq[2][AQ];
  typename F::Raw r_w[2];

  auto fetch_a = [&](auto stage, int t) {
    constexpr int S = decltype(stage)::value;
#pragma unroll
    for (int i = 0; i < AQ; ++i) r_aq[S][i] = *(const u32x4*)(aq_src[i] + t * KS);  // rows are padded with zeros to a multiple of 512
  };
  auto write_a = [&](auto stage, int buf) {
    constexpr int S = decltype(stage)::value;
    _Float16* xs = tiles + buf * TILE;
#pragma unroll
    for (int i = 0; i < AQ; ++i) {
      const int p = tid + NT * i;
      *(u32x4*)(xs + (p / GR) * LDH + 8 * (p % GR)) = r_aq[S][i];
    }
  };
  auto fetch_w = [&](auto stage, int t) {
    constexpr int S = decltype(stage)::value;
    r_w[S] = F::fetch(w_row, min(t * KB + kb_dec, nkb_total - 1));  // clamped: a block past K is re-read and decoded to zeros
  };
  auto decode = [&](auto stage, int t, int buf) {
    constexpr int S = decltype(stage)::value;
    _Float16* wt = tiles + buf * TILE + M_T * LDH;
    const int kb = t * KB + kb_dec;
    uint32_t q[8];
    float s0, s1, mn = 0.0f, mn1 = 0.0f;
    C::unpack(r_w[S], kb, q, s0, s1, mn, mn1);
    if (!F::MIN16) mn1 = mn;   // one offset factor per 32-block unless the format has one per 16
    if (kb >= nkb_total) s0 = s1 = mn = mn1 = 0.0f;
    uint4 h[4];
    codes_to_half<C::FLIP, C::BIAS, C::WITH_MIN>(q, s0, s1, C::PLUS_MIN ? -mn : mn, C::PLUS_MIN ? -mn1 : mn1, h);
#pragma unroll
    for (int j = 0; j < 4; ++j) *(uint4*)(wt + n_dec * LDH + 32 * kb_dec + 8 * j) = h[j];
  };

  v16f acc[TM][TN];
#pragma unroll
  for (int j = 0; j < TM; ++j)
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][i][r] = 0.0f;

  // One step of K from buffer `buf`.  All operand reads of the step are issued before its first MFMA: every wave then
  // keeps the LDS pipe busy for the whole step, and the matrix work of one wave runs under the reads of the other
  // wave on its SIMD.
  auto contract = [&](int buf, int slices) {
    const _Float16* xs = tiles + buf * TILE;
    const _Float16* wt = xs + M_T * LDH;
    v8h af[KS / 16][TM], bf[KS / 16][TN];
#pragma unroll
    for (int kk = 0; kk < KS / 16; ++kk) {
#pragma unroll
      for (int j = 0; j < TM; ++j) af[kk][j] = *(const v8h*)(xs + (32 * (wm * TM + j) + lrow) * LDH + 16 * kk + 8 * lhalf);
#pragma unroll
      for (int i = 0; i < TN; ++i) bf[kk][i] = *(const v8h*)(wt + (32 * (wn * TN + i) + lrow) * LDH + 16 * kk + 8 * lhalf);
    }
#pragma unroll
    for (int kk = 0; kk < KS / 16; ++kk) {
      if (kk >= slices) break;
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int i = 0; i < TN; ++i) {
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[kk][j], bf[kk][i], acc[j][i], 0, 0, 0);
        }
    }
    // Instruction order for the scheduler: the first slice's operand reads, then one operand read behind every MFMA
    // until the reads run out.  An MFMA occupies the matrix unit for 32 cycles but issues in 4, so the reads of the
    // coming slices issue and complete under the matrix work instead of in front of it.
    if (slices == KS / 16) {
      constexpr int READS = (KS / 16) * (TM + TN), MFMAS = (KS / 16) * TM * TN, LEAD = TM + TN;
      __builtin_amdgcn_sched_group_barrier(0x100, LEAD, 0);          // DS reads
#pragma unroll
      for (int i = 0; i < MFMAS; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);           // one MFMA
        if (i < READS - LEAD) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
    }
  };

  // Software pipeline over the steps, two LDS buffers, one barrier per step.  In iteration s every wave first moves
  // step s+1 into the other buffer -- the activations from the registers loaded one iteration ago, and, if it is this
  // wave's turn, the weight block decoded from the registers loaded DG iterations ago -- issues the global loads that
  // refill those registers, and then contracts step s.  Waves whose turn it is not go straight to the matrix work, so
  // a SIMD always has one wave decoding and one multiplying.
  // A tile whose K is split leaves one fp32 partial tile per split in `partial`; a second kernel adds them.  Splitting
  // serves shapes whose output has too few tiles to occupy the chip, and the last, partly filled round of workgroups
  // of any shape: instead of a few CUs working through whole tiles while the rest idle, all CUs share those tiles.
  const int per_split = (nsteps + nsplit - 1) / nsplit;
  const int t0 = split * per_split, t1 = min(nsteps, t0 + per_split);
  const int n = t1 - t0;                               // steps of this workgroup; step j of them is step t0 + j of K
  const int gpar = ((grp - t0) % DG + DG) % DG;         // this group decodes the steps j with j % DG == gpar
  constexpr std::integral_constant<int, 0> S0{};
  constexpr std::integral_constant<int, 1> S1{};
  if (n > 0) fetch_a(S0, t0);
  if (n > 1) fetch_a(S1, t0 + 1);
  if (gpar < n) fetch_w(S0, t0 + gpar);
  if (gpar + DG < n) fetch_w(S1, t0 + gpar + DG);
  // turn j: stage step j (activation stage j % 2; weight stage (j / DG) % 2 if it is this group's turn), refill the
  // stages just emptied with the loads of two turns ahead, contract step j - 1, barrier
  auto turn = [&](auto jmod, int j) {
    constexpr int J = decltype(jmod)::value;           // j % (2 * DG), so that every stage index is a constant
    constexpr std::integral_constant<int, J & 1> sa{};
    constexpr std::integral_constant<int, (J / DG) & 1> sw{};
    if (j > n) return;
    if (j < n) {
      write_a(sa, j & 1);
      if (j + 2 < n) fetch_a(sa, t0 + j + 2);
      if (J % DG == gpar) {
        decode(sw, t0 + j, j & 1);
        if (j + 2 * DG < n) fetch_w(sw, t0 + j + 2 * DG);
      }
    }
    if (j >= 1) contract((j - 1) & 1, KS / 16);
    __syncthreads();
  };
  for (int j = 0; j <= n; j += 2 * DG) {
    turn(std::integral_constant<int, 0>{}, j);
    turn(std::integral_constant<int, 1>{}, j + 1);
    turn(std::integral_constant<int, 2>{}, j + 2);
    turn(std::integral_constant<int, 3>{}, j + 3);
  }
  _Float16* const xs = tiles;                // the offset pass below reuses the first buffer
  _Float16* const wt = tiles + M_T * LDH;

  if constexpr (C::SUM_PASS) if (split == 0) {
    // Offset term (the first split adds it).  The reference's MMQ semantics multiply the offset factor mn by the stored sum s8 of the block's
    // unquantized activations (vecdotq.cuh:61-64, 369-372) while the codes meet the quantized ones, whose sum times
    // d8 is du.  With the codes centred at C in the main loop,
    //   s * sum q x^ - mn * s8  =  s * sum (q - C) x^  +  C s (du - s8)  +  (C s - mn) s8,
    // what remains is a short second product with two columns per 32-block: A = (du - s8, s8), B = (C s, C s - mn).
    // du - s8 is the small rounding residue of the block and C s - mn is small for blocks spread about their centre,
    // so the half-precision operands of this product cost far less accuracy than an uncentred main loop would.
    constexpr int SB = KS / 2;                      // blocks per step of this loop
    const float* as_src[AQ];
#pragma unroll
    for (int i = 0; i < AQ; ++i) {
      const int p = tid + NT * i, m = p / GR, g = p % GR;
      as_src[i] = (const float*)(ws + (int64_t)min(m_base + m, M - 1) * ws_row_bytes + Kp) + Kp / 32 + 4 * g;  // s8 plane; du follows
    }
    constexpr int UNITS = N_T * (SB / 8);           // (weight row, group of 8 blocks) pairs per step
    constexpr int WB = (UNITS + NT - 1) / NT;
    for (int b0 = 0; b0 < nkb_total; b0 += SB) {
      __syncthreads();
#pragma unroll
      for (int i = 0; i < AQ; ++i) {
        const int p = tid + NT * i, m = p / GR, g = p % GR;
        v8h o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const bool in = b0 + 4 * g + e < nkb_total;
          const float s8 = in ? as_src[i][b0 + e] : 0.0f, du = in ? as_src[i][b0 + e + Kp / 32] : 0.0f;
          o[2 * e] = (_Float16)(du - s8);
          o[2 * e + 1] = (_Float16)s8;
        }
        *(v8h*)(xs + m * LDH + 8 * g) = o;
      }
#pragma unroll
      for (int i = 0; i < WB; ++i) {
        const int p = tid + NT * i, n = p / (SB / 8), q = p % (SB / 8);
        if (p >= UNITS) continue;
        float cs[8], cm[8];
        F::offs8(W + (int64_t)min(n_base + n, N - 1) * rowbytes, b0 / 8 + q, nkb_total, cs, cm);
        v8h o0, o1;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o0[2 * e] = (_Float16)(cs[e] * HP_SCALE);     o0[2 * e + 1] = (_Float16)(cm[e] * HP_SCALE);
          o1[2 * e] = (_Float16)(cs[4 + e] * HP_SCALE); o1[2 * e + 1] = (_Float16)(cm[4 + e] * HP_SCALE);
        }
        *(v8h*)(wt + n * LDH + 16 * q) = o0;
        *(v8h*)(wt + n * LDH + 16 * q + 8) = o1;
      }
      __syncthreads();
      contract(0, (2 * min(nkb_total - b0, SB) + 15) / 16);
    }
  }

  float* const my_partial = nsplit > 1 ? partial + ((int64_t)(tile - whole_tiles) * splits + split) * (M_T * N_T) : nullptr;
#pragma unroll
  for (int j = 0; j < TM; ++j) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int ml = 32 * (wm * TM + j) + 8 * (r >> 2) + 4 * lhalf + (r & 3), mt = m_base + ml;
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int nl = 32 * (wn * TN + i) + lrow, n = n_base + nl;
        if (my_partial) my_partial[ml * N_T + nl] = acc[j][i][r];   // the whole tile, edges included: the adder masks them
        else if (mt < M && n < N) Y[(int64_t)mt * ldy + n] = finish<T>(acc[j][i][r] * HP_UNSCALE, bias, n);
      }
    }
  }
}

// Y tile = T(sum of its `splits` fp32 partial tiles / 16), gridDim.y workgroups per split tile, fixed order of addition
template <int M_T, int N_T, typename T>
__global__ __launch_bounds__(256) void mmqh_reduce_kernel(const float* __restrict__ partial, T* __restrict__ Y, int M, int N,
                                                          int tiles_x, int whole_tiles, int splits, int64_t ldy,
                                                          const T* __restrict__ bias) {
  const int tile = whole_tiles + blockIdx.x;
  const int m_base = (tile / tiles_x) * M_T, n_base = (tile % tiles_x) * N_T;
  const float* p = partial + (int64_t)blockIdx.x * splits * (M_T * N_T);
  for (int i = (blockIdx.y * 256 + threadIdx.x) * 4; i < M_T * N_T; i += gridDim.y * 256 * 4) {
    float4 acc = *(const float4*)(p + i);
    for (int z = 1; z < splits; ++z) {
      const float4 v = *(const float4*)(p + (int64_t)z * (M_T * N_T) + i);
      acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    const int m = m_base + i / N_T, n = n_base + i % N_T;
    if (m >= M) continue;
    const float out[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (n + e < N) Y[(int64_t)m * ldy + n + e] = finish<T>(out[e] * HP_UNSCALE, bias, n + e);
  }
}

// How the tiles of one launch are handed out: `whole` tiles get a workgroup each, the remaining `shared` tiles are
// split `splits` ways along K.  partial_bytes() is the fp32 scratch the shared tiles need.
struct MmqhPlan {
  int cfg;            // 0: 256x128, 1: 128x128, 2: 128x64, 3: 64x64
  int whole, shared, splits;
  int64_t partial_bytes() const {
    static const int tile_elems[4] = {256 * 128, 128 * 128, 128 * 64, 64 * 64};
    return (int64_t)shared * splits * tile_elems[cfg] * 4;
  }
};
MmqhPlan mmq_half_plan(int M, int N, int K, int64_t partial_bytes_available);  // mmq_h.hip

template <class C, int WM, int WN, int TM, int TN, int OCC, typename T>
static void launch_mmqh(const void* W, const void* ws, void* Y, int M, int N, int K, hipStream_t stream, int whole = -1, int shared = 0,
                        int splits = 1, float* partial = nullptr, const LinearArgs& la = LinearArgs()) {
  using F = typename C::Fmt;
  const int64_t w_pitch = la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS, ldy = la.ldy ? la.ldy : (int64_t)N;
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  constexpr size_t lds = (size_t)(M_T + N_T) * (64 + 8) * 2 * 2;
  auto kern = mmqh_kernel<C, WM, WN, TM, TN, OCC, T>;
  if constexpr (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, lds, done);
  }
  const int tiles_x = (N + N_T - 1) / N_T, tiles = tiles_x * ((M + M_T - 1) / M_T);
  if (whole < 0) { whole = tiles; shared = 0; splits = 1; }
  const _Float16* xh = (const _Float16*)((const char*)ws + (int64_t)M * q8_row_bytes(K));
  hipLaunchKernelGGL(kern, dim3(whole + shared * splits), dim3(64 * WM * WN), lds, stream, (const uint8_t*)W, xh, (const char*)ws,
                     q8_row_bytes(K), (T*)Y, partial, M, N, K, (int)q8_kp(K), tiles_x, whole, shared > 0 ? shared : 1, splits, w_pitch, ldy,
                     (const T*)la.bias);
  if (shared > 0)
    hipLaunchKernelGGL((mmqh_reduce_kernel<M_T, N_T, T>), dim3(shared, M_T * N_T / 1024), dim3(256), 0, stream, partial, (T*)Y, M, N, tiles_x,
                       whole, splits, ldy, (const T*)la.bias);
}


template <class C, typename T>
static int mmqh_typed(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, int64_t partial_bytes,
                      hipStream_t stream, const LinearArgs& la = LinearArgs()) {
  const MmqhPlan p = mmq_half_plan(M, N, K, partial_bytes);
  switch (p.cfg) {
    case 0: launch_mmqh<C, 4, 2, 2, 2, 1, T>(W, ws, Y, M, N, K, stream, p.whole, p.shared, p.splits, partial, la); break;  // 256 x 128, 8 waves
    case 1: launch_mmqh<C, 4, 2, 1, 2, 2, T>(W, ws, Y, M, N, K, stream, p.whole, p.shared, p.splits, partial, la); break;  // 128 x 128, 8 waves
    case 2: launch_mmqh<C, 2, 2, 2, 1, 2, T>(W, ws, Y, M, N, K, stream, p.whole, p.shared, p.splits, partial, la); break;  // 128 x 64, 4 waves
    default: launch_mmqh<C, 2, 2, 1, 1, 4, T>(W, ws, Y, M, N, K, stream, p.whole, p.shared, p.splits, partial, la); break; // 64 x 64, 4 waves
  }
  return launch_status();
}

}  // namespace gguf
