// Prefill-path GEMM on packed GGUF weights with q8_1 activations: the integer engine.
//
//   Y[m, n] = sum_kb  d8[m, kb] * dw[n, kb] * S[m, n, kb]  ( - offset terms )
//   S[m, n, kb] = sum over the 32 (or 16) elements of block kb of  xq[m, k] * wq[n, k]      (int32, exact)
//
// The reference computes S with dp4a on the vector ALU from re-packed LDS tiles (csrc/gguf/mmq.cuh:2-104,
// vecdotq.cuh load_tiles_* / vec_dot_*_mul_mat) and applies the block scales in fp32.  Here S is one
// v_mfma_i32_32x32x32_i8 per 32x32 output tile and 32-element block (two v_mfma_i32_32x32x16_i8 for the formats whose
// weight scale changes every 16 elements) and the block scales are applied in fp32 exactly as there; only the order
// of the fp32 additions differs.
//
// What sets the pace is the vector ALU, not the matrix unit: a q8_1 block is 32 values deep, so every MFMA result
// must be rescaled by d8[m, kb] * dw[n, kb] before the next block can be added.  Measured on this chip (4 waves per
// SIMD, independent instruction streams): v_fma_f32 / v_fmac_f32 / v_mul_f32 issue in about 1.0-1.1 ns per wave,
// v_fmac_f32 with a DPP operand, v_cvt_f32_i32 and the integer multiply-adds in about 1.75 ns, one 32x32x32 int8 MFMA
// occupies the SIMD for 14.2 ns (a 32x32x16 for 13.5 ns) of which only about a third hides under vector work of the
// same SIMD.  The loop is therefore built from plain fp32 multiply-adds only:
//   * int32 -> fp32 costs nothing: the MFMA accumulates onto the bit pattern of 1.5 * 2^23, so the integer sum S
//     leaves the matrix unit as the float 1.5 * 2^23 + S, and fma(1.5 * 2^23 + S, dw, -1.5 * 2^23 * dw) is exactly
//     RN(S * dw) (the constant is exact: every weight scale is an fp16 value times an integer of at most 8 bits);
//   * the activation scales of the 16 token rows a lane holds sit in 16 registers, read from LDS as four 16-byte
//     loads per block, and meet the product in a plain v_fmac_f32.
// That is two instructions per result and block (three with an offset term, four for the 16-deep formats).
//
// Work split: a workgroup of four waves owns an (M_T x N_T) output tile -- 128 x 64, or 64 x 128 for few tokens --
// and walks K in steps of 128 values.  Global loads run one step ahead in registers; the packed blocks are decoded
// once per workgroup and step into the LDS buffer the previous step has released (two buffers, one barrier per
// step).  Two workgroups share a CU, so a SIMD always holds a wave of each: one can rescale while the other waits at
// its barrier.  Output tiles are handed out linearly; when the last round of workgroups would leave most CUs idle,
// or the output has too few tiles for the chip, the affected tiles are split along K into fp32 partial tiles that a
// second kernel adds in fixed order (the result depends on the shape only, not on the run).
#pragma once
#include "mmq_formats.h"

namespace gguf {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr float kSeed = 12582912.0f;   // 1.5 * 2^23: unit in the last place 1, room for |S| < 2^22
constexpr int kSeedBits = 0x4B400000;

// fma on the float whose bits are `bits`.  Takes the MFMA element by value: a bit cast applied directly to a vector
// element expression reads element 0 with this compiler.
__device__ __forceinline__ float seeded_times(int bits, float dw, float neg_seed_dw) {
  return __builtin_fmaf(__int_as_float(bits), dw, neg_seed_dw);
}

// LDS row pitch in bytes.  Operands are read 16 bytes per lane: a 16-byte skew (KS + 16) spreads 8 consecutive rows
// over all banks.  The 16-deep formats multiply a 32-value block with two K=16 MFMAs, each of which wants 8 consecutive
// k per lane half; their blocks are stored as [k 0-7 | k 16-23 | k 8-15 | k 24-31], so that the 16 bytes at 16 * lhalf
// are this lane's operands of both MFMAs (one 16-byte read instead of two 8-byte reads at a pitch with bank conflicts).
template <int G, int KS> struct Pitch { static constexpr int value = KS + 16; };

constexpr int MMQI_KS = 128;  // values of K per step

template <class F, int M_T, int N_T>
__host__ __device__ constexpr size_t mmqi_buffer_bytes() {
  constexpr int KB = MMQI_KS / 32;
  // activation planes of KB x M_T floats: the block scales, then the stored block sums (offset formats) or the quant
  // sums of both 16-value groups of a block (MIN16); weight planes of KB x N_T float pairs: scales (and offset factors)
  constexpr int XP = !F::HAS_MIN ? 1 : F::MIN16 ? 3 : 2, WPL = F::MIN16 ? 2 : 1;
  return (size_t)(M_T + N_T) * Pitch<F::G, MMQI_KS>::value + (size_t)KB * M_T * 4 * XP + (size_t)KB * N_T * 8 * WPL;
}

// The grouped MoE contraction on this kernel: the rows of the workspace are the slots of the routing sort in order (slot s
// holds the quantized activations of the pair sorted_token_ids[s], zeros in padding), so a block of `block` slots is a
// run of rows like any other and only the weight matrix changes with it; the results are rows in slot order too.
struct MmqiMoe {
  const int32_t* expert_ids;              // expert of each block of slots; null = an ordinary product
  const int32_t* num_tokens_post_padded;  // slots in use: tiles past them leave
  int64_t expert_stride;                  // bytes between the matrices of two experts
  int block;                              // slots per block, a multiple of the tile's rows
};

template <class F, int WM, int WN, int TN, typename T>
__global__ __launch_bounds__(64 * WM * WN, 2) void mmqi_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                                int64_t ws_row_bytes, T* __restrict__ Y, float* __restrict__ partial,
                                                                int M, int N, int K, int Kp, int tiles_m, int whole_tiles,
                                                                int shared_tiles, int splits, int64_t w_pitch, int64_t ldy,
                                                                const T* __restrict__ bias, MmqiMoe moe) {
  constexpr int NT = 64 * WM * WN;
  constexpr int KS = MMQI_KS, KB = KS / 32, GR = KS / 16;
  constexpr int LDK = Pitch<F::G, KS>::value;
  constexpr int M_T = 32 * WM, N_T = 32 * WN * TN;
  constexpr int AQ = M_T * GR / NT;       // activation granules (16 bytes) per thread and step
  constexpr int PAIRS = N_T * KB;         // (weight row, 32-block) pairs per step
  constexpr int WP = (PAIRS + NT - 1) / NT;  // of them per thread
  static_assert(M_T * GR % NT == 0 && (PAIRS % NT == 0 || PAIRS < NT) && M_T <= NT, "tile and workgroup sizes must divide evenly");
  constexpr size_t BUF = mmqi_buffer_bytes<F, M_T, N_T>();
  static_assert(BUF % 16 == 0, "buffers keep 16-byte alignment");
  extern __shared__ __align__(16) char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int lrow = lane & 31, lhalf = lane >> 5;

  // Workgroup -> work.  The first `whole_tiles` workgroups take one output tile each over all of K; behind them every
  // further tile is shared by `splits` workgroups, each taking a stretch of K.  Workgroups go to the eight XCDs in
  // turn, so the whole tiles are renumbered to give an XCD a contiguous run of tiles: the tiles of one weight-row
  // block (consecutive numbers, token tile fastest) then share that XCD's L2.
  int wg = blockIdx.x;
  const int whole8 = whole_tiles & ~7;
  if (wg < whole8) wg = (wg & 7) * (whole8 >> 3) + (wg >> 3);
  int sw = wg - whole_tiles;                       // (>= 0: a workgroup on a shared tile; numbered the same way)
  const int shared8 = (shared_tiles * splits) & ~7;
  if (sw >= 0 && sw < shared8 && (whole_tiles & 7) == 0) sw = (sw & 7) * (shared8 >> 3) + (sw >> 3);
  const int tile = wg < whole_tiles ? wg : whole_tiles + sw % shared_tiles;
  const int split = wg < whole_tiles ? 0 : sw / shared_tiles;
  const int nsplit = wg < whole_tiles ? 1 : splits;
  const int m_base = (tile % tiles_m) * M_T, n_base = (tile / tiles_m) * N_T;
  if (moe.expert_ids) {
    if (m_base >= moe.num_tokens_post_padded[0]) return;
    const int e = moe.expert_ids[m_base / moe.block];
    if (e < 0 || e > 255) return;                    // the reference's guard on expert ids (moe.cuh:33)
    W += (int64_t)e * moe.expert_stride;
  }
  const int nkb_total = K >> 5;
  const int nsteps = (K + KS - 1) / KS;
  const int per_split = (nsteps + nsplit - 1) / nsplit;
  const int t0 = split * per_split, t1 = min(nsteps, t0 + per_split);

  // ---- per-thread staging plan, fixed over K
  const char* aq_src[AQ];
#pragma unroll
  for (int i = 0; i < AQ; ++i) {
    const int p = tid + NT * i, m = p / GR, g = p % GR;
    aq_src[i] = ws + (int64_t)min(m_base + m, M - 1) * ws_row_bytes + 16 * g;   // rows past M repeat the last row; never stored
  }
  const float* const as_src = (const float*)(ws + (int64_t)min(m_base + min(tid, M_T - 1), M - 1) * ws_row_bytes + Kp);
  const uint8_t* w_src[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int p = min(tid + NT * i, PAIRS - 1), n = p / KB;
    w_src[i] = W + (int64_t)min(n_base + n, N - 1) * w_pitch;
  }

  uint4 r_aq[AQ];
  f32x4 r_ad, r_as;
  typename F::Raw r_w[WP];

  auto fetch = [&](int t) {
    const int k0 = t * KS, kb0 = t * KB;
#pragma unroll
    for (int i = 0; i < AQ; ++i) r_aq[i] = *(const uint4*)(aq_src[i] + k0);   // q8 rows are padded to a multiple of 512
    if (tid < M_T) {
      r_ad = *(const f32x4*)(as_src + kb0);
      if (F::HAS_MIN && !F::MIN16) r_as = *(const f32x4*)(as_src + Kp / 32 + kb0);
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      if (PAIRS < NT && tid >= PAIRS) continue;   // wave-uniform: more threads than pairs
      const int kb = min(kb0 + ((tid + NT * i) % KB), nkb_total - 1);  // clamped: a block past K is re-read and scaled to nothing
      r_w[i] = F::fetch(w_src[i], kb);
    }
  };
  auto stash = [&](int t, int buf) {
    const int kb0 = t * KB;
    int8_t* xq = (int8_t*)smem + buf * BUF;
    int8_t* wq = xq + M_T * LDK;
    float* xd = (float*)(wq + N_T * LDK);
    float* xs = xd + KB * M_T;
    f32x2* wsc = (f32x2*)(xd + KB * M_T * (!F::HAS_MIN ? 1 : F::MIN16 ? 3 : 2));
    f32x2* wmn = wsc + KB * N_T;   // MIN16: {-min of group 0, -min of group 1} per block
#pragma unroll
    for (int i = 0; i < AQ; ++i) {
      const int p = tid + NT * i, m = p / GR, g = p % GR;
      const uint4 v = r_aq[i];   // past K the padded row holds zeros, past Kp the scales below are zero
      if constexpr (F::MIN16)    // this granule is one 16-value group: the sum of its quants, for the per-group offset term
        xs[g * M_T + m] = (float)dot4(0x01010101, (int)v.x, dot4(0x01010101, (int)v.y, dot4(0x01010101, (int)v.z, dot4(0x01010101, (int)v.w, 0))));
      if constexpr (F::G == 32) {
        *(uint4*)(xq + m * LDK + 16 * g) = v;
      } else {   // granule g holds k 0-15 (g even) or k 16-31 (g odd) of block g / 2: see Pitch
        int8_t* blk = xq + m * LDK + 32 * (g >> 1) + 8 * (g & 1);
        *(uint2*)blk = make_uint2(v.x, v.y);
        *(uint2*)(blk + 16) = make_uint2(v.z, v.w);
      }
    }
    if (tid < M_T) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const bool in = kb0 + kb < nkb_total;
        xd[kb * M_T + tid] = in ? r_ad[kb] : 0.0f;
        if (F::HAS_MIN && !F::MIN16) xs[kb * M_T + tid] = in ? r_as[kb] : 0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + NT * i, n = p / KB, kb = p % KB;
      if (PAIRS < NT && tid >= PAIRS) continue;
      uint32_t q[8];
      float s0, s1, mn = 0.0f, mn1 = 0.0f;
      F::unpack(r_w[i], kb0 + kb, q, s0, s1, mn, mn1);
      if (kb0 + kb >= nkb_total) s0 = s1 = mn = mn1 = 0.0f;
      if constexpr (F::G == 32) {
        *(uint4*)(wq + n * LDK + 32 * kb) = make_uint4(q[0], q[1], q[2], q[3]);
        *(uint4*)(wq + n * LDK + 32 * kb + 16) = make_uint4(q[4], q[5], q[6], q[7]);
      } else {
        *(uint4*)(wq + n * LDK + 32 * kb) = make_uint4(q[0], q[1], q[4], q[5]);
        *(uint4*)(wq + n * LDK + 32 * kb + 16) = make_uint4(q[2], q[3], q[6], q[7]);
      }
      wsc[kb * N_T + n] = F::G == 32 ? (f32x2){s0, -mn} : (f32x2){s0, s1};
      if constexpr (F::MIN16) wmn[kb * N_T + n] = (f32x2){-mn, -mn1};
    }
  };

  float acc[TN][16];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;

  v16i seed;
#pragma unroll
  for (int r = 0; r < 16; ++r) seed[r] = kSeedBits;

  // Operands of one 32-block for this wave.  Matrix operands: the activation rows (shared by the TN tiles) and the
  // weight rows of every tile.  Scale operands: the weight scales of every tile and the q8_1 scales (and stored sums)
  // of the 16 token rows a lane holds -- register r of an MFMA result is row 8 * (r / 4) + 4 * lhalf + r % 4.
  struct MmaOps {
    v4i a;          // 16-deep formats: {half 0 lo, half 0 hi, half 1 lo, half 1 hi}, 8 bytes per K=16 MFMA
    v4i b[TN];
  };
  struct ScaleOps {
    f32x2 sc[TN];   // 32-deep: {dw, -offset factor}; 16-deep: {dw of half 0, dw of half 1}
    f32x2 mn[F::MIN16 ? TN : 1];   // MIN16: {-min of half 0, -min of half 1}
    f32x4 d8[4], s8[4];           // s8: the stored block sums; MIN16: d8 x the quant sum of half 0
    f32x4 u8[F::MIN16 ? 4 : 1];   // MIN16: d8 x the quant sum of half 1
  };
  auto load_mma = [&](int buf, int kb, MmaOps& o) {
    const int8_t* xq = (const int8_t*)smem + buf * BUF;
    const int8_t* wq = xq + M_T * LDK;
    const int8_t* arow = xq + (32 * wm + lrow) * LDK + 32 * kb;
    o.a = *(const v4i*)(arow + 16 * lhalf);   // (16-deep formats: both halves' operands of this lane, see Pitch)
#pragma unroll
    for (int i = 0; i < TN; ++i) o.b[i] = *(const v4i*)(wq + (32 * (wn * TN + i) + lrow) * LDK + 32 * kb + 16 * lhalf);
  };
  auto load_scales = [&](int buf, int kb, ScaleOps& o) {
    const float* xd = (const float*)(smem + buf * BUF + (M_T + N_T) * LDK);
    const float* xs = xd + KB * M_T;
    const f32x2* wsc = (const f32x2*)(xd + KB * M_T * (!F::HAS_MIN ? 1 : F::MIN16 ? 3 : 2));
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      o.sc[i] = wsc[kb * N_T + 32 * (wn * TN + i) + lrow];
      if constexpr (F::MIN16) o.mn[i] = wsc[(KB + kb) * N_T + 32 * (wn * TN + i) + lrow];
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      o.d8[g] = *(const f32x4*)(xd + kb * M_T + 32 * wm + 8 * g + 4 * lhalf);
      if constexpr (F::MIN16) {   // d8 x the groups' quant sums, once per block and lane for all the tiles
        o.s8[g] = o.d8[g] * *(const f32x4*)(xs + (2 * kb) * M_T + 32 * wm + 8 * g + 4 * lhalf);
        o.u8[g] = o.d8[g] * *(const f32x4*)(xs + (2 * kb + 1) * M_T + 32 * wm + 8 * g + 4 * lhalf);
      } else if constexpr (F::HAS_MIN) {
        o.s8[g] = *(const f32x4*)(xs + kb * M_T + 32 * wm + 8 * g + 4 * lhalf);
      }
    }
  };
  // A unit is one MFMA and the rescale of its 16 results per lane: a (block, tile) pair for the 32-deep formats, one
  // 16-element half of such a pair for the 16-deep ones.
  constexpr int H = F::G == 32 ? 1 : 2;   // units per (block, tile)
  constexpr int UB = TN * H;              // units per block, tile-major, then half
  auto issue = [&](const MmaOps& o, int ub, v16i& s_out) {
    const int i = ub / H, h = ub % H;
    if constexpr (F::G == 32) {
      s_out = __builtin_amdgcn_mfma_i32_32x32x32_i8(o.a, o.b[i], seed, 0, 0, 0);
    } else {
      const long av = __builtin_bit_cast(long, (v2i){o.a[2 * h], o.a[2 * h + 1]});
      const long bv = __builtin_bit_cast(long, (v2i){o.b[i][2 * h], o.b[i][2 * h + 1]});
      s_out = __builtin_amdgcn_mfma_i32_32x32x16_i8(av, bv, seed, 0, 0, 0);
    }
  };
  auto rescale = [&](const ScaleOps& o, int ub, const v16i& s_in) {
    const int i = ub / H, h = ub % H;
    const float dw = F::G == 32 ? o.sc[i][0] : o.sc[i][h];
    const float nsd = -kSeed * dw;
    if constexpr (F::HALFPROD) {
      // Q4_1, Q5_1: S * half(d * d8) + half(m * s8), both products rounded to half precision as the reference's
      // __hmul2 leaves them (vecdotq.cuh:179-198); d, d8, m and s8 are half values held in floats
      const _Float16 dh = (_Float16)dw, mh = (_Float16)-o.sc[i][1];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const _Float16 dd = dh * (_Float16)o.d8[r >> 2][r & 3];
        const _Float16 ms = mh * (_Float16)o.s8[r >> 2][r & 3];
        acc[i][r] += (__int_as_float(s_in[r]) - kSeed) * (float)dd + (float)ms;
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float c = seeded_times(s_in[r], dw, nsd);   // = RN(S * dw)
        acc[i][r] = __builtin_fmaf(c, o.d8[r >> 2][r & 3], acc[i][r]);
        if constexpr (F::MIN16) {   // Q2_K: the group's min times d8 x the sum of the group's activation quants
          acc[i][r] = __builtin_fmaf(h ? o.u8[r >> 2][r & 3] : o.s8[r >> 2][r & 3], o.mn[i][h], acc[i][r]);
        } else if constexpr (F::HAS_MIN) {
          acc[i][r] = __builtin_fmaf(o.s8[r >> 2][r & 3], o.sc[i][1], acc[i][r]);
        }
      }
    }
  };
  // One step of K from buffer `buf`.  The matrix operands of block kb + 1 are requested while block kb is worked
  // through, and the MFMA of unit u + 1 is issued before unit u is rescaled, so that the matrix unit runs under the
  // vector instructions of the same wave.
  auto contract = [&](int buf) {
    MmaOps mo[2];
    ScaleOps so;
    v16i s_u[2];
    load_mma(buf, 0, mo[0]);
    issue(mo[0], 0, s_u[0]);
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      __builtin_amdgcn_sched_barrier(0);   // keeps the operand reads of later blocks from being hoisted up here
      load_scales(buf, kb, so);
      if (kb + 1 < KB) load_mma(buf, kb + 1, mo[(kb + 1) & 1]);
#pragma unroll
      for (int ub = 0; ub < UB; ++ub) {
        const int u = kb * UB + ub;
        if (ub + 1 < UB) issue(mo[kb & 1], ub + 1, s_u[(u + 1) & 1]);
        else if (kb + 1 < KB) issue(mo[(kb + 1) & 1], 0, s_u[(u + 1) & 1]);
        rescale(so, ub, s_u[u & 1]);
      }
    }
  };

  // Software pipeline, one register stage, two LDS buffers, one barrier per turn: in turn j the registers (step j+1,
  // loaded during turn j-1) are decoded into the other buffer, the loads of step j+2 are issued, and step j is
  // contracted.
  const int n = t1 - t0;
  if (n > 0) {
    fetch(t0);
    stash(t0, 0);
    if (n > 1) fetch(t0 + 1);
    __syncthreads();
    for (int j = 0; j < n; ++j) {
      if (j + 1 < n) {
        stash(t0 + j + 1, (j + 1) & 1);
        if (j + 2 < n) fetch(t0 + j + 2);
      }
      contract(j & 1);
      __syncthreads();
    }
  }

  // ---- store: lane = one output feature, 16 token rows per tile
  float* const my_partial = nsplit > 1 ? partial + ((int64_t)(tile - whole_tiles) * splits + split) * (M_T * N_T) : nullptr;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int ml = 32 * wm + 8 * (r >> 2) + 4 * lhalf + (r & 3), mt = m_base + ml;
#pragma unroll
    for (int i = 0; i < TN; ++i) {
      const int nl = 32 * (wn * TN + i) + lrow, nn = n_base + nl;
      if (my_partial) my_partial[ml * N_T + nl] = acc[i][r];   // the whole tile, edges included: the adder masks them
      else if (mt < M && nn < N) Y[(int64_t)mt * ldy + nn] = finish<T>(acc[i][r], bias, nn);
    }
  }
}

// Y tile = T(sum of its `splits` fp32 partial tiles), gridDim.y workgroups per split tile, fixed order of addition
template <int M_T, int N_T, typename T>
__global__ __launch_bounds__(256) void mmqi_reduce_kernel(const float* __restrict__ partial, T* __restrict__ Y, int M, int N,
                                                          int tiles_m, int whole_tiles, int splits, int64_t ldy,
                                                          const T* __restrict__ bias) {
  const int tile = whole_tiles + blockIdx.x;
  const int m_base = (tile % tiles_m) * M_T, n_base = (tile / tiles_m) * N_T;
  const float* p = partial + (int64_t)blockIdx.x * splits * (M_T * N_T);
  for (int i = (blockIdx.y * 256 + threadIdx.x) * 4; i < M_T * N_T; i += gridDim.y * 256 * 4) {
    f32x4 acc = *(const f32x4*)(p + i);
    for (int z = 1; z < splits; ++z) acc += *(const f32x4*)(p + (int64_t)z * (M_T * N_T) + i);
    const int m = m_base + i / N_T, nn = n_base + i % N_T;
    if (m >= M) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (nn + e < N) Y[(int64_t)m * ldy + nn + e] = finish<T>(acc[e], bias, nn + e);
  }
}

// How the tiles of one launch are handed out: `whole` tiles get a workgroup each, the remaining `shared` tiles are
// split `splits` ways along K.  partial_bytes() is the fp32 scratch the shared tiles need.
struct MmqiPlan {
  int cfg;            // 0: 128 x 64 tiles, four waves; 1: 64 x 128, four waves; 2: 256 x 128, eight waves; 3: 128 x 64, eight waves
  int whole, shared, splits;
  int mt() const { return cfg == 1 ? 64 : cfg == 2 ? 256 : 128; }
  int nt() const { return cfg == 1 || cfg == 2 ? 128 : 64; }
  int64_t partial_bytes() const { return (int64_t)shared * splits * mt() * nt() * 4; }
};
// `wide_ok`: the format's 256 x 128 kernel keeps its registers (Q5_K's does not)
MmqiPlan mmq_int_plan(int M, int N, int K, int64_t partial_bytes_available, bool wide_ok);  // mmq_i.hip

template <class F, int WM, int WN, int TN, typename T>
static void launch_mmqi(const void* W, const void* ws, void* Y, int M, int N, int K, hipStream_t stream, const MmqiPlan& p, float* partial,
                        const LinearArgs& la, const MmqiMoe& moe = MmqiMoe{nullptr, nullptr, 0, 0}) {
  const int64_t w_pitch = la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS, ldy = la.ldy ? la.ldy : (int64_t)N;
  constexpr int M_T = 32 * WM, N_T = 32 * WN * TN;
  constexpr size_t lds = 2 * mmqi_buffer_bytes<F, M_T, N_T>();
  auto kern = mmqi_kernel<F, WM, WN, TN, T>;
  if constexpr (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, lds, done);
  }
  const int tiles_m = (M + M_T - 1) / M_T;
  hipLaunchKernelGGL(kern, dim3(p.whole + p.shared * p.splits), dim3(64 * WM * WN), lds, stream, (const uint8_t*)W, (const char*)ws,
                     q8_row_bytes(K), (T*)Y, partial, M, N, K, (int)q8_kp(K), tiles_m, p.whole, p.shared > 0 ? p.shared : 1, p.splits, w_pitch,
                     ldy, (const T*)la.bias, moe);
  if (p.shared > 0)
    hipLaunchKernelGGL((mmqi_reduce_kernel<M_T, N_T, T>), dim3(p.shared, M_T * N_T / 1024), dim3(256), 0, stream, partial, (T*)Y, M, N,
                       tiles_m, p.whole, p.splits, ldy, (const T*)la.bias);
}

// Formats whose 256 x 128 kernel fits the register file without scratch worth mentioning.
template <class F> struct MmqiWide { static constexpr bool ok = true; };
template <> struct MmqiWide<MQ5_K> { static constexpr bool ok = false; };
template <> struct MmqiWide<MQ2_K> { static constexpr bool ok = false; };   // (three activation planes per block in registers)
template <> struct MmqiWide<MQ4_1> { static constexpr bool ok = false; };   // (the half-precision products' temporaries)
template <> struct MmqiWide<MQ5_1> { static constexpr bool ok = false; };

template <class F, typename T>
static int mmqi_typed(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, int64_t partial_bytes,
                      hipStream_t stream, const LinearArgs& la) {
  const MmqiPlan p = mmq_int_plan(M, N, K, partial_bytes, MmqiWide<F>::ok);
  if (p.cfg == 0) launch_mmqi<F, 4, 1, 2, T>(W, ws, Y, M, N, K, stream, p, partial, la);        // 128 x 64
  else if (p.cfg == 1) launch_mmqi<F, 2, 2, 2, T>(W, ws, Y, M, N, K, stream, p, partial, la);   // 64 x 128
  else if (p.cfg == 3) launch_mmqi<F, 4, 2, 1, T>(W, ws, Y, M, N, K, stream, p, partial, la);   // 128 x 64, eight waves
  else if constexpr (MmqiWide<F>::ok) launch_mmqi<F, 8, 1, 4, T>(W, ws, Y, M, N, K, stream, p, partial, la);   // 256 x 128
  return launch_status();
}

// The grouped contraction over `slots` rows in slot order (see MmqiMoe): blocks of 64 slots on 64 x 128 tiles, one block
// per row of tiles, every tile whole (the tiles of blocks past the padded total leave at once).
template <class F, typename T>
static int mmqi_moe_typed(const void* W, const void* ws, void* Y, int slots, int N, int K, const MmqiMoe& moe, hipStream_t stream) {
  const int rows = slots / 64 * 64;
  const MmqiPlan p = {1, (rows / 64) * ((N + 127) / 128), 0, 1};
  if (p.whole == 0) return GGUF_OK;
  launch_mmqi<F, 2, 2, 2, T>(W, ws, Y, rows, N, K, stream, p, nullptr, LinearArgs(), moe);
  return launch_status();
}

}  // namespace gguf
