// 16-row tiles of the integer engine on v_mfma_i32_16x16x32_i8, for the two places where a 32-row tile is mostly
// padding: the grouped MoE contraction for experts with few pairs (blocks of 16 sorted slots instead of 32), and the
// plain tile GEMM with 9 to 32 rows of X.
//
// With about eight pairs per expert (64 tokens, top-8 of 64 experts) three quarters of a 32-row tile are padding,
// and what the integer engine pays per tile -- the rescale of every MFMA result by its two block scales on the vector
// ALU -- does not shrink with the padding.  A 16 x 16 tile holds four results per lane instead of the sixteen of a
// 32 x 32 one, so the vector work per weight block halves.  Arithmetic and semantics are those of the 32-row kernels
// (reference: csrc/gguf/moe.cuh:5-129 and mmq.cuh:2-104; block dot products exact in int32, scales in fp32).  The
// formats whose weight scale changes every 16 values (Q6_K, Q3_K) issue the K=32 instruction twice per block, each
// time with the activations of the other half zeroed: gfx950 has no 16 x 16 x 16 int8 MFMA.
//
// Work split: a workgroup of NW waves owns 16 rows x (32 NW) output features and walks K in steps of 128 values; a
// wave owns 32 features = two 16 x 16 tiles.  The packed blocks of the weight rows are decoded once per step into LDS
// (two buffers, one barrier per step); global loads run two steps ahead in registers (one for Q6_K / Q3_K).
#include "mmq_i_core.h"
#include "q8_1_device.h"

namespace gguf {

typedef int v4i_t __attribute__((ext_vector_type(4)));

// Dense mode (MOE = false): the same tile for a plain product with 9 to 32 rows of X, where the 64 x 128 tiles of the
// integer engine would multiply mostly padding and leave most of the chip idle.  `tiles` output tiles of 16 rows x
// 16 CT NW features, each split `splits` ways along K when the output alone has too few tiles to fill the chip; split
// tiles leave fp32 partial tiles that mmqi_reduce_kernel adds in fixed order.
struct Dense16 {
  int M, splits;
  int64_t w_pitch, ldy;
  float* partial;
};

// GATE (with MOE): the first expert GEMM of a layer with its seam (Gate16, mmq_formats.h): a tile's 128 columns are the
// SAME 64 features of the gate and the up half.

template <class F, typename T, int NW, int OCC, bool MOE = true, bool GATE = false, int CT = 2>
__global__ __launch_bounds__(64 * NW, OCC) void moe16_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws, int64_t ws_row_bytes,
                                                        T* __restrict__ Y, int N, int K, int Kp, int tiles_m, int tiles, MoeArgs moe,
                                                        Dense16 dn, const T* __restrict__ bias, Gate16 gate) {
  static_assert(!GATE || (MOE && NW == 4 && CT == 2), "the gated epilogue pairs the halves of a 128-column tile");
  static_assert(!(F::G == 16 && F::HAS_MIN), "16-deep formats with per-group offsets keep the 32-row kernel");
  constexpr int NT = 64 * NW, KS = MMQI_KS, KB = KS / 32, GR = KS / 16, LDK = Pitch<32, KS>::value;
  constexpr int M_T = 16, N_T = 16 * CT * NW;   // CT 16-feature tiles per wave: two, or one where the output has few tiles
  constexpr int PAIRS = N_T * KB, WP = PAIRS / NT;  // (weight row, 32-block) pairs per step, per thread
  constexpr int DEPTH = F::G == 16 ? 1 : 2;          // (two stages of the large Q6_K / Q3_K blocks do not fit the registers)
  constexpr size_t BUF = (size_t)(M_T + N_T) * LDK + (size_t)KB * M_T * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)KB * N_T * 8;
  static_assert(BUF % 16 == 0 && PAIRS % NT == 0 && M_T * GR <= NT, "buffers keep 16-byte alignment; shares divide evenly");
  extern __shared__ __align__(16) char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lcol = lane & 15, lgrp = lane >> 4;     // MFMA operand: row / column lcol, k values [8 lgrp, +8); result rows 4 lgrp + r

  int wg = blockIdx.x;
  const int nsplit = MOE ? 1 : dn.splits;
  const int total = tiles * nsplit, total8 = total & ~7;   // workgroups go to the 8 XCDs in turn: give each a contiguous run
  if (wg < total8) wg = (wg & 7) * (total8 >> 3) + (wg >> 3);
  const int tile = wg % tiles, split = wg / tiles;
  const int block = tile % tiles_m, m_base = block * M_T, n_base = (tile / tiles_m) * (GATE ? N_T / 2 : N_T);
  int64_t w_pitch = (int64_t)(K / F::QK) * F::BS;
  if constexpr (MOE) {
    if (m_base >= moe.num_tokens_post_padded[0]) return;
    const int e = moe.expert_ids[block];
    if (e < 0 || e > 255) return;                   // the reference's guard (moe.cuh:33)
    W += (int64_t)e * moe.expert_stride;
  } else {
    w_pitch = dn.w_pitch;
  }
  const int nkb_total = K >> 5, nsteps_all = (K + KS - 1) / KS;
  const int per_split = (nsteps_all + nsplit - 1) / nsplit;
  const int t0 = split * per_split, nsteps = max(0, min(nsteps_all, t0 + per_split) - t0);
  const auto src_row = [&](int m) {                 // the row of the quantized activations behind tile row m
    if constexpr (MOE) {
      const int pair = moe.sorted_token_ids[m_base + m];
      return pair < moe.num_pairs ? pair / moe.top_k : 0;    // row 0 stands in for padding
    } else {
      return min(m_base + m, dn.M - 1);             // rows past M repeat the last row; never stored
    }
  };

  // ---- per-thread staging plan, fixed over K
  const char* const aq_src = ws + (int64_t)src_row(min(tid / GR, M_T - 1)) * ws_row_bytes + 16 * (tid % GR);   // threads < 128
  const float* const as_src = (const float*)(ws + (int64_t)src_row(min(tid, M_T - 1)) * ws_row_bytes + Kp);     // threads < 16
  const int sum_plane = (MOE && moe.gemv_sums ? 2 : 1) * (Kp / 32);
  const uint8_t* w_src[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int n = (tid + NT * i) / KB;   // column of the tile
    // GATE: columns 0..63 are features n_base .. of the gate half, 64..127 the same features of the up half
    const int row = GATE ? (n < N_T / 2 ? 0 : gate.inner) + min(n_base + (n & (N_T / 2 - 1)), gate.inner - 1) : min(n_base + n, N - 1);
    w_src[i] = W + (int64_t)row * w_pitch;
  }

  struct Stage {
    uint4 aq;
    f32x4 ad, as;
    typename F::Raw w[WP];
  };
  Stage stage[DEPTH];
  auto fetch = [&](int t, Stage& r) {
    const int k0 = t * KS, kb0 = t * KB;
    if (tid < M_T * GR) r.aq = *(const uint4*)(aq_src + k0);   // q8 rows are padded to a multiple of 512
    if (tid < M_T) {
      r.ad = *(const f32x4*)(as_src + kb0);
      if (F::HAS_MIN) r.as = *(const f32x4*)(as_src + sum_plane + kb0);
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) r.w[i] = F::fetch(w_src[i], min(kb0 + ((tid + NT * i) % KB), nkb_total - 1));
  };
  auto stash = [&](int t, int buf, const Stage& r) {
    const int kb0 = t * KB;
    int8_t* xq = (int8_t*)smem + buf * BUF;
    int8_t* wq = xq + M_T * LDK;
    float* xd = (float*)(wq + N_T * LDK);
    float* xs = xd + KB * M_T;
    f32x2* wsc = (f32x2*)(xd + KB * M_T * (F::HAS_MIN ? 2 : 1));
    if (tid < M_T * GR) *(uint4*)(xq + (tid / GR) * LDK + 16 * (tid % GR)) = r.aq;
    if (tid < M_T) {
#pragma unroll
      for (int kb = 0; kb < KB; ++kb) {
        const bool in = kb0 + kb < nkb_total;
        xd[kb * M_T + tid] = in ? r.ad[kb] : 0.0f;
        if (F::HAS_MIN) xs[kb * M_T + tid] = in ? r.as[kb] : 0.0f;
      }
    }
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + NT * i, n = p / KB, kb = p % KB;
      uint32_t q[8];
      float s0, s1, mn = 0.0f, mn1 = 0.0f;
      F::unpack(r.w[i], kb0 + kb, q, s0, s1, mn, mn1);
      if (kb0 + kb >= nkb_total) s0 = s1 = mn = 0.0f;   // a block past K was re-read: scaled to nothing
      *(uint4*)(wq + n * LDK + 32 * kb) = make_uint4(q[0], q[1], q[2], q[3]);
      *(uint4*)(wq + n * LDK + 32 * kb + 16) = make_uint4(q[4], q[5], q[6], q[7]);
      wsc[kb * N_T + n] = F::G == 32 ? (f32x2){s0, -mn} : (f32x2){s0, s1};   // 16-deep formats: one scale per half
    }
  };

  float acc[CT][4];
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[c][r] = 0.0f;
  const v4i_t seed = {kSeedBits, kSeedBits, kSeedBits, kSeedBits};

  auto contract = [&](int buf) {
    const int8_t* xq = (const int8_t*)smem + buf * BUF;
    const int8_t* wq = xq + M_T * LDK;
    const float* xd = (const float*)(wq + N_T * LDK);
    const float* xs = xd + KB * M_T;
    const f32x2* wsc = (const f32x2*)(xd + KB * M_T * (F::HAS_MIN ? 2 : 1));
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const f32x4 d8 = *(const f32x4*)(xd + kb * M_T + 4 * lgrp);
      f32x4 s8 = {0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (F::HAS_MIN) s8 = *(const f32x4*)(xs + kb * M_T + 4 * lgrp);
      if constexpr (F::G == 32) {
        const long a = *(const long*)(xq + lcol * LDK + 32 * kb + 8 * lgrp);
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          const int col = 16 * CT * wave + 16 * c + lcol;
          const long b = *(const long*)(wq + col * LDK + 32 * kb + 8 * lgrp);
          const f32x2 sc = wsc[kb * N_T + col];
          const v4i_t s = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, seed, 0, 0, 0);
          const float nsd = -kSeed * sc[0];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float t = seeded_times(s[r], sc[0], nsd);   // = RN(S * dw)
            acc[c][r] = __builtin_fmaf(t, d8[r], acc[c][r]);
            if constexpr (F::HAS_MIN) acc[c][r] = __builtin_fmaf(s8[r], sc[1], acc[c][r]);
          }
        }
      } else {
        // the weight scale changes every 16 values: one MFMA per half block, the same K=32 instruction with the
        // activations of the other half zeroed (k groups 0, 1 are the first half, 2, 3 the second)
        const long a = *(const long*)(xq + lcol * LDK + 32 * kb + 8 * lgrp);
        const long a0 = lgrp < 2 ? a : 0L, a1 = lgrp < 2 ? 0L : a;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
          const int col = 16 * CT * wave + 16 * c + lcol;
          const long b = *(const long*)(wq + col * LDK + 32 * kb + 8 * lgrp);
          const f32x2 sc = wsc[kb * N_T + col];
          const v4i_t sa = __builtin_amdgcn_mfma_i32_16x16x32_i8(a0, b, seed, 0, 0, 0);
          const v4i_t sb = __builtin_amdgcn_mfma_i32_16x16x32_i8(a1, b, seed, 0, 0, 0);
          const float nsa = -kSeed * sc[0], nsb = -kSeed * sc[1];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            acc[c][r] = __builtin_fmaf(seeded_times(sa[r], sc[0], nsa), d8[r], acc[c][r]);
            acc[c][r] = __builtin_fmaf(seeded_times(sb[r], sc[1], nsb), d8[r], acc[c][r]);
          }
        }
      }
    }
  };

  // Software pipeline: in turn j the registers of step j+1 are decoded into the other buffer, the loads of step
  // j+1+DEPTH are issued into the registers just freed, and step j is contracted.  (Because some of the loads are
  // issued by part of the threads only, the compiler cannot count the loads in flight exactly and waits for all of
  // them before a stage is decoded, which leaves the second stage about one turn of lead.  Making every thread issue
  // every load gives exact counts and was measured slower, 63 against 53 us for the first expert GEMM of the 64-token
  // layer: the redundant activation loads cost more than the lead gains.)
  if (nsteps > 0) {
    fetch(t0, stage[0]);
    stash(t0, 0, stage[0]);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (1 + d < nsteps) fetch(t0 + 1 + d, stage[d]);
    __syncthreads();
    for (int j0 = 0; j0 < nsteps; j0 += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {   // (stage indices are compile-time: the stages live in registers)
        const int j = j0 + d;
        if (j < nsteps) {
          if (j + 1 < nsteps) {
            stash(t0 + j + 1, (j + 1) & 1, stage[d]);
            if (j + 1 + DEPTH < nsteps) fetch(t0 + j + 1 + DEPTH, stage[d]);
          }
          contract(j & 1);
          __syncthreads();
        }
      }
    }
  }

  if constexpr (GATE) {
    // ---- the tile's sums, rounded as the operator stores them, meet in LDS (the buffers are free: the loop ends on a
    // barrier); then 8 threads per slot take 8 features each of both halves, and every four of them form one q8_1 block
    float* yt = (float*)smem;   // [16][128]
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int c = 0; c < CT; ++c) yt[(4 * lgrp + r) * N_T + 16 * CT * wave + 16 * c + lcol] = to_f32<T>(from_f32<T>(acc[c][r]));
    __syncthreads();
    if (tid < 16 * 8) {
      const int slot = tid >> 3, part = tid & 7;
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
  // ---- store: lane = one output feature of each of its tiles, four rows
  if constexpr (!MOE) {
    if (nsplit > 1) {   // the whole partial tile, edges included: the adder masks them
      float* const mine = dn.partial + ((int64_t)tile * nsplit + split) * (M_T * N_T);
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < CT; ++c) mine[(4 * lgrp + r) * N_T + 16 * CT * wave + 16 * c + lcol] = acc[c][r];
      return;
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    int64_t row;
    if constexpr (MOE) {
      const int pair = moe.sorted_token_ids[m_base + 4 * lgrp + r];
      if (pair >= moe.num_pairs) continue;
      row = (int64_t)pair * N;
    } else {
      if (m_base + 4 * lgrp + r >= dn.M) continue;
      row = (int64_t)(m_base + 4 * lgrp + r) * dn.ldy;
    }
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const int nn = n_base + 16 * CT * wave + 16 * c + lcol;
      if (nn < N) Y[row + nn] = finish<T>(acc[c][r], MOE ? (const T*)nullptr : bias, nn);
    }
  }
}

// Three workgroups of the MoE tile kernel fit a CU.  When the blocks that hold pairs make a little more than one round
// of those (how many there are is known on the device only: the estimate takes the pairs as spread over the experts at
// random), the second round's few workgroups land three to a CU where the first finished first and take as long as the
// first round; with two per CU the same tiles make two full rounds, which is shorter: Q4_0, 64 experts [2048,2048], 32
// tokens top-8, 62 blocks of 64: 63 -> 55 us (the gated first GEMM of the layer 60 -> 51 us); 70 blocks the other way
// round, 64 against 71 us.  A larger LDS request is what limits a CU to two: the bytes to ask for.
static inline size_t moe16_lds_request(size_t lds, int num_sorted, int num_pairs, int tiles_n) {
  const double experts = (double)(num_sorted - num_pairs) / 15.0;   // the sorted array has room for 15 padding slots per expert
  if (experts < 1.0) return lds;
  const double lam = (double)num_pairs / experts;
  double blocks = 0.0, term = exp(-lam), cdf = 0.0, one_block = 0.0;   // sum over j >= 0 of P(pairs of an expert > 16 j)
  for (int c = 0; c <= 64; ++c) {
    cdf += term;
    if (c % 16 == 0) blocks += 1.0 - cdf;
    if (c == 16) one_block = cdf - exp(-lam);          // P(1 .. 16 pairs): the expert has exactly one block
    term *= lam / (c + 1);
  }
  const double est = blocks * experts * tiles_n, cus = (double)num_cus();
  // (exactly four tiles per CU is the one case in which three per CU do finish as three and one: 53 us above, and
  //  the layer's second GEMM 28 against 31 us -- kept when every expert is likely to have exactly one block)
  const bool four_each = (int)(experts + 0.5) * tiles_n == 4 * (int)cus && pow(one_block, experts) >= 0.8;
  return est > 3.0 * cus && est <= 4.0 * cus && !four_each && lds < 54 * 1024 ? (size_t)54 * 1024 : lds;
}

// The same contraction on tiles of 64 features (one 16-feature tile per wave, four or five workgroups per CU): what a GEMM
// with few blocks and a narrow output takes, whose 128-feature tiles would leave CUs idle (8 experts x [4096,14336] at 64
// tokens: 256 .. 512 tiles of 112 steps each for 768 places).
template <class F, typename T>
static int moe16_narrow_typed(const void* W, const void* ws, void* Y, int N, int K, int num_sorted, const MoeArgs& moe, hipStream_t stream) {
  constexpr int NW = 4, N_T = 16 * NW, OCC = 4;
  constexpr size_t BUF = (size_t)(16 + N_T) * Pitch<32, MMQI_KS>::value + (size_t)4 * 16 * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)4 * N_T * 8;
  constexpr size_t lds = 2 * BUF;
  auto kern = moe16_kernel<F, T, NW, OCC, true, false, 1>;
  const int tiles_n = (N + N_T - 1) / N_T, tiles_m = num_sorted / 16, tiles = tiles_m * tiles_n;
  if (tiles == 0) return GGUF_OK;
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(64 * NW), lds, stream, (const uint8_t*)W, (const char*)ws, q8_row_bytes(K), (T*)Y, N, K,
                     (int)q8_kp(K), tiles_m, tiles, moe, Dense16{}, (const T*)nullptr, Gate16{});
  return launch_status();
}

template <class F, typename T>
static int moe16_typed(const void* W, const void* ws, void* Y, int N, int K, int num_sorted, const MoeArgs& moe, hipStream_t stream) {
  // four waves, three workgroups per CU (two for Q5_K, whose packed block needs the registers); eight waves with one
  // workgroup per CU, or two waves with four, measured within 5 % of this
  constexpr int NW = 4, N_T = 32 * NW, OCC = sizeof(typename F::Raw) > 64 ? 2 : 3;
  constexpr size_t BUF = (size_t)(16 + N_T) * Pitch<32, MMQI_KS>::value + (size_t)4 * 16 * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)4 * N_T * 8;
  constexpr size_t lds = 2 * BUF;
  auto kern = moe16_kernel<F, T, NW, OCC>;
  if constexpr (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, lds, done);
  }
  const int tiles_n = (N + N_T - 1) / N_T, tiles_m = num_sorted / 16, tiles = tiles_m * tiles_n;
  if (tiles == 0) return GGUF_OK;
  // (the blocks that hold pairs, estimated: fewer tiles than the chip has places -> tiles of 64 features)
  if (moe_blocks_estimate(num_sorted, moe.num_pairs, 16) * tiles_n < (double)(OCC * num_cus()))
    return moe16_narrow_typed<F, T>(W, ws, Y, N, K, num_sorted, moe, stream);
  const size_t lds_req = OCC == 3 ? moe16_lds_request(lds, num_sorted, moe.num_pairs, tiles_n) : lds;
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(64 * NW), lds_req, stream, (const uint8_t*)W, (const char*)ws, q8_row_bytes(K), (T*)Y, N, K,
                     (int)q8_kp(K), tiles_m, tiles, moe, Dense16{}, (const T*)nullptr, Gate16{});
  return launch_status();
}

// The first expert GEMM of a layer with the gated activation and the q8_1 quantisation of its result in the epilogue
// (see Gate16): W is [experts][2 inner][K packed], the result goes to q8h.
template <class F, typename T>
static int moe16_gate_typed(const void* W, const void* ws, void* q8h, int inner, int K, int num_sorted, const MoeArgs& moe, int act,
                            hipStream_t stream) {
  constexpr int NW = 4, N_T = 32 * NW, OCC = sizeof(typename F::Raw) > 64 ? 2 : 3;
  constexpr size_t BUF = (size_t)(16 + N_T) * Pitch<32, MMQI_KS>::value + (size_t)4 * 16 * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)4 * N_T * 8;
  constexpr size_t lds = 2 * BUF;
  static_assert(lds >= 16 * N_T * 4, "the tile of sums fits the buffers");
  auto kern = moe16_kernel<F, T, NW, OCC, true, true>;
  if constexpr (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, lds, done);
  }
  const int tiles_n = (inner + N_T / 2 - 1) / (N_T / 2), tiles_m = num_sorted / 16, tiles = tiles_m * tiles_n;
  if (tiles == 0) return GGUF_OK;
  const size_t lds_req = OCC == 3 ? moe16_lds_request(lds, num_sorted, moe.num_pairs, tiles_n) : lds;
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(64 * NW), lds_req, stream, (const uint8_t*)W, (const char*)ws, q8_row_bytes(K), (T*)nullptr, 2 * inner, K,
                     (int)q8_kp(K), tiles_m, tiles, moe, Dense16{}, (const T*)nullptr,
                     Gate16{(char*)q8h, q8_row_bytes(inner), inner, (int)q8_kp(inner), act});
  return launch_status();
}

// The plain product for 9 .. 32 rows of X on the same tile.  The chip holds 3 x 256 workgroups of this kernel: an output
// with fewer tiles is split along K (at least four steps of 128 values per stretch, at most 16 ways) when the workspace
// has room for the partial tiles.  Measured on Q4_K [14336,4096] at 16 rows: aiming at 384 workgroups 26.3 us, 768
// 24.4 us, 1536 28.7 us, no split 46.5 us.
static inline int dense16_splits(int M, int N, int K, int64_t partial_bytes_available) {
  const int64_t tiles = (int64_t)((M + 15) / 16) * ((N + 127) / 128);
  const int nsteps = (K + MMQI_KS - 1) / MMQI_KS;
  int s = tiles > 0 ? (int)(768 / tiles) : 1;
  if (s > nsteps / 4) s = nsteps / 4;   // a stretch shorter than four steps is mostly prologue
  if (s > 16) s = 16;
  if (s < 2) return 1;
  return tiles * s * (16 * 128 * 4) <= partial_bytes_available ? s : 1;
}
int64_t rows16_direct_partial_bytes(int M, int N, int K);   // rows16_direct.hip
int64_t mmq_rows16_partial_bytes(int M, int N, int K) {
  const int s = dense16_splits(M, N, K, INT64_MAX);
  const int64_t tiled = s > 1 ? (int64_t)((M + 15) / 16) * ((N + 127) / 128) * s * (16 * 128 * 4) : 0;
  return std::max(tiled, rows16_direct_partial_bytes(M, N, K));
}

template <class F, typename T>
static int dense16_typed(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, int64_t partial_bytes,
                         hipStream_t stream, const LinearArgs& la) {
  constexpr int NW = 4, N_T = 32 * NW, OCC = sizeof(typename F::Raw) > 64 ? 2 : 3;
  constexpr size_t BUF = (size_t)(16 + N_T) * Pitch<32, MMQI_KS>::value + (size_t)4 * 16 * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)4 * N_T * 8;
  constexpr size_t lds = 2 * BUF;
  auto kern = moe16_kernel<F, T, NW, OCC, false>;
  if constexpr (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, lds, done);
  }
  const int tiles_m = (M + 15) / 16, tiles = tiles_m * ((N + N_T - 1) / N_T);
  const int splits = dense16_splits(M, N, K, partial_bytes);
  const int64_t w_pitch = la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS, ldy = la.ldy ? la.ldy : (int64_t)N;
  hipLaunchKernelGGL(kern, dim3(tiles * splits), dim3(64 * NW), lds, stream, (const uint8_t*)W, (const char*)ws, q8_row_bytes(K), (T*)Y, N, K,
                     (int)q8_kp(K), tiles_m, tiles, MoeArgs{}, Dense16{M, splits, w_pitch, ldy, partial}, (const T*)la.bias, Gate16{});
  if (splits > 1)
    hipLaunchKernelGGL((mmqi_reduce_kernel<16, N_T, T>), dim3(tiles, 2), dim3(256), 0, stream, partial, (T*)Y, M, N, tiles_m, 0, splits,
                       ldy, (const T*)la.bias);
  return launch_status();
}

template <class F>
static int dense16_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, float* partial, int64_t partial_bytes,
                       hipStream_t s, const LinearArgs& la) {
  GGUF_DISPATCH_DTYPE(dtype, return (dense16_typed<F, scalar_t>(W, ws, Y, M, N, K, partial, partial_bytes, s, la)));
  return GGUF_ERR_DTYPE;
}

int rows16_direct(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial, int64_t partial_bytes,
                  hipStream_t s, const LinearArgs& la, bool gemv_sums);   // rows16_direct.hip
bool rows16_direct_pays(int type, int M, int64_t N, int64_t K, bool against_gemv);

// q8_1(X) . W^T for a few rows of X (the quantized rows are in the workspace); GGUF_NOT_TAKEN for other formats.
int mmq_rows16(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial, int64_t partial_bytes,
               hipStream_t s, const LinearArgs& la) {
  if (rows16_direct_pays(type, M, N, K, false)) {   // straight from the packed blocks (the K-quants up to 32 rows, Q4_0 / Q8_0 up to 16)
    const int rc = rows16_direct(W, ws, Y, dtype, type, M, N, K, partial, partial_bytes, s, la, false);
    if (rc != GGUF_NOT_TAKEN) return rc;
  }
  // the 16-deep formats pay two MFMAs and four vector instructions per result and block on the staged tiles as in the
  // large tiles, and with two 16-row tiles (17 .. 32 rows) the large tiles are as fast: Q3_K [14336,4096] 44 us either way
  if ((type == T_Q6_K || type == T_Q3_K) && M > 16) return GGUF_NOT_TAKEN;
  switch (type) {
    case T_Q4_0: return dense16_fmt<MQ4_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q8_0: return dense16_fmt<MQ8_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_0: return dense16_fmt<MQ5_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q3_K: return dense16_fmt<MQ3_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q6_K: return dense16_fmt<MQ6_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q4_K: return dense16_fmt<MQ4_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_K: return dense16_fmt<MQ5_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_IQ4_XS: return dense16_fmt<MIQ4_XS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_IQ2_XXS: return dense16_fmt<MIQ2_XXS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
  }
  return GGUF_NOT_TAKEN;
}

template <class F>
static int moe16_fmt(const void* W, const void* ws, void* Y, int dtype, int N, int K, int num_sorted, const MoeArgs& moe, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe16_typed<F, scalar_t>(W, ws, Y, N, K, num_sorted, moe, s)));
  return GGUF_ERR_DTYPE;
}

bool moe_tiles16_ok(int type) {
  switch (type) {
    case T_Q4_0: case T_Q8_0: case T_Q3_K: case T_Q4_K: case T_Q5_K: case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: return true;
    default: return false;   // formats with other scale rules (Q4_1, Q5_1, Q2_K; Q5_0 in the per-pair operator) keep the 32-slot kernel
  }
}

template <class F>
static int moe16_gate_fmt(const void* W, const void* ws, void* q8h, int dtype, int inner, int K, int num_sorted, const MoeArgs& moe, int act,
                          hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe16_gate_typed<F, scalar_t>(W, ws, q8h, inner, K, num_sorted, moe, act, s)));
  return GGUF_ERR_DTYPE;
}

// The first expert GEMM over blocks of 16 slots with the activation and the quantisation of its result inside; dtype is
// the dtype the separate operator would have stored its result in.  GGUF_NOT_TAKEN for formats without 16-slot tiles.
int moe_tiles16_gate(const void* W, const void* ws, void* q8h, int dtype, int type, int inner, int K, int num_sorted, const MoeArgs& moe,
                     int act, hipStream_t s) {
  switch (type) {
    case T_Q4_0: return moe16_gate_fmt<MQ4_0>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_Q8_0: return moe16_gate_fmt<MQ8_0>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_Q3_K: return moe16_gate_fmt<MQ3_K>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_Q6_K: return moe16_gate_fmt<MQ6_K>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_Q4_K: return moe16_gate_fmt<MQ4_K>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_Q5_K: return moe16_gate_fmt<MQ5_K>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_IQ4_XS: return moe16_gate_fmt<MIQ4_XS>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
    case T_IQ2_XXS: return moe16_gate_fmt<MIQ2_XXS>(W, ws, q8h, dtype, inner, K, num_sorted, moe, act, s);
  }
  return GGUF_NOT_TAKEN;
}

// The contraction over blocks of 16 sorted slots (moe_align_block_size with block 16); GGUF_NOT_TAKEN for other formats.
int moe_tiles16(const void* W, const void* ws, void* Y, int dtype, int type, int N, int K, int num_sorted, const MoeArgs& moe,
                hipStream_t s) {
  switch (type) {
    case T_Q4_0: return moe16_fmt<MQ4_0>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q8_0: return moe16_fmt<MQ8_0>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q3_K: return moe16_fmt<MQ3_K>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q6_K: return moe16_fmt<MQ6_K>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q4_K: return moe16_fmt<MQ4_K>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q5_K: return moe16_fmt<MQ5_K>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_IQ4_XS: return moe16_fmt<MIQ4_XS>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_IQ2_XXS: return moe16_fmt<MIQ2_XXS>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
  }
  return GGUF_NOT_TAKEN;
}

}  // namespace gguf
