// The grouped MoE contraction for experts with few pairs: 16 sorted slots per block instead of 32.
//
// With about eight pairs per expert (64 tokens, top-8 of 64 experts) three quarters of a 32-row tile are padding,
// and what the integer engine pays per tile -- the rescale of every MFMA result by its two block scales on the vector
// ALU -- does not shrink with the padding.  This kernel contracts a block of 16 slots with v_mfma_i32_16x16x32_i8:
// four results per lane and 16 x 16 tile instead of sixteen per 32 x 32, so the vector work per weight block halves
// and the kernel's time is set by how fast the experts' weights stream in.  Arithmetic and semantics are those of
// the 32-slot kernels (reference: csrc/gguf/moe.cuh:5-129; block dot products exact in int32, scales in fp32).
//
// Work split: a workgroup of NW waves owns (one block of 16 slots) x (32 NW output features) and walks K in steps of
// 128 values; a wave owns 32 features = two 16 x 16 tiles.  The packed blocks of the weight rows are decoded once per
// step into LDS (two buffers, one barrier per step); global loads run two steps ahead in registers.
#include "mmq_i_core.h"

namespace gguf {

typedef int v4i_t __attribute__((ext_vector_type(4)));

template <class F, typename T, int NW, int OCC>
__global__ __launch_bounds__(64 * NW, OCC) void moe16_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws, int64_t ws_row_bytes,
                                                        T* __restrict__ Y, int N, int K, int Kp, int tiles_m, int tiles, MoeArgs moe) {
  static_assert(F::G == 32, "formats whose weight scale holds for a whole 32-value block");
  constexpr int NT = 64 * NW, KS = MMQI_KS, KB = KS / 32, GR = KS / 16, LDK = Pitch<32, KS>::value;
  constexpr int M_T = 16, CT = 2, N_T = 16 * CT * NW;   // two 16-feature tiles per wave
  constexpr int PAIRS = N_T * KB, WP = PAIRS / NT;  // (weight row, 32-block) pairs per step, per thread
  constexpr int DEPTH = 2;
  constexpr size_t BUF = (size_t)(M_T + N_T) * LDK + (size_t)KB * M_T * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)KB * N_T * 8;
  static_assert(BUF % 16 == 0 && PAIRS % NT == 0 && M_T * GR <= NT, "buffers keep 16-byte alignment; shares divide evenly");
  extern __shared__ __align__(16) char smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lcol = lane & 15, lgrp = lane >> 4;     // MFMA operand: row / column lcol, k values [8 lgrp, +8); result rows 4 lgrp + r

  int wg = blockIdx.x;
  const int tiles8 = tiles & ~7;                    // workgroups go to the 8 XCDs in turn: give each a contiguous run
  if (wg < tiles8) wg = (wg & 7) * (tiles8 >> 3) + (wg >> 3);
  const int block = wg % tiles_m, m_base = block * M_T, n_base = (wg / tiles_m) * N_T;
  if (m_base >= moe.num_tokens_post_padded[0]) return;
  const int e = moe.expert_ids[block];
  if (e < 0 || e > 255) return;                     // the reference's guard (moe.cuh:33)
  W += (int64_t)e * moe.expert_stride;
  const int64_t w_pitch = (int64_t)(K / F::QK) * F::BS;
  const int nkb_total = K >> 5, nsteps = (K + KS - 1) / KS;
  const auto src_row = [&](int m) {                 // the token row behind slot m of the block; row 0 stands in for padding
    const int pair = moe.sorted_token_ids[m_base + m];
    return pair < moe.num_pairs ? pair / moe.top_k : 0;
  };

  // ---- per-thread staging plan, fixed over K
  const char* const aq_src = ws + (int64_t)src_row(min(tid / GR, M_T - 1)) * ws_row_bytes + 16 * (tid % GR);   // threads < 128
  const float* const as_src = (const float*)(ws + (int64_t)src_row(min(tid, M_T - 1)) * ws_row_bytes + Kp);     // threads < 16
  const int sum_plane = (moe.gemv_sums ? 2 : 1) * (Kp / 32);
  const uint8_t* w_src[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) w_src[i] = W + (int64_t)min(n_base + (tid + NT * i) / KB, N - 1) * w_pitch;

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
      if (kb0 + kb >= nkb_total) s0 = mn = 0.0f;      // a block past K was re-read: scaled to nothing
      *(uint4*)(wq + n * LDK + 32 * kb) = make_uint4(q[0], q[1], q[2], q[3]);
      *(uint4*)(wq + n * LDK + 32 * kb + 16) = make_uint4(q[4], q[5], q[6], q[7]);
      wsc[kb * N_T + n] = (f32x2){s0, -mn};
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
      const long a = *(const long*)(xq + lcol * LDK + 32 * kb + 8 * lgrp);
      const f32x4 d8 = *(const f32x4*)(xd + kb * M_T + 4 * lgrp);
      f32x4 s8 = {0.0f, 0.0f, 0.0f, 0.0f};
      if constexpr (F::HAS_MIN) s8 = *(const f32x4*)(xs + kb * M_T + 4 * lgrp);
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        const int col = 32 * wave + 16 * c + lcol;
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
    }
  };

  // Software pipeline: in turn j the registers of step j+1 are decoded into the other buffer, the loads of step
  // j+1+DEPTH are issued into the registers just freed, and step j is contracted.  (Because some of the loads are
  // issued by part of the threads only, the compiler cannot count the loads in flight exactly and waits for all of
  // them before a stage is decoded, which leaves the second stage about one turn of lead.  Making every thread issue
  // every load gives exact counts and was measured slower, 63 against 53 us for the first expert GEMM of the 64-token
  // layer: the redundant activation loads cost more than the lead gains.)
  fetch(0, stage[0]);
  stash(0, 0, stage[0]);
#pragma unroll
  for (int d = 0; d < DEPTH; ++d)
    if (1 + d < nsteps) fetch(1 + d, stage[d]);
  __syncthreads();
  for (int j0 = 0; j0 < nsteps; j0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {   // (stage indices are compile-time: the stages live in registers)
      const int j = j0 + d;
      if (j < nsteps) {
        if (j + 1 < nsteps) {
          stash(j + 1, (j + 1) & 1, stage[d]);
          if (j + 1 + DEPTH < nsteps) fetch(j + 1 + DEPTH, stage[d]);
        }
        contract(j & 1);
        __syncthreads();
      }
    }
  }

  // ---- store: lane = one output feature of each of its tiles, four slots
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int pair = moe.sorted_token_ids[m_base + 4 * lgrp + r];
    if (pair >= moe.num_pairs) continue;
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const int nn = n_base + 32 * wave + 16 * c + lcol;
      if (nn < N) Y[(int64_t)pair * N + nn] = finish<T>(acc[c][r], (const T*)nullptr, nn);
    }
  }
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
  const int tiles_m = num_sorted / 16, tiles = tiles_m * ((N + N_T - 1) / N_T);
  if (tiles == 0) return GGUF_OK;
  hipLaunchKernelGGL(kern, dim3(tiles), dim3(64 * NW), lds, stream, (const uint8_t*)W, (const char*)ws, q8_row_bytes(K), (T*)Y, N, K,
                     (int)q8_kp(K), tiles_m, tiles, moe);
  return launch_status();
}

template <class F>
static int moe16_fmt(const void* W, const void* ws, void* Y, int dtype, int N, int K, int num_sorted, const MoeArgs& moe, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe16_typed<F, scalar_t>(W, ws, Y, N, K, num_sorted, moe, s)));
  return GGUF_ERR_DTYPE;
}

bool moe_tiles16_ok(int type) {
  switch (type) {
    case T_Q4_0: case T_Q8_0: case T_Q4_K: case T_Q5_K: case T_IQ4_XS: case T_IQ2_XXS: return true;
    default: return false;   // 16-deep formats and those with other scale rules keep the 32-slot kernel
  }
}

// The contraction over blocks of 16 sorted slots (moe_align_block_size with block 16); GGUF_NOT_TAKEN for other formats.
int moe_tiles16(const void* W, const void* ws, void* Y, int dtype, int type, int N, int K, int num_sorted, const MoeArgs& moe,
                hipStream_t s) {
  switch (type) {
    case T_Q4_0: return moe16_fmt<MQ4_0>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q8_0: return moe16_fmt<MQ8_0>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q4_K: return moe16_fmt<MQ4_K>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_Q5_K: return moe16_fmt<MQ5_K>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_IQ4_XS: return moe16_fmt<MIQ4_XS>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
    case T_IQ2_XXS: return moe16_fmt<MIQ2_XXS>(W, ws, Y, dtype, N, K, num_sorted, moe, s);
  }
  return GGUF_NOT_TAKEN;
}

}  // namespace gguf
