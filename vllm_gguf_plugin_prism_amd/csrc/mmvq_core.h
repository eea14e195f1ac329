// Decode-path GEMV on packed GGUF weights with q8_1 activations (gfx950).
//
//   Y[m, n] = sum over blocks of  dot(W block of row n, q8_1 block(s) of X[m])
//
// with the per-format block formulas of the reference's vec_dot_<fmt>_q8_1
// functions (csrc/gguf/vecdotq.cuh; cited at each format below).  The work
// split is not the reference's "one 64-lane wave per (row, vector)" grid
// (csrc/gguf/mmvq.cuh:2-50): here
//   * a workgroup of four waves owns 4*RPW consecutive rows, so its weight bytes
//     are one contiguous span of HBM, and every lane pulls 16 bytes per load;
//   * the quantized activations of up to eight vectors are staged once per
//     workgroup in LDS (quants + block scales), and every weight byte loaded is
//     used for all of them, so weights cross HBM once per call for M <= 8;
//   * a "unit" is the 32 weights one lane turns into int8 dot products per step;
//     partial sums stay in fp32 registers and are reduced with DPP at the end.
#pragma once
#include <type_traits>

#include "q8_1_device.h"
#include "grid_codes.h"

namespace gguf {


enum { AUX_NONE = 0, AUX_S8 = 1, AUX_DU = 2 };

struct Act {            // LDS views of one staged activation vector
  const int8_t* q;      // [kc]
  const float* d;       // [kc/32] block scales
  const float* a;       // [kc/32] block sums (AUX_S8) or d*sum(q) (AUX_DU)
  const char* tab;      // format lookup tables in LDS (i-quants)
};

// Every format splits its work in two: load() only issues global loads into raw registers (no use of
// the loaded values, so consecutive loads stay in flight together), dot() decodes and multiplies.
__device__ __forceinline__ float h2f(uint32_t bits) { return (float)__builtin_bit_cast(_Float16, (uint16_t)bits); }


}  // namespace gguf

#include "mmvq_formats.h"

namespace gguf {

// ------------------------------------------------------------------ kernel
// MOE selects the per-pair variant (reference: csrc/gguf/moe_vec.cuh:3-53): blockIdx.y is the flat
// (token, k) pair z; its expert topk_ids[z] picks the weight matrix (experts densely packed), its
// token z / top_k picks the activation row, and the result goes to row z of Y.
// With MoeVecArgs::sorted_ids set, blockIdx.y is instead a block of MT slots of one expert out of the routing sort
// (moe_aux.hip): the MT pairs share every weight byte the workgroup loads, so an expert that serves many pairs
// crosses HBM about once instead of once per pair.
//
// FUSEQ: `xsrc` is the raw activation matrix (dtype T, row pitch K) and every workgroup quantizes
// the vectors it needs straight into LDS, so a call is one launch and no workspace is touched;
// otherwise `xsrc` is the q8_1 workspace written by the stand-alone quantizer.
//
// The first weight loads of a chunk are issued before the activations are staged, and the loop
// keeps one step of loads in flight ahead of the dot products.
struct MoeVecArgs {
  const int32_t* topk_ids;    // [pairs] expert of every pair
  const int32_t* sorted_ids;  // routing sort in blocks of MT slots, or null for one pair per workgroup row
  const int32_t* expert_ids;  // [blocks]
  int top_k, pairs, act;
};

template <class F, int MT, int RPW, typename T, bool MOE, bool FUSEQ>
__global__ __launch_bounds__(256) void mmvq_kernel(const uint8_t* __restrict__ W, const char* __restrict__ xsrc,
                                                    T* __restrict__ Y, int N, int K, int kchunk, int64_t x_row_bytes,
                                                    int64_t y_vec_stride, MoeVecArgs moe, int64_t w_pitch, const T* __restrict__ bias) {
  extern __shared__ __align__(16) char smem[];
  __shared__ int s_xrow[MT], s_yrow[MT];  // activation row and output row of every staged vector (MOE)
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Kp = (int)q8_kp(K);
  const int act = moe.act;
  if (MOE) {
    int e;
    if (moe.sorted_ids == nullptr) {
      const int z = blockIdx.y;
      e = moe.topk_ids[z];
      if (tid < MT) { s_xrow[tid] = z / moe.top_k; s_yrow[tid] = tid == 0 ? z : -1; }
    } else {
      e = moe.expert_ids[blockIdx.y];
      if (e < 0) return;  // past the padded total
      if (tid < MT) {
        const int p = moe.sorted_ids[blockIdx.y * MT + tid];
        const bool ok = p < moe.pairs;
        s_xrow[tid] = ok ? p / moe.top_k : 0;
        s_yrow[tid] = ok ? p : -1;
      }
    }
    W += (int64_t)e * N * ((int64_t)(K / F::QK) * F::BS);
    __syncthreads();
  }
  int8_t* lq = (int8_t*)smem;                         // [MT][kchunk]
  float* ldv = (float*)(smem + MT * kchunk);          // [MT][kchunk/32]
  float* lav = ldv + MT * (kchunk / 32);              // [MT][kchunk/32]
  char* tab = (char*)(lav + (F::AUX != AUX_NONE ? MT * (kchunk / 32) : 0));
  F::init_tables(tab);
  if (F::TABLE_BYTES > 0) __syncthreads();

  const int row0 = (blockIdx.x * 4 + wave) * RPW;
  const int64_t rowbytes = w_pitch;   // bytes between rows: the dense row size unless the caller's tensor is padded
  const uint8_t* rows[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) rows[r] = W + (int64_t)min(row0 + r, N - 1) * rowbytes;

  float acc[RPW][MT];
#pragma unroll
  for (int r = 0; r < RPW; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;

  for (int k0 = 0; k0 < K; k0 += kchunk) {
    const int kc = min(kchunk, K - k0);
    const int nb = kc >> 5;
    const int u0 = k0 >> 5;  // first unit of this chunk within the row

    // weights of the first step: in flight while the activations are staged
    int u = lane;
    bool have = u < nb;
    typename F::Regs cur[RPW];
    if (have) {
#pragma unroll
      for (int r = 0; r < RPW; ++r) cur[r] = F::load(rows[r], u0, u, tab);
    }

    if (k0 > 0) __syncthreads();
    if (FUSEQ) {
      // four lanes quantize one 32-value block; kc/8 is a multiple of 4, so quads stay whole
      const int g8 = kc >> 3;
      for (int i = tid; i < MT * g8; i += 256) {
        const int m = i / g8, j = i - m * g8;
        float v[8];
        const T* xrow = (const T*)(xsrc + (int64_t)(MOE ? s_xrow[m] : m) * x_row_bytes);
        if (act == ACT_NONE) load8<T>(xrow + k0 + 8 * j, v);
        else load8_gated<T>(xrow + k0 + 8 * j, xrow + K + k0 + 8 * j, act, v);  // rows are [gate | up], K values each
        const Q8Quad qq = q8_1_quantize8(v);
        *(uint2*)(lq + m * kchunk + 8 * j) = qq.q;
        if ((j & 3) == 0) {
          ldv[m * (kchunk / 32) + (j >> 2)] = qq.d;
          if (F::AUX == AUX_S8) lav[m * (kchunk / 32) + (j >> 2)] = qq.s;
          if (F::AUX == AUX_DU) lav[m * (kchunk / 32) + (j >> 2)] = qq.du;
        }
      }
    } else {
      // copy quants (16-byte granules) and block scales of the MT vectors from the workspace
      const int g16 = kc >> 4;
      for (int i = tid; i < MT * g16; i += 256) {
        const int m = i / g16, j = i - m * g16;
        *(uint4*)(lq + m * kchunk + 16 * j) = *(const uint4*)(xsrc + (int64_t)(MOE ? s_xrow[m] : m) * x_row_bytes + k0 + 16 * j);
      }
      for (int i = tid; i < MT * nb; i += 256) {
        const int m = i / nb, j = i - m * nb;
        const float* fd = (const float*)(xsrc + (int64_t)(MOE ? s_xrow[m] : m) * x_row_bytes + Kp) + u0 + j;
        ldv[m * (kchunk / 32) + j] = fd[0];
        if (F::AUX == AUX_S8) lav[m * (kchunk / 32) + j] = fd[Kp / 32];
        if (F::AUX == AUX_DU) lav[m * (kchunk / 32) + j] = fd[2 * (Kp / 32)];
      }
    }
    __syncthreads();

    while (have) {
      const int un = u + 64;
      const bool hn = un < nb;
      typename F::Regs nxt[RPW];
      if (hn) {
#pragma unroll
        for (int r = 0; r < RPW; ++r) nxt[r] = F::load(rows[r], u0, un, tab);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        Act x;
        x.q = lq + m * kchunk;
        x.d = ldv + m * (kchunk / 32);
        x.a = lav + m * (kchunk / 32);
        x.tab = tab;
#pragma unroll
        for (int r = 0; r < RPW; ++r) acc[r][m] += F::dot(cur[r], x, u, lane);
      }
#pragma unroll
      for (int r = 0; r < RPW; ++r) cur[r] = nxt[r];
      u = un;
      have = hn;
    }
  }

#pragma unroll
  for (int r = 0; r < RPW; ++r) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float v = wave_sum(acc[r][m]);
      const int yrow = MOE ? s_yrow[m] : m;
      if (lane == 0 && row0 + r < N && yrow >= 0) Y[(int64_t)yrow * y_vec_stride + row0 + r] = finish<T>(v, bias, row0 + r);
    }
  }
}

// ------------------------------------------------------------------ streaming kernel (M <= 8)
// The decode case is one pass over a few tens of MB, i.e. a handful of HBM latencies long, so the
// whole game is to keep a steady, bounded stream of weight requests going from the first microsecond
// and to have nothing else on the critical path.
//   * One fat workgroup (NW waves) per CU owns a contiguous band of rows.  A row of K/32 units needs
//     S = ceil(K/2048) waves; the workgroup runs NW/S rows side by side ("slots"), and a lane keeps
//     the same unit column for its whole life.
//   * Every wave first requests the activation values it will quantize, then the weights of its first
//     D rows, and only then does arithmetic: the workgroup quantizes the MT activation vectors into LDS
//     (q8_1_device.h) once, while the weights fly.  A call is a single launch, no workspace traffic.
//   * After one barrier each lane pulls the quantized activations of its column into registers, so the
//     row loop touches no LDS except for one partial sum per (row, wave), and refills the load slot it
//     has just consumed: D row-loads stay in flight per wave.
//   * Row totals are summed from the per-wave partials in a fixed order.
constexpr int MMVQ_NW = 16;            // waves per workgroup of the streaming kernel
// D = 2: measured against 1, 3, 4, 5 and "every row at once" on 33 MB matrices, two row-loads in flight per wave
// (32 per CU and lane column) give the highest rate; deeper pipelines lose bandwidth, they do not gain latency cover.
constexpr int MMVQ_DEPTH = 2;

// MT per-lane values -> the sum over this lane's row of 16 lanes of value number (lane mod MT), in every lane.
// Exchange step k pairs lanes 2^k apart: a lane keeps the half of its values whose class bit k equals its own lane
// bit and adds the partner's copy of the same values.  The order of additions is fixed by the lane numbers.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int MT>
__device__ __forceinline__ float rows16_sums(const float (&a)[MT], int lane) {
  constexpr int XOR1 = 0xB1, XOR2 = 0x4E, ROR4 = 0x124, ROR8 = 0x128, ROR12 = 0x12C;
  float v;
  if constexpr (MT == 1) {
    v = a[0];
    v += dpp_f<XOR1>(v);
    v += dpp_f<XOR2>(v);
    v += dpp_f<ROR4>(v);
  } else {
    const bool b0 = lane & 1;
    float k[MT / 2];
#pragma unroll
    for (int p = 0; p < MT / 2; ++p) {          // classes 2p and 2p+1
      const float keep = b0 ? a[2 * p + 1] : a[2 * p], give = b0 ? a[2 * p] : a[2 * p + 1];
      k[p] = keep + dpp_f<XOR1>(give);
    }
    if constexpr (MT == 2) {
      v = k[0] + dpp_f<XOR2>(k[0]);
      v += dpp_f<ROR4>(v);
    } else {
      const bool b1 = lane & 2;
      float q[MT / 4];
#pragma unroll
      for (int p = 0; p < MT / 4; ++p) {        // classes 4p + (lane & 1) and 4p + 2 + (lane & 1)
        const float keep = b1 ? k[2 * p + 1] : k[2 * p], give = b1 ? k[2 * p] : k[2 * p + 1];
        q[p] = keep + dpp_f<XOR2>(give);
      }
      if constexpr (MT == 4) {
        v = q[0] + dpp_f<ROR4>(q[0]);
      } else {
        static_assert(MT == 8, "tiles of 1, 2, 4 or 8 rows");
        const bool b2 = lane & 4;
        const float keep = b2 ? q[1] : q[0], give = b2 ? q[0] : q[1];
        // the partner four lanes away: below for lanes with bit 2 set, above for the others
        const float down = dpp_f<ROR4>(give), up = dpp_f<ROR12>(give);
        v = keep + (b2 ? down : up);
      }
    }
  }
  v += dpp_f<ROR8>(v);
  return v;
}

// The reference's GEMV and its tile GEMM (ggml_mul_mat_a8) differ in three formats, and only in which per-block sum
// of the activations meets the offset: Q4_K / Q5_K multiply their mins by d8*sum(q) in the GEMV (vecdotq.cuh:328-351,
// 384-441) and by the stored sum of the unquantized values in the tiles (:369-372, :1325-1415); Q5_0 subtracts
// 16 * (stored sum) in the GEMV (:98-125) while its tiles use signed codes, i.e. 16 * d8*sum(q) (:668-749).  With
// TILE set the streaming kernel keeps the other plane of the quantizer's output for these formats, which turns it
// into the tile GEMM for a handful of rows of X.
template <class F> struct TileSums { static constexpr bool swaps = false; };
template <> struct TileSums<FmtQ5_0> { static constexpr bool swaps = true; };
template <> struct TileSums<FmtQ4_K> { static constexpr bool swaps = true; };
template <> struct TileSums<FmtQ5_K> { static constexpr bool swaps = true; };

// Profiling builds (the probe library only) record when the first and the last wave of every workgroup pass eight
// points of the kernel, on the 100 MHz wall clock that all CUs share.
#ifdef GGUF_TRACE_PHASES
__device__ unsigned long long g_mmvq_phases[1024 * 2 * 8];
#define GGUF_PHASE(i)                                                                                 \
  do {                                                                                                \
    if ((tid & 63) == 0 && (wave == 0 || wave == NW - 1) && blockIdx.x < 1024)                        \
      g_mmvq_phases[(blockIdx.x * 2 + (wave ? 1 : 0)) * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); \
  } while (0)
#else
#define GGUF_PHASE(i) do {} while (0)
#endif

// Formats whose 64-unit stretch of a row is a whole number of blocks (F::SPAN contiguous bytes) can be fetched by the
// streaming kernel as plain 16-byte pieces, lane after lane, every byte requested once, and handed to the lanes
// through LDS.  Requests that never meet a second request for the same cache line can carry the non-temporal hint,
// which the memory system rewards (a plain streaming read of 33 MB: 6.7 us with the hint, 7.3 us without).
#ifndef MMVQ_STAGED_MT
#define MMVQ_STAGED_MT 2   // rows of X up to which rows of W are fetched this way (at four the gain is gone)
#endif
template <class F, class = void> struct SpanOf { static constexpr int value = 0; };
template <class F> struct SpanOf<F, std::void_t<decltype(F::SPAN)>> { static constexpr int value = F::SPAN; };
// STAGED: rows are fetched per lane (0) or as whole 16-byte pieces: from aligned stretches of rows that are whole
// stretches (K a multiple of 2048: nothing to clamp), from stretches that start at any even address, or from aligned
// stretches of rows whose last stretch is shorter
constexpr int STAGED_ALIGNED = 1, STAGED_ANY = 2, STAGED_PART = 3;
// A fourth way to run the kernel, with per-lane loads: rows are handed out to half-waves of 32 lanes.  A row of 160
// units (K = 5120) takes five half-waves instead of three waves, so six rows instead of five run side by side and no
// lane is without a unit (of sixteen waves five were half empty and one had no row); K = 1024 fills a wave with two rows.
constexpr int LANES_HALF = 4;
// A fifth: whole aligned stretches as under STAGED_ALIGNED, but requested with loads that write LDS directly, into a
// ring of D stretches per wave: no registers hold the rows in flight and no store carries them to LDS.  What it
// does not buy is depth: a wave's whole share requested at once (its 7 or 8 rows fit LDS for the [14336,4096] and
// [4096,14336] matrices) ran 16 % slower, because requests beyond what the CU's memory pipeline accepts block the wave
// that issues them, and the activations, which every wave needs first, were quantized 3 us later.
constexpr int STAGED_DMA = 5;
#ifndef MMVQ_DMA_MT
#define MMVQ_DMA_MT 4   // rows of X up to which the ring serves
#endif
#ifndef MMVQ_DMA_DEPTH
#define MMVQ_DMA_DEPTH 2   // (3 and 4 stretches in flight per wave, and a wave's whole share at once, measured slower: requests
#endif                     //  beyond what the CU's memory pipeline holds block the waves that issue them)
template <class F, class = void> struct SpanAny { static constexpr bool value = false; };   // spans may start at any even address
template <class F> struct SpanAny<F, std::void_t<decltype(F::SPAN_ANY)>> { static constexpr bool value = F::SPAN_ANY; };
template <class F, class = void> struct SpanSlack { static constexpr int value = 0; };   // bytes a reader may touch behind the last span
template <class F> struct SpanSlack<F, std::void_t<decltype(F::SPAN_SLACK)>> { static constexpr int value = F::SPAN_SLACK; };
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
// Orders this wave's LDS accesses before the call against those after it, for data that lanes hand to each other
// through LDS without a workgroup barrier (the hardware keeps one wave's LDS accesses in order).
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
template <int SPAN, bool ANY = false> struct SpanRegs {
  static_assert(SPAN % 16 == 0 && SPAN > 0, "whole 16-byte pieces");
  // ANY: the span starts anywhere inside its first piece, so it may reach into one piece more
  static constexpr int PIECES = SPAN / 16 + (ANY ? 1 : 0), NR = (PIECES + 63) / 64, TAIL = PIECES - 64 * (NR - 1);
  u32x4_t r[NR];   // pieces lane, 64 + lane, ...; the last set has TAIL pieces (idle lanes repeat one of them)
  // `first` is the 16-byte boundary at or below the span; `valid` pieces from there hold bytes of the row (the last
  // stretch of a row may be shorter): later ones repeat the last
  __device__ __forceinline__ void load(const uint8_t* first, int lane, int valid) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int p = 64 * i + ((i < NR - 1 || TAIL == 64) ? lane : lane % TAIL);
      r[i] = __builtin_nontemporal_load((const u32x4_t*)(first + 16 * min(p, valid - 1)));
    }
  }
  __device__ __forceinline__ void load(const uint8_t* first, int lane) {   // a whole stretch
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int p = 64 * i + ((i < NR - 1 || TAIL == 64) ? lane : lane % TAIL);
      r[i] = __builtin_nontemporal_load((const u32x4_t*)(first + 16 * p));
    }
  }
  __device__ __forceinline__ void store(char* lds, int lane) const {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (i < NR - 1 || TAIL == 64 || lane < TAIL) *(u32x4_t*)(lds + 1024 * i + 16 * lane) = r[i];
  }
};

// Waits until at most N of this wave's vector-memory loads are outstanding; a compiler barrier for memory as well, so
// that reads of LDS filled by such loads stay behind it.
__device__ __forceinline__ void wait_vm_upto(int n) {   // n must fold to a constant (it is the instruction's immediate)
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(n) : "memory");
}

// What the streaming kernel needs before its first memory requests, worked out on the host so that the kernel starts
// without a division, and packed so that all of its arguments fit the first 64 bytes of the argument block (one
// fetch).  The quotients by S and by K/8 are taken by multiplication with a rounded-up reciprocal, exact for the small
// numerators here: wave < 16 with S <= 16 (half-wave < 32 with S <= 32), and group index * K/8 < 2^32 because
// K <= 32768 for this kernel.
struct StreamGeom {
  uint32_t w_pitch;       // bytes between rows of W
  int N, K, rows_per_wg;
  uint32_t packed;        // m_act | S << 4 | slots << 10 | (4096 / S + 1) << 16
  uint32_t g8_inv;        // 2^32 / (K / 8) + 1
  __device__ __forceinline__ int m_act() const { return packed & 15; }
  __device__ __forceinline__ int S() const { return (packed >> 4) & 63; }          // waves (half-waves) per row
  __device__ __forceinline__ int slots() const { return (packed >> 10) & 63; }     // rows side by side (>= 1)
  __device__ __forceinline__ int slot_of(int w) const { return (int)(((unsigned)w * (packed >> 16)) >> 12); }  // w / S for w < 32
};
// `half`: rows are handed out to half-waves of 32 lanes instead of waves (LANES_HALF)
static inline StreamGeom stream_geom(int N, int K, int rows_per_wg, int64_t w_pitch, int m_act, int nw, bool half = false) {
  StreamGeom g;
  const int per = half ? 32 : 64;
  const int S = (K / 32 + per - 1) / per;
  g.w_pitch = (uint32_t)w_pitch;
  g.N = N;
  g.K = K;
  g.rows_per_wg = rows_per_wg;
  g.packed = (uint32_t)m_act | (uint32_t)S << 4 | (uint32_t)((half ? 2 * nw : nw) / S) << 10 | (4096u / (uint32_t)S + 1u) << 16;
  g.g8_inv = (uint32_t)((1ull << 32) / (uint32_t)(K / 8)) + 1u;
  return g;
}

// GATED (one activation row only): the row of X is [gate | up], K values each, and what is quantized is
// T(T(act(gate)) * up), the values a separate act-and-multiply kernel would have stored (fused_moe.py:44-51,80).
template <class F, int MT, int NW, int D, typename T, bool TILE, bool FULL, int STAGED, bool GATED>
__device__ __forceinline__ void mmvq_stream_body(const uint8_t* __restrict__ W, const T* __restrict__ X, T* __restrict__ Y,
                                                 const T* __restrict__ bias, int64_t ldy, const StreamGeom& geom, int act_fn) {
  static_assert(!GATED || MT == 1, "the gated variant quantizes one row");
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: row arithmetic stays on the scalar unit
  const int N = geom.N, K = geom.K, rows_per_wg = geom.rows_per_wg, m_act = geom.m_act();
  GGUF_PHASE(0);                               // entry
  const int nb = K >> 5;                       // 32-weight units per row
  const int S = geom.S();                      // waves per row
  const int slots = geom.slots();              // rows in flight side by side (>= 1, checked by the host)
  int8_t* lq = (int8_t*)smem;                  // [MT][K]
  float* ldv = (float*)(smem + (size_t)MT * K);  // [MT][nb]
  float* lav = ldv + MT * nb;                  // [MT][nb]
  char* tab = (char*)(lav + (F::AUX != AUX_NONE ? MT * nb : 0));
  float* part = (float*)(tab + F::TABLE_BYTES);  // [rows_per_wg][S][4 (HALF: 2) groups of 16 lanes][MT]
  constexpr bool HALF = STAGED == LANES_HALF, SPANS = STAGED != 0 && !HALF, DMA = STAGED == STAGED_DMA;
  constexpr int SPAN = SPANS ? SpanOf<F>::value : 0;

  const int r_begin = blockIdx.x * rows_per_wg;   // (the host launches ceil(N / rows_per_wg) workgroups: r_begin < N)
  const int r_end = min(N, r_begin + rows_per_wg);
  const int nrows = r_end - r_begin;
  if (nrows > 0) GGUF_PHASE(5);                // kernel arguments have arrived
  const int64_t rowbytes = geom.w_pitch;   // bytes between rows: the dense row size unless the caller's tensor is padded

  // this wave: slot (which of the side-by-side rows) and step (which 64-unit stretch of the row)
  // (HALF: the same per half-wave, so these are per-lane values there)
  const int wh = HALF ? 2 * wave + (lane >> 5) : wave;
  const int slot = geom.slot_of(wh), step = wh - slot * S;   // wh / S, wh % S
  const bool wave_on = slot < slots;           // NW - slots*S waves have no weights to fetch; they still quantize
  const int u_raw = HALF ? step * 32 + (lane & 31) : step * 64 + lane;
  constexpr int GW = HALF ? 2 : 4;             // 16-lane groups of a wave (half-wave): each leaves one partial sum per row
  const int G = GW * S;                        // partial sums per row
  const bool lane_on = wave_on && u_raw < nb;
  const int u = min(u_raw, nb - 1);

  if (F::TABLE_BYTES > 0) {
    F::init_tables(tab);
    __syncthreads();
  }

  // Loads are issued unconditionally (row index clamped into the band) so that every iteration issues the
  // same number of loads and the hardware load counter can be waited on exactly, slot by slot.
  const uint8_t* wbase = W + (int64_t)r_begin * rowbytes;
  // bytes of this wave's stretch that lie inside the row
  constexpr bool ANY = STAGED == STAGED_ANY;
  const int span_bytes = STAGED == STAGED_ALIGNED || DMA ? SPAN : SPANS ? max(16, min(SPAN, (K / F::QK) * F::BS - (wave_on ? step : 0) * SPAN)) : 0;
  typedef SpanRegs<SPANS ? SPAN : 16, ANY> Span;
  [[maybe_unused]] uint32_t mis[D];   // ANY: where in its first 16-byte piece the stretch of each row in flight starts
  auto load_row = [&](int i, [[maybe_unused]] uint32_t& m16) {
    const int row = min(slot + slots * i, nrows - 1);
    if constexpr (SPANS) {   // (the host takes this variant only for rows it can fetch as whole 16-byte pieces)
      Span r;
      const uint8_t* a = wbase + (int64_t)row * rowbytes + (int64_t)(wave_on ? step : 0) * SPAN;
      if constexpr (ANY) {
        m16 = (uint32_t)(uintptr_t)a & 15u;
        r.load(a - m16, lane, (int)(m16 + span_bytes + 15) >> 4);
      } else if constexpr (STAGED == STAGED_PART) {
        r.load(a, lane, span_bytes >> 4);
      } else {
        r.load(a, lane);
      }
      return r;
    } else {
      return F::load(wbase + (int64_t)row * rowbytes, 0, u, tab);
    }
  };
  // this wave's staging area for one span (DMA: a ring of D), behind the partial sums
  constexpr int STAGE_BYTES = SPANS ? 16 * Span::PIECES : 0;
  char* stage = (char*)(part + (size_t)rows_per_wg * G * MT) + wave * (DMA ? D * 1024 * Span::NR : STAGE_BYTES);
  // DMA: row i of this wave's share -> ring slot r, 16 bytes per lane and instruction straight into LDS (the LDS address is
  // the instruction's base plus 16 x lane).  Span::NR instructions per row with every lane at work -- lanes past the last
  // piece fetch it once more, into the padding of the slot, which is a whole number of KB -- so that no branch surrounds
  // a load: the kernel counts the loads in flight itself (see the waits), and code the compiler moves or copies around
  // a branch would not match the count.
  constexpr int DMA_SLOT = 1024 * Span::NR, DMA_INSTRS = DMA ? D * Span::NR : 0;   // (the loads of the first D rows)
  [[maybe_unused]] auto dma_row = [&](int i, int r) {
    if constexpr (DMA) {
      typedef const __attribute__((address_space(1))) void* gptr_t;
      typedef __attribute__((address_space(3))) void* lptr_t;
      const int row = min(slot + slots * i, nrows - 1);
      const uint8_t* a = wbase + (int64_t)row * rowbytes + (int64_t)step * SPAN;
      char* dst = stage + r * DMA_SLOT;
#pragma unroll
      for (int j = 0; j < Span::NR; ++j)
        __builtin_amdgcn_global_load_lds((gptr_t)(a + 16 * min(64 * j + lane, Span::PIECES - 1)), (lptr_t)(dst + 1024 * j), 16, 0, 2);
    }
  };
  // Prologue, in one basic block per variant: request this thread's first QG groups of activation values,
  // then the weights of the first D rows, then quantize the activations into LDS (four lanes per 32-value
  // block) while the weights fly.  The activation loads go first so that waiting for them does not also
  // wait for the weight loads behind them.  Groups past the end are clamped and their stores predicated.
  constexpr int NT = 64 * NW;
  const int g8 = K >> 3;
  // FULL: all MT rows of the tile exist (m_act == MT), known at compile time.  Otherwise rows m_act .. MT-1 are
  // computed on whatever the LDS holds and never stored.
  const int rows_x = FULL ? MT : m_act;
  const int qtotal = rows_x * g8;  // a multiple of 4, so quads stay whole
  std::conditional_t<DMA, int, std::conditional_t<SPANS, Span, typename F::Regs>> pre[DMA ? 1 : D];
  // the first D rows of this wave's share: D load slots in registers, or (DMA) all of the share; a fixed number of loads,
  // rows past the share clamped, so that the loads behind the activation requests can be counted
  auto first_rows = [&](auto on_tag) {
    if constexpr (DMA) {
      if constexpr (decltype(on_tag)::value) {
#pragma unroll
        for (int d = 0; d < D; ++d) dma_row(d, d);
      }
    } else {
#pragma unroll
      for (int d = 0; d < D; ++d) pre[d] = load_row(d, mis[d]);
    }
  };
  const auto row_of_group = [&](int qc) { return MT == 1 ? 0 : (int)__umulhi((unsigned)qc, geom.g8_inv); };  // qc / g8
  auto quantize_group = [&](const raw8<T>& raw, const raw8<T>& up, int q) {
    const int qc = min(q, qtotal - 1);
    const int m = row_of_group(qc), j = qc - m * g8;
    float xv[8];
    raw.cvt(xv);
    if constexpr (GATED) {
      float uv[8];
      up.cvt(uv);
      gate8<T>(xv, uv, act_fn);
    }
    const Q8Quad qq = q8_1_quantize8(xv);
    if (q < qtotal) {
      *(uint2*)(lq + (size_t)m * K + 8 * j) = qq.q;
      if ((j & 3) == 0) {
        ldv[m * nb + (j >> 2)] = qq.d;
        constexpr bool SWAP = TILE && TileSums<F>::swaps;
        if (F::AUX == AUX_S8) lav[m * nb + (j >> 2)] = SWAP ? qq.du : qq.s;
        if (F::AUX == AUX_DU) lav[m * nb + (j >> 2)] = SWAP ? qq.s : qq.du;
      }
    }
  };
  // Where one request per thread covers the activations, the waves hold their weight requests back until all of those
  // are out (the reason stands at the barrier below).  With a single activation vector and weights fetched straight
  // into LDS, letting the weight requests go at once measured 1-4 % faster for every format of 100 bytes or more per
  // 256 weights and 1-3 % slower for Q2_K's 84; with two or more vectors the barrier measured up to 2 % faster.
  constexpr bool PRE_BARRIER = !(DMA && MT == 1 && F::BS * 256 >= 100 * F::QK);
  auto prologue = [&](auto qg_tag, auto on_tag) {
    constexpr int QG = decltype(qg_tag)::value;
    if constexpr (QG == 0) {   // a wave with no activation values to quantize: its weights only
      if (PRE_BARRIER && qtotal <= NT) __builtin_amdgcn_s_barrier();   // (see below: the others' activation requests go first)
      GGUF_PHASE(6);
      first_rows(on_tag);
      __builtin_amdgcn_sched_barrier(0);
      GGUF_PHASE(7);
      return;
    }
    raw8<T> xraw[QG > 0 ? QG : 1], xup[GATED && QG > 0 ? QG : 1];
#pragma unroll
    for (int g = 0; g < QG; ++g) {
      const int qc = min(tid + g * NT, qtotal - 1);
      const int m = row_of_group(qc), j = qc - m * g8;
      if constexpr (DMA) {   // (not counted by the compiler: see the wait below)
        xraw[g].load_uncounted(X + (int64_t)m * K + 8 * j);
        if constexpr (GATED) xup[g].load_uncounted(X + K + 8 * j);
      } else {
        xraw[g].load(X + (int64_t)m * K + 8 * j);
        if constexpr (GATED) xup[g].load(X + K + 8 * j);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (QG == 1 && PRE_BARRIER) {
      // One request per thread covers the activations: hold every wave's weight requests back until all of those
      // are out.  The memory pipeline serves a CU's requests in order, and a late wave's activation request would
      // otherwise wait behind the weight requests of the waves that started before it, and the barrier below with it.
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    }
    GGUF_PHASE(6);                             // activation requests are out (every wave's, where one request covers them)
    first_rows(on_tag);
    __builtin_amdgcn_sched_barrier(0);
    GGUF_PHASE(7);                             // weight requests of the first rows are out
#pragma unroll
    for (int g = 0; g < QG; ++g) {   // (keeps the conversions below from moving above the weight requests)
      if constexpr (DMA) {
        // The compiler orders loads that write LDS like flat accesses and would wait for every load in flight, the
        // weights included, before the first use of an activation value.  The activation loads are older than the
        // weight loads and loads return in order: they have landed when no more than the weight loads are outstanding.
        constexpr int BEHIND = decltype(on_tag)::value ? DMA_INSTRS : 0;
        xraw[g].template landed<BEHIND>();
        if constexpr (GATED) xup[g].template landed<BEHIND>();
      } else {
        xraw[g].hold();
        if constexpr (GATED) xup[g].hold();
      }
    }
#pragma unroll
    for (int g = 0; g < QG; ++g) quantize_group(xraw[g], xup[GATED ? g : 0], tid + g * NT);
  };
  // (wave-uniform: a wave whose first lane is past the last group takes no part in the quantisation and reaches the
  // barrier as soon as its weight requests are out, instead of after a load and a quantisation nobody uses)
  auto prologue_for = [&](auto on_tag) {
    if (wave * 64 >= qtotal) prologue(std::integral_constant<int, 0>{}, on_tag);
    else if (qtotal <= NT) prologue(std::integral_constant<int, 1>{}, on_tag);
    else if (qtotal <= 2 * NT) prologue(std::integral_constant<int, 2>{}, on_tag);
    else prologue(std::integral_constant<int, 4>{}, on_tag);
  };
  // (DMA: a wave without a slot asks for no weights; its prologue is a copy of its own, so that the one with the
  //  requests has them outside any branch and the wait for the activations can count them)
  if (DMA && !wave_on) prologue_for(std::false_type{});
  else prologue_for(std::true_type{});
  for (int q = tid + 4 * NT; q - tid < qtotal; q += NT) {  // uniform trip count; only for K * MT > 32 * NT
    const int qc = min(q, qtotal - 1);
    const int m2 = row_of_group(qc), j2 = qc - m2 * g8;
    raw8<T> r, ru;
    r.load(X + (int64_t)m2 * K + 8 * j2);
    if constexpr (GATED) ru.load(X + K + 8 * j2);
    quantize_group(r, GATED ? ru : r, q);
  }
  GGUF_PHASE(1);                               // own share of the activations quantized
  __syncthreads();
  GGUF_PHASE(2);                               // every wave's share is in LDS
  // (the two quotients below are the kernel's only divisions; here they run while the first weights are still on their way)
  const int my_rows = wave_on && nrows > slot ? (nrows - slot + slots - 1) / slots : 0;  // rows slot, slot+slots, ...
  const int max_rows = (nrows + slots - 1) / slots;  // trip count of the row loop, same for every wave

  // this lane's column of every activation vector, held in registers for the whole row loop
  typename F::ActRegs act[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    Act x;
    x.q = lq + (size_t)m * K;
    x.d = ldv + m * nb;
    x.a = lav + m * nb;
    x.tab = tab;
    act[m] = F::load_act(x, u);
  }

  // (a wave without a slot -- NW is not always a multiple of the waves a row takes -- has quantized its share of the
  //  activations and waits at the barrier behind the loop)
  // one row's dot products -> its partial sums in LDS
  auto finish_row = [&](const typename F::Regs& cur, int i, bool row_ok) {
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float v = F::dot(cur, act[m], u);
      acc[m] = lane_on ? v : 0.0f;
    }
    const float v = rows16_sums<MT>(acc, lane);
    if ((lane & 15) < MT && row_ok) part[((slot + slots * i) * G + step * GW + ((lane >> 4) & (GW - 1))) * MT + (lane & 15)] = v;
  };
  if constexpr (DMA) {
    // Loads return in order: row i has landed once no more loads are outstanding than those of the rows requested
    // behind it, `ahead` of them (the counter's operand is an immediate: one case per count).
    constexpr int NRI = Span::NR;
    int r = 0;
    for (int i = 0; wave_on && i < max_rows; ++i) {
      const int ahead = min(D - 1, max_rows - 1 - i);
      if (ahead >= D - 1) wait_vm_upto((D - 1) * NRI);
      else if (D > 2 && ahead == D - 2) wait_vm_upto((D > 2 ? D - 2 : 0) * NRI);
      else if (D > 3 && ahead == D - 3) wait_vm_upto((D > 3 ? D - 3 : 0) * NRI);
      else wait_vm_upto(0);
      const typename F::Regs cur = F::from_span(stage + r * DMA_SLOT, lane);
      if (i + D < max_rows) {
        // the slot is asked for again only after this lane's reads of it have returned
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        dma_row(i + D, r);
      }
      finish_row(cur, i, i < my_rows);
      r = r + 1 == D ? 0 : r + 1;
    }
  }
  if constexpr (!DMA)
  for (int i0 = 0; (HALF || wave_on) && i0 < max_rows; i0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int i = i0 + d;
      const bool row_ok = i < my_rows;
      float acc[MT];
      typename F::Regs cur;
      if constexpr (SPANS) {
        // through LDS to the lanes that use the bytes (one wave's LDS accesses keep their order: no barrier), and the
        // slot is free for the next request before the arithmetic starts
        // (The fences are for the compiler, which reasons about one lane and would otherwise keep a value read from
        //  the previous row's copy where this lane's own stores cannot reach it, or move the next row's stores above
        //  these reads; they cost no instruction.)
        pre[d].store(stage, lane);
        wave_lds_fence();
        if constexpr (ANY) {
          const int at = (int)mis[d];
          pre[d] = load_row(i + D, mis[d]);
          cur = F::from_span(stage, lane, at);
        } else {
          pre[d] = load_row(i + D, mis[d]);
          cur = F::from_span(stage, lane);
        }
        wave_lds_fence();
      } else {
        cur = pre[d];
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const float v = F::dot(cur, act[m], u);
        acc[m] = lane_on ? v : 0.0f;
      }
      if constexpr (!SPANS) pre[d] = load_row(i + D, mis[d]);  // refill the slot: D - 1 other slots are still in flight
      // The MT sums over the wave are formed together: after log2(MT) exchange steps in which a lane keeps the value
      // of the class (lane mod MT) it belongs to and hands the other to its partner, one value per lane is left to
      // add up over lanes of equal class, instead of MT values over all lanes.  Rotations by 4 and 8 inside a row of 16
      // lanes finish that; the four rows of the wave leave their totals in LDS for the adder below.
      const float v = rows16_sums<MT>(acc, lane);
      if ((lane & 15) < MT && row_ok) part[((slot + slots * i) * G + step * GW + ((lane >> 4) & (GW - 1))) * MT + (lane & 15)] = v;
    }
  }
  GGUF_PHASE(3);                               // own rows walked
  __syncthreads();
  // The partial sums of a result meet in eight lanes: lane j of the eight adds partials j, j + 8, ... and three exchange
  // steps inside the group of eight add those up (a fixed order, like every sum here).  One lane per result walking
  // all G of them kept the first wave at work for 0.25 us behind the barrier at G = 8 and 0.45 us at G = 28, after
  // every other wave had left: Q4_K [4096,14336] 9.15 -> 8.93 us per launch; rows of one or two stretches are unchanged.
  for (int base = 0; base < nrows * MT; base += 8 * NW) {   // (uniform trip count: every lane takes part in the exchanges)
    const int i = base + (tid >> 3), j = tid & 7;
    const bool on = i < nrows * MT;
    const int row = on ? i / MT : 0, m = i - row * MT;
    float v = 0.0f;
    if (on)
      for (int st = j; st < G; st += 8) v += part[(row * G + st) * MT + m];
    v += dpp_mov<0xB1>(v);    // quad_perm [1,0,3,2]: lane ^ 1
    v += dpp_mov<0x4E>(v);    // quad_perm [2,3,0,1]: lane ^ 2
    v += dpp_mov<0x104>(v);   // row_shl 4: lane + 4 (the first lane of each eight gets the other quad's total)
    if (on && j == 0 && (FULL || m < m_act)) Y[(int64_t)m * ldy + r_begin + row] = finish<T>(v, bias, r_begin + row);
  }
  GGUF_PHASE(4);                               // results stored
}

template <class F, int MT, int NW, int D, typename T, bool TILE = false, bool FULL = true, int STAGED = 0>
__global__ __launch_bounds__(64 * NW) void mmvq_stream_kernel(const uint8_t* __restrict__ W, const T* __restrict__ X,
                                                               T* __restrict__ Y, const T* __restrict__ bias, int64_t ldy,
                                                               StreamGeom geom) {
  mmvq_stream_body<F, MT, NW, D, T, TILE, FULL, STAGED, false>(W, X, Y, bias, ldy, geom, ACT_NONE);
}

// The per-pair MoE operator on the same kernel (reference: csrc/gguf/moe_vec.cuh:3-53): blockIdx.y is the flat
// (token, k) pair z; its expert topk_ids[z] picks the weight matrix (experts densely packed), its token z / top_k the
// activation row, and the result is row z of Y.  A pair whose expert id is outside [0, num_experts) (when the caller
// says how many there are) names no weights and is left out.
struct MoeStreamArgs {
  const int32_t* topk_ids;
  int64_t expert_bytes;   // between the matrices of two experts
  int64_t x_pitch;        // elements between activation rows: K, or 2 K for [gate | up] rows
  int top_k, num_experts, act;
};
template <class F, int NW, int D, typename T, int STAGED, bool GATED>
__global__ __launch_bounds__(64 * NW) void mmvq_stream_moe_kernel(const uint8_t* __restrict__ W, const T* __restrict__ X,
                                                                   T* __restrict__ Y, MoeStreamArgs moe, StreamGeom geom) {
  const int z = blockIdx.y;
  const int e = moe.topk_ids[z];
  if (moe.num_experts > 0 && (e < 0 || e >= moe.num_experts)) return;
  mmvq_stream_body<F, 1, NW, D, T, false, true, STAGED, GATED>(W + (int64_t)e * moe.expert_bytes, X + (int64_t)(z / moe.top_k) * moe.x_pitch,
                                                               Y + (int64_t)z * geom.N, nullptr, (int64_t)geom.N, geom, moe.act);
}

// Whether the rows of W are whole 16-byte pieces at 16-byte aligned addresses.  Q3_K and Q6_K, whose rows are that only
// when K is a multiple of 2048, have a second variant for any even address and pitch: its pieces start at the 16-byte
// boundary below a stretch and the readers cut their fields out of the LDS copy from wherever it starts (nothing outside
// the 16-byte granules that hold bytes of W is read).
template <class F>
static bool span_aligned(const void* W, int64_t pitch, int K) {
  return (int64_t)(K / F::QK) * F::BS % 16 == 0 && pitch % 16 == 0 && (uintptr_t)W % 16 == 0;
}

// Formats whose aligned stretches the streaming kernel fetches straight into LDS (STAGED_DMA)
template <class F> struct DmaRing { static constexpr bool on = SpanOf<F>::value > 0; };

template <class F, int MT, int D, typename T, bool TILE, bool FULL, int NW, int STAGED = 0>
static void launch_stream_d(const void* W, const T* X, T* Y, int N, int K, int rows_per_wg, int grid, size_t lds, const LinearArgs& la,
                            hipStream_t stream, int m_act) {
  auto kern = mmvq_stream_kernel<F, MT, NW, D, T, TILE, FULL, STAGED>;
  if (lds > 64 * 1024) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, 160 * 1024, done);
  }
  const int64_t w_pitch = la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * NW), lds, stream, (const uint8_t*)W, X, Y, (const T*)la.bias,
                     la.ldy ? la.ldy : (int64_t)N, stream_geom(N, K, rows_per_wg, w_pitch, m_act, NW, STAGED == LANES_HALF));
}

// Returns false when the shape does not fit the streaming kernel (a row longer than NW waves, or activations
// that do not fit in LDS); the caller then takes the workspace path.
template <class F, int MT, typename T, bool TILE = false, int NW = MMVQ_NW>
static bool launch_stream(const void* W, const T* X, T* Y, int N, int K, hipStream_t stream, const LinearArgs& la, int m_act = MT) {
  // m_act <= MT rows of X are there; the kernel computes MT and stores m_act
  const int nb = K / 32, S = (nb + 63) / 64;
  if (S > NW) return false;
  if ((la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS) > (int64_t)UINT32_MAX) return false;   // (the kernel holds it in 32 bits)
  const int slots = NW / S;
  const int target = num_cus();
  int rows_per_wg = (N + target - 1) / target;
  if (rows_per_wg < slots) rows_per_wg = slots;  // at least one row per slot
  const int grid = (N + rows_per_wg - 1) / rows_per_wg;
  const size_t lds = (size_t)MT * K + (size_t)MT * nb * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES +
                     (size_t)rows_per_wg * S * 4 * MT * 4;
  if (lds > 160 * 1024) return false;
  const int per_wave = (rows_per_wg + slots - 1) / slots;  // rows each wave walks; the pipeline depth never exceeds it
  const auto go = [&](auto full) {
    constexpr bool FULL = decltype(full)::value;
    if constexpr (MT <= 4) {
      // (for Q4_K, whose per-lane loads are aligned 16-byte pieces already, the trip through LDS costs the 8-wave kernel
      //  of the small matrices as much as it gains; [4096,4096]: Q8_0 6.4 -> 5.1 us, Q4_0 5.1 -> 4.4 us, Q6_K 6.2 -> 5.4 us)
      // (Q8_0, most bytes per weight, still gains at four rows: [14336,4096] 16.6 -> 15.4 us)
      if constexpr (MT <= (std::is_same<F, FmtQ8_0>::value || DmaRing<F>::on ? 4 : MMVQ_STAGED_MT) && (NW == MMVQ_NW || !std::is_same<F, FmtQ4_K>::value || DmaRing<F>::on) && SpanOf<F>::value > 0) {
        // rows of whole 16-byte pieces at aligned addresses: every byte is requested once (see SpanRegs)
        const int64_t pitch = la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS;
        const size_t lds_staged = lds + (size_t)NW * 16 * SpanRegs<SpanOf<F>::value, SpanAny<F>::value>::PIECES + SpanSlack<F>::value;
        // (a row shorter than one stretch leaves half the lanes of its wave without a block: not worth the trip through LDS,
        //  Q8_0 [3072,1024] 3.3 -> 3.8 us)
        if (per_wave >= MMVQ_DEPTH && nb >= 64 && lds_staged <= 160 * 1024) {
          if constexpr (DmaRing<F>::on && MT <= MMVQ_DMA_MT) {
            // whole aligned stretches straight into a ring in LDS, as deep as the rows a wave walks where LDS has the room
            // (the activations must be quantized by the prologue's straight-line code: its loads are counted)
            const size_t slot = 1024 * SpanRegs<SpanOf<F>::value>::NR;
            const auto fits = [&](int d) { return per_wave >= d && lds + (size_t)NW * d * slot <= 160 * 1024; };
            // (rows of up to two stretches on the 16-wave kernel: Q4_K [14336,4096] 8.9 -> 8.5 us; longer rows and the 8-wave
            //  kernel of small matrices lose a little; with three and four rows of X, [14336,4096] 13.5 -> 13.0 us but
            //  [4096,4096] 7.1 -> 7.4 us, hence the floor on N)
            if (NW == MMVQ_NW && S <= 2 && nb % 64 == 0 && span_aligned<F>(W, pitch, K) && (size_t)MT * K <= 32 * 64 * NW &&
                (MT <= 2 || N >= 8192)) {
              if (fits(MMVQ_DMA_DEPTH)) { launch_stream_d<F, MT, MMVQ_DMA_DEPTH, T, TILE, FULL, NW, STAGED_DMA>(W, X, Y, N, K, rows_per_wg, grid, lds + (size_t)NW * MMVQ_DMA_DEPTH * slot, la, stream, m_act); return; }
            }
          }
          // (through registers the trip costs the 8-wave kernel of Q4_K as much as it gains: per-lane loads below)
          if constexpr ((NW == MMVQ_NW || !std::is_same<F, FmtQ4_K>::value) && MT <= (std::is_same<F, FmtQ8_0>::value ? 4 : MMVQ_STAGED_MT)) {
            if (span_aligned<F>(W, pitch, K)) {
              if (nb % 64 == 0) launch_stream_d<F, MT, MMVQ_DEPTH, T, TILE, FULL, NW, STAGED_ALIGNED>(W, X, Y, N, K, rows_per_wg, grid, lds_staged, la, stream, m_act);
              else launch_stream_d<F, MT, MMVQ_DEPTH, T, TILE, FULL, NW, SpanAny<F>::value ? STAGED_ANY : STAGED_PART>(W, X, Y, N, K, rows_per_wg, grid, lds_staged, la, stream, m_act);
              return;
            }
            if constexpr (SpanAny<F>::value) {
              if (pitch % 2 == 0 && (uintptr_t)W % 2 == 0) {
                launch_stream_d<F, MT, MMVQ_DEPTH, T, TILE, FULL, NW, STAGED_ANY>(W, X, Y, N, K, rows_per_wg, grid, lds_staged, la, stream, m_act);
                return;
              }
            }
          }
        }
      }
      if constexpr (MT == 1) {
        // rows handed out to half-waves where that puts more rows side by side (K = 5120: six instead of five)
        const int sh = (nb + 31) / 32, slots_h = sh <= 2 * NW ? 2 * NW / sh : 0;
        // (not where that would take more rows per workgroup and so fewer workgroups than the chip has CUs, and only
        //  where a half-wave then walks fewer rows than a wave did: 20 rows per workgroup are four turns either way)
        if (nb % 32 == 0 && slots_h > slots && rows_per_wg >= slots_h && (rows_per_wg + slots_h - 1) / slots_h < per_wave) {
          const int rows_h = rows_per_wg;
          const size_t lds_h = (size_t)K + (size_t)nb * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES + (size_t)rows_h * sh * 2 * 4;
          if ((rows_h + slots_h - 1) / slots_h >= MMVQ_DEPTH && lds_h <= 160 * 1024) {
            launch_stream_d<F, MT, MMVQ_DEPTH, T, TILE, FULL, NW, LANES_HALF>(W, X, Y, N, K, rows_h, (N + rows_h - 1) / rows_h, lds_h, la, stream, m_act);
            return;
          }
        }
      }
      if (per_wave >= MMVQ_DEPTH) { launch_stream_d<F, MT, MMVQ_DEPTH, T, TILE, FULL, NW>(W, X, Y, N, K, rows_per_wg, grid, lds, la, stream, m_act); return; }
    }
    // eight activation rows in registers leave room for one weight row in flight per wave
    launch_stream_d<F, MT, 1, T, TILE, FULL, NW>(W, X, Y, N, K, rows_per_wg, grid, lds, la, stream, m_act);
  };
  if constexpr (MT <= 2) go(std::true_type{});   // the callers of the 1- and 2-row tiles always fill them
  else if (m_act == MT) go(std::true_type{});
  else go(std::false_type{});
  return true;
}

// The per-pair MoE operator on the streaming kernel: about one workgroup per CU in all, each walking a band of one
// pair's expert matrix.  Returns false for shapes the streaming kernel does not take.
template <class F, typename T, bool GATED>
static bool launch_stream_moe(const void* W, const T* X, T* Y, int N, int K, const int32_t* topk_ids, int top_k, int pairs, int act,
                              int num_experts, hipStream_t stream) {
  constexpr int NW = MMVQ_NW;
  const int nb = K / 32, S = (nb + 63) / 64;
  if (S > NW || pairs > 65535) return false;
  const int64_t pitch = (int64_t)(K / F::QK) * F::BS;
  if (pitch > (int64_t)UINT32_MAX) return false;
  const int slots = NW / S;
  // Bands of rows per pair such that the workgroups (one per CU at a time) make whole rounds: N * pairs / CUs rows each
  // would give 3 bands x 96 pairs = 288 workgroups for 12 tokens top-8 of [2048,2048], a full round and an eighth.
  // Cost of a choice: rounds x (rows of a band + what a workgroup spends before its first row, about sixteen turns).
  const int64_t target = num_cus();
  int rows_per_wg = N;
  int64_t best = INT64_MAX;
  // (up to as many bands as put a workgroup on every CU: with one to three pairs, the batch-1 decode of a top-2 layer,
  //  64 bands a pair would leave most of the chip idle)
  const int max_bands = (int)(pairs > 0 && (target + pairs - 1) / pairs > 64 ? (target + pairs - 1) / pairs : 64);
  for (int b = 1; b <= max_bands; ++b) {
    const int rows = (N + b - 1) / b;
    if (rows < slots && b > 1) break;
    const int64_t wgs = (int64_t)((N + rows - 1) / rows) * pairs, rounds = (wgs + target - 1) / target;
    const int64_t cost = rounds * (rows + 16 * slots);
    if (cost < best) { best = cost; rows_per_wg = rows; }
  }
  if (rows_per_wg < slots) rows_per_wg = slots < N ? slots : N;
  const int grid = (N + rows_per_wg - 1) / rows_per_wg;
  const size_t lds = (size_t)K + (size_t)nb * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES + (size_t)rows_per_wg * S * 4 * 4;
  if (lds > 160 * 1024) return false;
  const int per_wave = (rows_per_wg + slots - 1) / slots;
  const MoeStreamArgs moe = {topk_ids, (int64_t)N * pitch, (int64_t)K * (GATED ? 2 : 1), top_k, num_experts, act};
  const StreamGeom geom = stream_geom(N, K, rows_per_wg, pitch, 1, NW);
  const auto go = [&](auto kern, size_t bytes) {
    if (bytes > 64 * 1024) {
      static std::atomic<uint64_t> done{0};   // (one per kernel: the lambda's body is instantiated per argument type)
      allow_large_lds(kern, 160 * 1024, done);
    }
    hipLaunchKernelGGL(kern, dim3(grid, pairs), dim3(64 * NW), bytes, stream, (const uint8_t*)W, X, Y, moe, geom);
  };
  // (experts shared between pairs come from the caches at more than the HBM rate, and there the trip through LDS costs
  //  more than the tidier requests gain: Q4_0, 64 experts [2048,2048], 8 tokens 45 -> 48 us; Q4_K keeps it)
  if constexpr (std::is_same<F, FmtQ4_K>::value) {
    const size_t lds_staged = lds + (size_t)NW * 16 * SpanRegs<SpanOf<F>::value, SpanAny<F>::value>::PIECES + SpanSlack<F>::value;
    if (per_wave >= MMVQ_DEPTH && nb % 64 == 0 && span_aligned<F>(W, pitch, K) && lds_staged <= 160 * 1024) {
      go(mmvq_stream_moe_kernel<F, NW, MMVQ_DEPTH, T, STAGED_ALIGNED, GATED>, lds_staged);
      return true;
    }
  }
  {
    // rows handed out to half-waves where that saves turns of the row loop (K = 1024, the second expert GEMM of a layer
    // with 1024 intermediate features: two rows per wave)
    const int sh = (nb + 31) / 32, slots_h = sh <= 2 * NW ? 2 * NW / sh : 0;
    if (nb % 32 == 0 && slots_h > slots && rows_per_wg >= slots_h && (rows_per_wg + slots_h - 1) / slots_h < per_wave &&
        (rows_per_wg + slots_h - 1) / slots_h >= MMVQ_DEPTH) {
      const size_t lds_h = (size_t)K + (size_t)nb * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES + (size_t)rows_per_wg * sh * 2 * 4;
      const StreamGeom geom_h = stream_geom(N, K, rows_per_wg, pitch, 1, NW, true);
      auto kern = mmvq_stream_moe_kernel<F, NW, MMVQ_DEPTH, T, LANES_HALF, GATED>;
      if (lds_h > 64 * 1024) {
        static std::atomic<uint64_t> done{0};
        allow_large_lds(kern, 160 * 1024, done);
      }
      hipLaunchKernelGGL(kern, dim3(grid, pairs), dim3(64 * NW), lds_h, stream, (const uint8_t*)W, X, Y, moe, geom_h);
      return true;
    }
  }
  if (per_wave >= MMVQ_DEPTH) go(mmvq_stream_moe_kernel<F, NW, MMVQ_DEPTH, T, 0, GATED>, lds);
  else go(mmvq_stream_moe_kernel<F, NW, 1, T, 0, GATED>, lds);
  return true;
}

constexpr int MMVQ_RPW = 2;     // rows per wave of the workspace kernel

static inline int kchunk_for(int mt, int K) {
  int kchunk = mt == 1 ? 32768 : mt == 2 ? 16384 : mt == 4 ? 8192 : 4096;
  const int kround = (K + 511) / 512 * 512;
  return kchunk > kround ? kround : kchunk;
}
template <class F, int MT>
static inline size_t mmvq_lds(int kchunk) {
  return (size_t)MT * kchunk + (size_t)MT * (kchunk / 32) * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES;
}

template <class F, int MT, typename T, bool FUSEQ>
static void launch_mt(const void* W, const char* xsrc, T* Y, int N, int K, hipStream_t stream, const LinearArgs& la) {
  constexpr int RPW = MMVQ_RPW;
  const int kchunk = kchunk_for(MT, K);
  const int grid = (N + 4 * RPW - 1) / (4 * RPW);
  const int64_t xrb = FUSEQ ? (int64_t)K * (int64_t)sizeof(T) : q8_row_bytes(K);
  const size_t lds = mmvq_lds<F, MT>(kchunk);
  hipLaunchKernelGGL((mmvq_kernel<F, MT, RPW, T, false, FUSEQ>), dim3(grid), dim3(256), lds, stream,
                     (const uint8_t*)W, xsrc, Y, N, K, kchunk, xrb, la.ldy ? la.ldy : (int64_t)N,
                     MoeVecArgs{nullptr, nullptr, nullptr, 1, 0, (int)ACT_NONE}, la.w_pitch ? la.w_pitch : (int64_t)(K / F::QK) * F::BS,
                     (const T*)la.bias);
}


// Rows of X the streaming kernel takes in one launch.  Eight rows of activation registers spill for the formats whose
// units carry the most scale data (measured on [14336,4096]: Q6_K 83 us at eight rows against 19 us at four, Q2_K 82
// against 20, Q3_K 73 against 20): those take four rows per pass.
template <class F> struct StreamRows { static constexpr int max = 8; };
template <> struct StreamRows<FmtQ2_K> { static constexpr int max = 4; };
template <> struct StreamRows<FmtQ3_K> { static constexpr int max = 4; };
template <> struct StreamRows<FmtQ6_K> { static constexpr int max = 4; };

template <class F, typename T>
static int mmvq_typed(const void* W, const void* x, void* ws, void* Y, int xdtype, int64_t N, int64_t K, int64_t M,
                      hipStream_t stream, const LinearArgs& la) {
  const int64_t ldy = la.ldy ? la.ldy : N;
  constexpr int MAXR = StreamRows<F>::max;
  if (la.tile_sums) {
    // the tile GEMM's arithmetic for a handful of rows; GGUF_NOT_TAKEN sends the caller back to its tile kernels
    if (M > MAXR) return GGUF_NOT_TAKEN;
    const T* xs = (const T*)x;
    bool ok = false;
    if constexpr (TileSums<F>::swaps) {
      if (M <= 4) ok = launch_stream<F, 4, T, true>(W, xs, (T*)Y, (int)N, (int)K, stream, la, (int)M);
      else if constexpr (MAXR == 8) ok = launch_stream<F, 8, T, true>(W, xs, (T*)Y, (int)N, (int)K, stream, la, (int)M);
    } else {  // the two operators agree on these formats: the GEMV's own kernels serve
      if (M == 1) ok = launch_stream<F, 1, T>(W, xs, (T*)Y, (int)N, (int)K, stream, la);
      else if (M == 2) ok = launch_stream<F, 2, T>(W, xs, (T*)Y, (int)N, (int)K, stream, la);
      else if (M <= 4) ok = launch_stream<F, 4, T>(W, xs, (T*)Y, (int)N, (int)K, stream, la, (int)M);
      else if constexpr (MAXR == 8) ok = launch_stream<F, 8, T>(W, xs, (T*)Y, (int)N, (int)K, stream, la, (int)M);
    }
    return ok ? launch_status() : GGUF_NOT_TAKEN;
  }
  {
    // Up to MAXR rows are one launch.  More rows than a tile holds go MAXR at a time through the same kernel: each pass
    // reads W again, as the workspace kernel below also does per eight rows, but at the streaming kernel's rate (Q4_K
    // [14336,4096] at 16 rows: 42 us against 76 us).  If the first pass does not fit the kernel none has been launched
    // and the workspace path runs.
    const T* xs = (const T*)x;
    bool ok = true;
    for (int64_t m0 = 0; m0 < M && ok; m0 += MAXR) {
      const int rows = (int)(M - m0 < MAXR ? M - m0 : MAXR);
      const T* xm = xs + m0 * K;
      T* ym = (T*)Y + m0 * ldy;
      // A small matrix (a row fits two waves, at most 16 rows per CU) is over in a few microseconds, much of it the
      // dispatch of the workgroups: half as many waves, each walking twice the rows, start and finish sooner.
      // (the 16-wave kernel with its LDS ring on [4096,4096]: 5.25 against 4.92 us)
      if (M == 1 && K <= 4096 && N <= 16 * num_cus()) ok = launch_stream<F, 1, T, false, 8>(W, xm, ym, (int)N, (int)K, stream, la);
      else if (rows == 1) ok = launch_stream<F, 1, T>(W, xm, ym, (int)N, (int)K, stream, la);
      else if (rows == 2) ok = launch_stream<F, 2, T>(W, xm, ym, (int)N, (int)K, stream, la);
      else if (rows <= 4) ok = launch_stream<F, 4, T>(W, xm, ym, (int)N, (int)K, stream, la, rows);
      else if constexpr (MAXR == 8) ok = launch_stream<F, 8, T>(W, xm, ym, (int)N, (int)K, stream, la, rows);
      if (!ok && m0 > 0) return GGUF_ERR_LAUNCH;   // cannot happen: a later pass needs no more than the first
    }
    if (ok) return launch_status();
  }
  const int rc = quantize_q8_1(x, xdtype, ws, M, K, stream);
  if (rc != GGUF_OK) return rc;
  const int64_t rb = q8_row_bytes(K);
  int64_t m0 = 0;
  while (m0 < M) {
    const int64_t left = M - m0;
    const char* wsm = (const char*)ws + m0 * rb;
    T* ym = (T*)Y + m0 * ldy;
    if (left >= 8) { launch_mt<F, 8, T, false>(W, wsm, ym, (int)N, (int)K, stream, la); m0 += 8; }
    else if (left >= 4) { launch_mt<F, 4, T, false>(W, wsm, ym, (int)N, (int)K, stream, la); m0 += 4; }
    else if (left >= 2) { launch_mt<F, 2, T, false>(W, wsm, ym, (int)N, (int)K, stream, la); m0 += 2; }
    else { launch_mt<F, 1, T, false>(W, wsm, ym, (int)N, (int)K, stream, la); m0 += 1; }
  }
  return launch_status();
}

extern "C" int gguf_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int64_t num_experts, int64_t block,
                                         int32_t* sorted_token_ids, int64_t sorted_capacity, int32_t* expert_ids,
                                         int64_t expert_capacity, int32_t* num_tokens_post_padded, gguf_stream_t stream);

constexpr int MOE_VEC_GROUP_RPW = 2;
constexpr int MOE_VEC_GROUP = 4;  // pairs of one expert that share a pass over its weights

// With the expert count known and a workspace large enough for the quantized activations plus the routing sort
// (q8 rows first, then the three sort arrays), pairs are grouped by expert: the activations are quantized once by the
// stand-alone kernel instead of once per workgroup, and MOE_VEC_GROUP pairs share each pass over an expert's rows.
// Otherwise every pair gets its own workgroup row and quantizes its token itself (one launch, no workspace).
template <class F, typename T>
static int moe_vec_typed(const void* W, const char* x, void* Y, int xdtype, int N, int K, const int32_t* topk_ids, int top_k,
                         int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t stream) {
  constexpr int RPW = MMVQ_RPW;
  const int grid = (N + 4 * RPW - 1) / (4 * RPW);
  const int64_t xrb = (int64_t)K * (int64_t)sizeof(T) * (act == ACT_NONE ? 1 : 2);
  const int tokens = pairs / top_k;
  const int64_t q8_bytes = (int64_t)tokens * q8_row_bytes(K);
  const int64_t sorted_cap = (int64_t)pairs + (int64_t)num_experts * (MOE_VEC_GROUP - 1);
  const int64_t block_cap = (sorted_cap + MOE_VEC_GROUP - 1) / MOE_VEC_GROUP;
  const int64_t need = q8_bytes + (sorted_cap + block_cap + 1) * (int64_t)sizeof(int32_t);
  // grouping pays once experts are shared
  if (num_experts > 0 && num_experts <= 1024 && moe_share_pays(pairs, num_experts, (int64_t)N * (K / F::QK) * F::BS) && block_cap <= 65535 &&
      need <= scratch_bytes) {
    int rc = quantize_q8_1(x, xdtype, scratch, tokens, K, stream, act);
    if (rc != GGUF_OK) return rc;
    int32_t* sorted = (int32_t*)((char*)scratch + q8_bytes);  // q8 rows are a multiple of 4 bytes long
    int32_t* experts = sorted + sorted_cap;
    int32_t* post = experts + block_cap;
    rc = gguf_moe_align_block_size(topk_ids, pairs, num_experts, MOE_VEC_GROUP, sorted, sorted_cap, experts, block_cap, post,
                                   (gguf_stream_t)stream);
    if (rc != GGUF_OK) return rc;
    const int kchunk = kchunk_for(MOE_VEC_GROUP, K);
    const size_t lds = mmvq_lds<F, MOE_VEC_GROUP>(kchunk);
    constexpr int GRPW = MOE_VEC_GROUP_RPW;  // rows per wave: more rows amortise the staging of the group's activations
    const int ggrid = (N + 4 * GRPW - 1) / (4 * GRPW);
    hipLaunchKernelGGL((mmvq_kernel<F, MOE_VEC_GROUP, GRPW, T, true, false>), dim3(ggrid, (unsigned)block_cap), dim3(256), lds, stream,
                       (const uint8_t*)W, (const char*)scratch, (T*)Y, N, K, kchunk, q8_row_bytes(K), (int64_t)N,
                       MoeVecArgs{topk_ids, sorted, experts, top_k, pairs, (int)ACT_NONE}, (int64_t)(K / F::QK) * F::BS, (const T*)nullptr);
    return launch_status();
  }
  // one workgroup row per pair: the streaming kernel where the shape fits it
  if (act == ACT_NONE ? launch_stream_moe<F, T, false>(W, (const T*)x, (T*)Y, N, K, topk_ids, top_k, pairs, act, num_experts, stream)
                      : launch_stream_moe<F, T, true>(W, (const T*)x, (T*)Y, N, K, topk_ids, top_k, pairs, act, num_experts, stream))
    return launch_status();
  const int kchunk = kchunk_for(1, K);
  const size_t lds = mmvq_lds<F, 1>(kchunk);
  for (int z0 = 0; z0 < pairs; z0 += 65535) {
    const int nz = pairs - z0 < 65535 ? pairs - z0 : 65535;
    // the pair index is rebuilt from blockIdx.y, so later slabs shift the id and output bases by whole tokens
    if (z0 % top_k != 0) return GGUF_ERR_SHAPE;
    hipLaunchKernelGGL((mmvq_kernel<F, 1, RPW, T, true, true>), dim3(grid, nz), dim3(256), lds, stream,
                       (const uint8_t*)W, x + (int64_t)(z0 / top_k) * xrb, (T*)Y + (int64_t)z0 * N, N, K, kchunk, xrb,
                       (int64_t)N, MoeVecArgs{topk_ids + z0, nullptr, nullptr, top_k, nz, act}, (int64_t)(K / F::QK) * F::BS, (const T*)nullptr);
  }
  return launch_status();
}

template <class F>
static int moe_vec_fmt(const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                       int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_vec_typed<F, scalar_t>(W, (const char*)x, Y, dtype, N, K, ids, top_k, pairs, act,
                                                                num_experts, scratch, scratch_bytes, s)));
  return GGUF_ERR_DTYPE;
}

template <class F>
static int mmvq_fmt(const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                    hipStream_t s, const LinearArgs& la) {
  GGUF_DISPATCH_DTYPE(dtype, return (mmvq_typed<F, scalar_t>(W, x, ws, Y, dtype, N, K, M, s, la)));
  return GGUF_ERR_DTYPE;
}


}  // namespace gguf
