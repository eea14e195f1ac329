// The tile GEMM for up to 16 rows of X without LDS staging of the weights (Q4_K).
//
// With at most 16 rows every weight is used by exactly one MFMA, so staging the decoded weights in LDS buys no reuse:
// it only reshapes them into the MFMA operand layout, at the price of a barrier per step of K.  For Q4_K that layout
// can be read straight from the packed block.  The 32 values of block kb of a super-block are the low (kb even) or
// high (kb odd) nibbles of the 32 bytes qs[32 (kb / 2) ..], and the operand lane (column c, k group g) of a 64-deep
// int8 MFMA supplies 16 values.  A lane fetches, per super-block and column, the 16-byte header and the two 16-byte
// pieces qs[64 i + 16 g ..], i = 0, 1: the four lanes of a column read 64 contiguous bytes per load (8-byte pieces,
// the layout of the 32-deep MFMA, stream at 60 % of that rate: 16 rows x 32 bytes per load instruction).  A piece
// holds half a block in its low nibbles and half of the next block in its high nibbles; k groups 0, 1 of a column hold
// one pair of blocks and groups 2, 3 the pair after it, so each MFMA runs with the activations of the other two groups
// zeroed: eight MFMAs per super-block and column tile, one per block.  Only the activations go through LDS.
//
// K is split over the eight waves of a workgroup, not over workgroups: a workgroup owns 16 or 32 columns, each wave
// takes up to two super-blocks, and the eight partial tiles are added through LDS in the order of K.  A split over
// workgroups writes and re-reads fp32 partial tiles in memory, and with about one workgroup per wave slot of the chip
// nothing overlaps that traffic: the kernel that did so spent 13 of its 17 us outside the weight stream (Q4_K
// [14336,4096], 16 rows).  Workgroups split K between them only when the stretch does not fit LDS (K > 4096) or the
// output has too few column groups to fill the chip.
// More than 16 rows as further passes of 16 over the weights a wave holds were measured and lose to the staged tiles:
// every pass repeats the rescaling, which is what the kernel spends its arithmetic on ([14336,4096] at 32 rows 37
// against 32 us, at 64 rows 60 against 37 us).  One workgroup per CU instead of two, so that the rounds of workgroups
// overlap each other's phases, is slower too (19.5 against 16.8 us).
// Arithmetic as in the other integer tile kernels (mmq.cuh:2-104, vecdotq.cuh:353-379: exact int32 block sums,
// `d*sc*d8*S - dmin*m*s8` with the stored block sums s8).
#include "mmq_i_core.h"

namespace gguf {

typedef int v4i_d __attribute__((ext_vector_type(4)));
typedef _Float16 h2_d __attribute__((ext_vector_type(2)));
typedef uint32_t u4_d __attribute__((ext_vector_type(4)));

constexpr int kDirectKspl = 8, kDirectMaxSb = 16;        // waves per workgroup; super-blocks of K per workgroup (74 KB of LDS)

struct Direct16Args {
  int M, N, K, Kp, gsplits, per_wg;   // per_wg: super-blocks of K per workgroup
  int64_t ws_row_bytes, w_pitch, ldy;
  float* partial;
};

template <typename T, int KSPL, int CT, bool Q5>
__global__ __launch_bounds__(64 * KSPL, 4) void rows16_q4k_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                                    T* __restrict__ Y, const T* __restrict__ bias, Direct16Args a) {
  constexpr int NT = 64 * KSPL, N_T = 16 * CT, BS = Q5 ? 176 : 144, QS = Q5 ? 48 : 16;   // block bytes, offset of qs
  constexpr int MAX_SB = kDirectMaxSb;
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lcol = lane & 15, lgrp = lane >> 4;
  const int ks = wave;                                    // this wave's stretch of K

  const int tiles = (a.N + N_T - 1) / N_T;
  int wg = blockIdx.x;
  const int total8 = (tiles * a.gsplits) & ~7;
  if (wg < total8) wg = (wg & 7) * (total8 >> 3) + (wg >> 3);
  const int tile = wg % tiles, gs = wg / tiles, n_base = tile * N_T;
  const int nsb = a.K >> 8;                               // super-blocks per row
  const int sb0 = gs * a.per_wg, nmine = min(nsb, sb0 + a.per_wg) - sb0;   // >= 1 (host)
  const int pw = (nmine + KSPL - 1) / KSPL;
  const int my0 = ks * pw, my1 = min(nmine, my0 + pw);    // this wave's super-blocks, relative to sb0

  // ---- this wave's columns; its first two super-blocks are requested before anything else.  Per super-block and
  // column a lane (column c, k group g) holds the header and two 16-byte pieces of qs, [64 i + 16 g, + 16) for i = 0, 1:
  // the four lanes of a column read 64 contiguous bytes per load.  Piece i of lane g is half g % 2 of the byte pair
  // row 2 i + g / 2, i.e. 16 values of block 4 i + 2 (g / 2) in the low nibbles and of the block after it in the high.
  const uint8_t* wrow[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c)
    wrow[c] = W + (int64_t)min(n_base + 16 * c + lcol, a.N - 1) * a.w_pitch + (int64_t)sb0 * BS;
  // Q5_K: the fifth bits of values l and 32 + l .. 224 + l of the super-block are the bits of qh[l]; a piece covers
  // l = 16 (g % 2) .. + 15 of its blocks, so the lane takes that half of qh (bit number = block number)
  struct Blk { uint4 hdr; u4_d q[2]; u4_d qh; };
  auto fetch = [&](int sb, Blk (&b)[CT]) {
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      const uint8_t* p = wrow[c] + sb * BS;
      b[c].hdr = *(const uint4*)p;
      if constexpr (Q5) b[c].qh = *(const u4_d*)(p + 16 + 16 * (lgrp & 1));
#pragma unroll
      for (int i = 0; i < 2; ++i) b[c].q[i] = *(const u4_d*)(p + QS + 64 * i + 16 * lgrp);
    }
  };
  // ---- activations of super-blocks [sb0, sb0 + nmine) -> LDS: xq[16][pitch] int8, xsc[nmine * 8][16] half2 (d8, s8).
  // Requested before the weights: loads return in order, so the wait for the activations must not include the
  // weights.  Every thread issues every load (clamped to the last granule) so that the loads in flight can be counted.
  // A thread stages pieces of one row: NT / 16 threads per row, consecutive threads consecutive pieces.
  constexpr int TPR = NT / 16, AI = 16 * MAX_SB / TPR, SI = 8 * MAX_SB / TPR;
  const int pitch = nmine * 256 + 16;
  int8_t* xq = (int8_t*)smem;
  h2_d* xsc = (h2_d*)(smem + 16 * pitch);
  const int gpr = nmine * 16, spr = nmine * 8;             // 16-byte granules, blocks per row
  const int am = tid / TPR, at = tid % TPR;
  const char* const arow = ws + (int64_t)min(am, a.M - 1) * a.ws_row_bytes;
  const float* const asc = (const float*)(arow + a.Kp) + sb0 * 8;
  u4_d areg[AI];
  float dreg[SI], sreg[SI];
#pragma unroll
  for (int i = 0; i < AI; ++i) areg[i] = *(const u4_d*)(arow + sb0 * 256 + 16 * min(at + TPR * i, gpr - 1));
#pragma unroll
  for (int i = 0; i < SI; ++i) {
    const int kb = min(at + TPR * i, spr - 1);
    dreg[i] = asc[kb];
    sreg[i] = asc[a.Kp / 32 + kb];
  }
  Blk cur[CT], nxt[CT];
  fetch(min(my0, nmine - 1), cur);
  fetch(min(my0 + 1, nmine - 1), nxt);
  // (threads past the end store the last piece once more: a guarded store would draw its load into the guard)
#pragma unroll
  for (int i = 0; i < AI; ++i) *(u4_d*)(xq + am * pitch + 16 * min(at + TPR * i, gpr - 1)) = areg[i];
#pragma unroll
  for (int i = 0; i < SI; ++i)   // both are half-precision values widened to fp32 by the quantizer: the narrowing is exact
    xsc[min(at + TPR * i, spr - 1) * 16 + am] = (h2_d){(_Float16)dreg[i], (_Float16)sreg[i]};

  float acc[CT][4];
#pragma unroll
  for (int c = 0; c < CT; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[c][r] = 0.0f;
  const v4i_d seed = {kSeedBits, kSeedBits, kSeedBits, kSeedBits};
  __syncthreads();

  // One super-block of this wave's two column tiles.  An MFMA of 64 values takes 16 per lane: k groups 0, 1 of a
  // piece hold one block and groups 2, 3 the block two further on, so each is contracted with the activations of the
  // other pair of groups zeroed.
  auto consume = [&](int s, const Blk (&b)[CT], bool valid) {
    const int8_t* xrow = xq + lcol * pitch + s * 256 + 64 * (lgrp >> 1) + 16 * (lgrp & 1);
#pragma unroll
    for (int c = 0; c < CT; ++c) {   // (one column tile at a time: both tiles' scales at once do not fit the registers)
      // 6-bit scales and mins of the 8 sub-blocks (dequantize.cuh:156-163), times d and dmin
      float dw[8], mw[8];
      const uint32_t dm = valid ? b[c].hdr.x : 0u;       // a super-block past the stretch was re-read: scaled to nothing
      const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(dm & 0xFFFF));
      const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(dm >> 16));
      // the twelve scale bytes: sc, m of blocks 0..3 in the low six bits of bytes 0..3, 4..7; of blocks 4..7 the
      // low four bits in the nibbles of bytes 8..11 and the high two in the top bits of bytes 0..3, 4..7
      const uint32_t s_lo = b[c].hdr.y, s_mid = b[c].hdr.z, s_hi = b[c].hdr.w;
      const uint32_t sc4[2] = {s_lo & 0x3F3F3F3Fu, (s_hi & 0x0F0F0F0Fu) | ((s_lo >> 2) & 0x30303030u)};
      const uint32_t mn4[2] = {s_mid & 0x3F3F3F3Fu, ((s_hi >> 4) & 0x0F0F0F0Fu) | ((s_mid >> 2) & 0x30303030u)};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        dw[j] = d * (float)((sc4[j >> 2] >> (8 * (j & 3))) & 0xFF);
        mw[j] = dmin * (float)((mn4[j >> 2] >> (8 * (j & 3))) & 0xFF);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          // this lane's 16 activations of block 4 i + 2 (lgrp / 2) + h
          const v4i_d av = *(const v4i_d*)(xrow + (4 * i + h) * 32);
          const v4i_d zero = {0, 0, 0, 0};
          v4i_d bv;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            uint32_t v = (h ? b[c].q[i][e] >> 4 : b[c].q[i][e]) & 0x0F0F0F0Fu;
            if constexpr (Q5) v |= ((b[c].qh[e] >> (4 * i + h + 2 * (lgrp >> 1))) & 0x01010101u) << 4;
            bv[e] = (int)v;
          }
#pragma unroll
          for (int sel = 0; sel < 2; ++sel) {
            const int blkno = 4 * i + 2 * sel + h;
            const v4i_d asel = (lgrp >> 1) == sel ? av : zero;
            const v4i_d S = __builtin_amdgcn_mfma_i32_16x16x64_i8(asel, bv, seed, 0, 0, 0);
            const uint4 sc4 = *(const uint4*)(xsc + (s * 8 + blkno) * 16 + 4 * lgrp);
            const uint32_t scw[4] = {sc4.x, sc4.y, sc4.z, sc4.w};
            const float w = dw[blkno], nsw = -kSeed * w, nm = -mw[blkno];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const h2_d hh = __builtin_bit_cast(h2_d, scw[r]);
              acc[c][r] = __builtin_fmaf(seeded_times(S[r], w, nsw), (float)hh[0], acc[c][r]);
              acc[c][r] = __builtin_fmaf((float)hh[1], nm, acc[c][r]);
            }
          }
        }
    }
  };
  static_assert(MAX_SB <= 2 * KSPL, "a wave holds at most two super-blocks");
  // (both unconditionally: a load whose only use is guarded is moved into the guard, behind the barrier)
  consume(min(my0, nmine - 1), cur, my0 < my1);
  consume(min(my0 + 1, nmine - 1), nxt, my0 + 1 < my1);

  // ---- the KSPL partial tiles are added in the order of K
  __syncthreads();                                        // every wave is done with the activations
  float* red = (float*)smem;                              // [KSPL][16][N_T]
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int c = 0; c < CT; ++c) red[(ks * 16 + 4 * lgrp + r) * N_T + 16 * c + lcol] = acc[c][r];
  __syncthreads();
  float* const mine = a.gsplits > 1 ? a.partial + ((int64_t)tile * a.gsplits + gs) * (16 * N_T) : nullptr;
  for (int e = tid; e < 16 * N_T; e += NT) {
    float sum = red[e];
#pragma unroll
    for (int z = 1; z < KSPL; ++z) sum += red[z * 16 * N_T + e];
    const int m = e / N_T, nn = n_base + e % N_T;
    if (mine) mine[e] = sum;
    else if (m < a.M && nn < a.N) Y[(int64_t)m * a.ldy + nn] = finish<T>(sum, bias, nn);
  }
}

// How a call is laid out.  One column tile per wave (16 columns per workgroup) until that gives 640 workgroups, two
// above (measured on K = 4096 at 16 rows: N = 4096 8.9 against 13.5 us, N = 8192 11.3, N = 14336 16.8 against 17.5 us).
// Workgroups split K between them when a stretch would not fit LDS (K > 4096), or down to one super-block per wave
// when the output has fewer than 192 column groups.
struct Direct16Plan {
  int ct, tiles, gsplits, per_wg;
  int64_t partial_bytes() const { return gsplits > 1 ? (int64_t)tiles * gsplits * (16 * 16 * ct * 4) : 0; }
};
static Direct16Plan direct16_plan(int type, int N, int K, int64_t partial_bytes_available) {
  Direct16Plan p;
  p.ct = type == T_Q4_K && (N + 31) / 32 >= 320 ? 2 : 1;   // (with Q5_K's fifth bits two column tiles do not fit the registers)
  p.tiles = (N + 16 * p.ct - 1) / (16 * p.ct);
  const int nsb = K / 256;
  p.gsplits = (nsb + kDirectMaxSb - 1) / kDirectMaxSb;
  if (p.tiles * p.gsplits < 192) p.gsplits = std::max(p.gsplits, std::min(384 / p.tiles, nsb / kDirectKspl));
  if (p.gsplits < 1) p.gsplits = 1;
  p.per_wg = (nsb + p.gsplits - 1) / p.gsplits;
  p.gsplits = (nsb + p.per_wg - 1) / p.per_wg;
  if (p.partial_bytes() > partial_bytes_available) {
    p.gsplits = nsb > kDirectMaxSb ? 0 : 1;               // 0: not without room for partial tiles
    p.per_wg = nsb;
  }
  return p;
}
int64_t rows16_direct_partial_bytes(int N, int K) {   // (the format is not known where the workspace is sized)
  if (K % 256) return 0;
  return std::max(direct16_plan(T_Q4_K, N, K, INT64_MAX).partial_bytes(), direct16_plan(T_Q5_K, N, K, INT64_MAX).partial_bytes());
}

template <typename T, int CT, bool Q5>
static int rows16_q4k_launch(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, const Direct16Plan& p,
                             hipStream_t stream, const LinearArgs& la) {
  constexpr int KSPL = kDirectKspl, N_T = 16 * CT;
  const size_t act = (size_t)16 * (p.per_wg * 256 + 16) + (size_t)p.per_wg * 8 * 16 * 4, red = (size_t)KSPL * 16 * N_T * 4;
  const size_t lds = act > red ? act : red;
  auto kern = rows16_q4k_kernel<T, KSPL, CT, Q5>;
  if (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, 80 * 1024, done);
  }
  Direct16Args a = {M, N, K, (int)q8_kp(K), p.gsplits, p.per_wg, q8_row_bytes(K), la.w_pitch ? la.w_pitch : (int64_t)(K / 256) * (Q5 ? 176 : 144),
                    la.ldy ? la.ldy : (int64_t)N, partial};
  hipLaunchKernelGGL(kern, dim3(p.tiles * p.gsplits), dim3(64 * KSPL), lds, stream, (const uint8_t*)W, (const char*)ws, (T*)Y,
                     (const T*)la.bias, a);
  if (p.gsplits > 1)
    hipLaunchKernelGGL((mmqi_reduce_kernel<16, N_T, T>), dim3(p.tiles, 1), dim3(256), 0, stream, partial, (T*)Y, M, N, 1, 0, p.gsplits,
                       a.ldy, (const T*)la.bias);
  return launch_status();
}

template <typename T, bool Q5>
static int rows16_q4k_typed(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, const Direct16Plan& p,
                            hipStream_t stream, const LinearArgs& la) {
  if constexpr (!Q5)
    if (p.ct == 2) return rows16_q4k_launch<T, 2, Q5>(W, ws, Y, M, N, K, partial, p, stream, la);
  return rows16_q4k_launch<T, 1, Q5>(W, ws, Y, M, N, K, partial, p, stream, la);
}

// Whether rows16_direct() would run this call.
bool rows16_direct_takes(const void* W, int64_t w_pitch, int type, int M, int N, int K, int64_t partial_bytes) {
  if ((type != T_Q4_K && type != T_Q5_K) || M > 16 || K % 256) return false;
  const int64_t pitch = w_pitch ? w_pitch : (int64_t)(K / 256) * (type == T_Q5_K ? 176 : 144);
  if (((uintptr_t)W & 15) || (pitch & 15)) return false;
  return direct16_plan(type, N, K, partial_bytes).gsplits != 0;
}

// Q4_K or Q5_K, at most 16 rows of X, W and its row pitch 16-byte aligned; GGUF_NOT_TAKEN otherwise.
int rows16_direct(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial, int64_t partial_bytes,
                  hipStream_t s, const LinearArgs& la) {
  if (!rows16_direct_takes(W, la.w_pitch, type, M, N, K, partial_bytes)) return GGUF_NOT_TAKEN;
  const Direct16Plan p = direct16_plan(type, N, K, partial_bytes);
  if (type == T_Q5_K) {
    GGUF_DISPATCH_DTYPE(dtype, return (rows16_q4k_typed<scalar_t, true>(W, ws, Y, M, N, K, partial, p, s, la)));
    return GGUF_ERR_DTYPE;
  }
  GGUF_DISPATCH_DTYPE(dtype, return (rows16_q4k_typed<scalar_t, false>(W, ws, Y, M, N, K, partial, p, s, la)));
  return GGUF_ERR_DTYPE;
}

}  // namespace gguf
