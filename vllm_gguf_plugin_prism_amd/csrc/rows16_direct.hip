// The tile GEMM for up to 32 rows of X without LDS staging of the weights (Q4_K, Q5_K, Q6_K; Q4_0, Q8_0 up to 16 rows).
//
// With so few rows every weight is used by one or two MFMAs, so staging the decoded weights in LDS buys no reuse:
// it only reshapes them into the MFMA operand layout, at the price of a barrier per step of K.  For these formats that
// layout can be read straight from the packed block.  The operand lane (column c, k group g) of a 64-deep int8 MFMA
// supplies 16 values.
//   Q4_K: the 32 values of block kb of a super-block are the low (kb even) or high (kb odd) nibbles of the 32 bytes
//   qs[32 (kb / 2) ..].  A lane fetches, per super-block and column, the 16-byte header and the two 16-byte pieces
//   qs[64 i + 16 g ..], i = 0, 1: the four lanes of a column read 64 contiguous bytes per load (8-byte pieces, the
//   layout of the 32-deep MFMA, stream at 60 % of that rate: 16 rows x 32 bytes per load instruction).  A piece holds
//   half a block in its low nibbles and half of the next block in its high nibbles; k groups 0, 1 of a column hold one
//   pair of blocks and groups 2, 3 the pair after it, so each MFMA runs with the activations of the other two groups
//   zeroed: eight MFMAs per super-block and column tile, one per block.
//   Q5_K: the same, with the 16 bytes of qh that hold the pieces' fifth bits.
//   Q6_K: a scale covers 16 values, which is what one lane holds: four MFMAs per piece and nibble, each with the
//   activations of one k group and zeros for the other three.  The 210-byte blocks sit at even addresses, so most of
//   the 16-byte loads are unaligned, which costs about 30 % (measured with the blocks moved to 208-byte spacing);
//   fetching whole dwords from the boundary below and funnel-shifting recovers 4 % of that and was not kept.
//   Q4_0, Q8_0: a lane owns whole 32-value blocks (18 and 34 bytes at even addresses: every 16-byte load unaligned),
//   two MFMAs per block onto one sum, one k group active at a time; the block scales reach the other lanes of the
//   column by two lane swaps.  These stream at 2.3 TB/s only and serve a narrower range (rows16_direct_pays).
// Only the activations go through LDS.
//
// K is split over the eight waves of a workgroup, not over workgroups: a workgroup owns 16 or 32 columns, each wave
// takes up to two super-blocks, and the eight partial tiles are added through LDS in the order of K.  A split over
// workgroups writes and re-reads fp32 partial tiles in memory, and with about one workgroup per wave slot of the chip
// nothing overlaps that traffic: the kernel that did so spent 13 of its 17 us outside the weight stream (Q4_K
// [14336,4096], 16 rows).  Workgroups split K between them only when the stretch does not fit LDS (K > 4096) or the
// output has too few column groups to fill the chip.
// With 32 columns a wave takes its two 16-column tiles in turn, the second requested as the registers of the first
// become free: the staged activations serve both, the second tile's loads overlap the first's arithmetic, and the
// kernel keeps the registers of one tile (both tiles held at once: Q4_K [14336,4096] 16.8 against 15.3 us; four tiles
// in turn gain nothing over two).
// 17 to 32 rows (the K-quants): two 16-row tiles of X, every weight operand multiplied with both.  The 32 rows of a
// 4096-value stretch fill LDS, so one workgroup runs per CU (with twice the registers) and owns up to 64 columns, so
// that one round of workgroups covers the output: Q4_K [14336,4096] 32 -> 22 us, Q5_K 47 -> 24 us, Q6_K 45 -> 29 us
// against the staged tiles.  Further rows as passes of 16 over the weights a wave holds, restaging the activations,
// lose to the staged tiles ([14336,4096] at 32 rows 37 against 32 us, at 64 rows 60 against 37 us), and for 16 rows one
// workgroup per CU instead of two is slower (19.5 against 16.8 us).
// Arithmetic as in the other integer tile kernels (mmq.cuh:2-104, vecdotq.cuh:353-379, 467-491: exact int32 block
// sums, `d*sc*d8*S - dmin*m*s8` with the stored block sums s8; Q6_K `d*sc*d8*S` per 16 values).
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

enum { DIRECT_Q4_K = 0, DIRECT_Q5_K = 1, DIRECT_Q6_K = 2, DIRECT_Q4_0 = 3, DIRECT_Q8_0 = 4 };

// NP: 16-column tiles a wave takes in turn (the workgroup owns 16 NP columns).  GSUM (Q4_K, Q5_K): the offset term
// multiplies d8 * sum(q8), the GEMV operator's arithmetic (vecdotq.cuh:328-351), instead of the stored block sum.
// RT: 16-row tiles of X (1 or 2).  With two, every weight operand meets both tiles' activations; the 32 rows of a
// 4096-value stretch fill LDS, so one workgroup runs per CU, with twice the registers.
template <typename T, int KSPL, int NP, int FMT, bool GSUM, int RT>
__global__ __launch_bounds__(64 * KSPL, RT == 2 ? 2 : 4) void rows16_direct_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                                      T* __restrict__ Y, const T* __restrict__ bias, Direct16Args a) {
  constexpr bool Q5 = FMT == DIRECT_Q5_K, Q6 = FMT == DIRECT_Q6_K, Q40 = FMT == DIRECT_Q4_0, Q80 = FMT == DIRECT_Q8_0;
  constexpr bool B32 = Q40 || Q80;                       // 32-value blocks: eight of them stand for a super-block
  constexpr int NT = 64 * KSPL, N_T = 16 * NP;
  constexpr int BS = Q6 ? 210 : Q5 ? 176 : Q40 ? 8 * 18 : Q80 ? 8 * 34 : 144;   // bytes of 256 values
  constexpr int QS = Q5 ? 48 : 16;                       // offset of qs (Q4_K, Q5_K)
  constexpr int XR = 16 * RT, XROWS = Q6 || B32 ? XR + 1 : XR;   // rows of X in LDS; a row of zeros behind them
  constexpr int MAX_SB = kDirectMaxSb;
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lcol = lane & 15, lgrp = lane >> 4;
  const int ks = wave;                                    // this wave's stretch of K

  const int tiles = (a.N + N_T - 1) / N_T;
  int wg = blockIdx.x;
  const int total8 = (tiles * a.gsplits) & ~7;
  if (wg < total8) wg = (wg & 7) * (total8 >> 3) + (wg >> 3);   // each of the 8 XCDs gets a contiguous run of tiles
  const int tile = wg % tiles, gs = wg / tiles, n_base = tile * N_T;
  const int nsb = a.K >> 8;                               // super-blocks per row
  const int sb0 = gs * a.per_wg, nmine = min(nsb, sb0 + a.per_wg) - sb0;   // >= 1 (host)
  const int pw = (nmine + KSPL - 1) / KSPL;
  const int my0 = ks * pw, my1 = min(nmine, my0 + pw);    // this wave's super-blocks, relative to sb0

  // ---- this wave's columns, and what a lane holds of one super-block of one column
  const uint8_t* wrow[NP];
#pragma unroll
  for (int q = 0; q < NP; ++q) wrow[q] = W + (int64_t)min(n_base + 16 * q + lcol, a.N - 1) * a.w_pitch + (int64_t)sb0 * BS;
  // Q4_K: the header and the pieces qs[64 i + 16 g ..]: piece i of lane g is half g % 2 of the byte pair row
  // 2 i + g / 2, i.e. 16 values of block 4 i + 2 (g / 2) in the low nibbles and of the block after it in the high.
  // Q5_K: the fifth bits of values l and 32 + l .. 224 + l of the super-block are the bits of qh[l]; a piece covers
  // l = 16 (g % 2) .. + 15 of its blocks, so the lane takes that half of qh (bit number = block number).
  // Q6_K (loads of any alignment): per half n of the super-block a lane takes ql[64 n + 16 g ..] -- its low nibbles
  // are the 16-value scale group 8 n + g, its high nibbles group 8 n + 4 + g.  The upper two bits of both halves are
  // in qh[32 n + 16 (g % 2) ..]; the lane fetches qh[16 g ..] and four of the 16 scales, and lane swaps complete both.
  // Q4_0, Q8_0 (blocks of 18 and 34 bytes at even addresses): a lane owns whole blocks, 4 i + g of every eight, i = 0, 1
  // -- the four lanes of a column read 72 or 136 contiguous bytes.  Values 0..15 of the block (Q4_0: the low nibbles)
  // and 16..31 go through two MFMAs onto one sum.
  struct Blk4 { uint4 hdr; u4_d q[2]; u4_d qh; };
  struct Blk6 { u4_d ql[2], qh; uint32_t sc, d; };   // qh: piece g of the four; sc: scales 4 g .. 4 g + 3
  struct Blk32 { u4_d q[Q80 ? 4 : 2]; uint32_t d[2]; };
  using Blk = std::conditional_t<Q6, Blk6, std::conditional_t<B32, Blk32, Blk4>>;
  auto fetch = [&](int q, int sb, Blk& b) {
    const uint8_t* p = wrow[q] + sb * BS;
    if constexpr (B32) {
      constexpr int BB = BS / 8;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint8_t* pb = p + (4 * i + lgrp) * BB;
        b.d[i] = ld<uint16_t>(pb);
        if constexpr (Q80) { b.q[2 * i] = ld<u4_d>(pb + 2); b.q[2 * i + 1] = ld<u4_d>(pb + 18); }
        else b.q[i] = ld<u4_d>(pb + 2);
      }
    } else if constexpr (Q6) {
#pragma unroll
      for (int n = 0; n < 2; ++n) b.ql[n] = ld<u4_d>(p + 64 * n + 16 * lgrp);
      b.qh = ld<u4_d>(p + 128 + 16 * lgrp);
      b.sc = ld<uint32_t>(p + 192 + 4 * lgrp);
      b.d = ld<uint16_t>(p + 208);
    } else {
      b.hdr = *(const uint4*)p;
      if constexpr (Q5) b.qh = *(const u4_d*)(p + 16 + 16 * (lgrp & 1));
#pragma unroll
      for (int i = 0; i < 2; ++i) b.q[i] = *(const u4_d*)(p + QS + 64 * i + 16 * lgrp);
    }
  };

  // ---- activations of super-blocks [sb0, sb0 + nmine) -> LDS: xq[16][pitch] int8, xsc[nmine * 8][16] half2 (d8, s8).
  // Requested before the weights: loads return in order, so the wait for the activations must not include the
  // weights.  Every thread issues every load (clamped to the last granule) so that the loads in flight can be counted.
  // A thread stages pieces of one row: NT / 16 threads per row, consecutive threads consecutive pieces.
  constexpr int TPR = NT / 16, AI = 16 * MAX_SB / TPR, SI = 8 * MAX_SB / TPR;
  const int pitch = nmine * 256 + 16;
  int8_t* xq = (int8_t*)smem;
  h2_d* xsc = (h2_d*)(smem + XROWS * pitch);
  const int gpr = nmine * 16, spr = nmine * 8;             // 16-byte granules, blocks per row
  const int am = tid / TPR, at = tid % TPR;
  u4_d areg[RT][AI];
  float dreg[RT][SI], sreg[RT][SI];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const char* const arow = ws + (int64_t)min(16 * rt + am, a.M - 1) * a.ws_row_bytes;
    const float* const asc = (const float*)(arow + a.Kp) + sb0 * 8;
#pragma unroll
    for (int i = 0; i < AI; ++i) areg[rt][i] = *(const u4_d*)(arow + sb0 * 256 + 16 * min(at + TPR * i, gpr - 1));
#pragma unroll
    for (int i = 0; i < SI; ++i) {
      const int kb = min(at + TPR * i, spr - 1);
      dreg[rt][i] = asc[kb];
      sreg[rt][i] = asc[(GSUM ? 2 : 1) * (a.Kp / 32) + kb];   // the stored sum s8, or du = d8 * sum(q8)
    }
  }
  Blk cur, nxt;
  fetch(0, min(my0, nmine - 1), cur);
  fetch(0, min(my0 + 1, nmine - 1), nxt);
  // (threads past the end store the last piece once more: a guarded store would draw its load into the guard)
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int i = 0; i < AI; ++i) *(u4_d*)(xq + (16 * rt + am) * pitch + 16 * min(at + TPR * i, gpr - 1)) = areg[rt][i];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
  for (int i = 0; i < SI; ++i) {
    // d8 and s8 are half-precision values widened to fp32 by the quantizer: the narrowing is exact.  du is not one, but
    // du / d8 = sum(q8) is an integer of at most 13 bits (|sum| <= 32 * 127 = 4064), exact as a quotient; a half holds
    // integers exactly only up to 2048, so the sum travels as a 16-bit integer in the place of the second half and is
    // widened again where d8 multiplies it together with the block sum.
    // (the hardware reciprocal's last-bit error rounds away: the quotient lies within 4065 * 2^-22 of an integer)
    h2_d pair = {(_Float16)dreg[rt][i], (_Float16)sreg[rt][i]};
    if constexpr (GSUM) {
      const int qsum = dreg[rt][i] != 0.0f ? (int)__builtin_rintf(sreg[rt][i] * __builtin_amdgcn_rcpf(dreg[rt][i])) : 0;
      const uint32_t bits = (uint32_t)__builtin_bit_cast(uint16_t, pair[0]) | ((uint32_t)qsum << 16);
      pair = __builtin_bit_cast(h2_d, bits);
    }
    xsc[min(at + TPR * i, spr - 1) * XR + 16 * rt + am] = pair;
  }
  if constexpr (XROWS > XR)
    for (int i = tid; i < gpr; i += NT) *(u4_d*)(xq + XR * pitch + 16 * i) = (u4_d){0u, 0u, 0u, 0u};

  float acc[RT][NP][4];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int q = 0; q < NP; ++q)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[rt][q][r] = 0.0f;
  const v4i_d seed = {kSeedBits, kSeedBits, kSeedBits, kSeedBits};
  __syncthreads();

  // One super-block of column tile q.  (A super-block past the wave's stretch was re-read: it is scaled to nothing.)
  auto consume = [&](int q, int s, const Blk& b, bool valid) {
    if constexpr (B32) {
      // the activations of the block that k group t owns for the lanes of that group, the row of zeros for the others
      const int8_t* xsel[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int t = 0; t < 4; ++t) xsel[rt][t] = xq + (lgrp == t ? 16 * rt + lcol : XR) * pitch + s * 256 + 32 * lgrp;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        // every lane of the column needs the scales of all four blocks: two lane swaps spread them (rows of 16 lanes
        // g0 g1 g2 g3 -> g0 g1 g0 g1 and g2 g3 g2 g3 -> four registers that hold one block's scale in every lane)
        const auto half01 = __builtin_amdgcn_permlane32_swap(b.d[i], b.d[i], false, false);
        const auto d01 = __builtin_amdgcn_permlane16_swap(half01[0], half01[0], false, false);
        const auto d23 = __builtin_amdgcn_permlane16_swap(half01[1], half01[1], false, false);
        const uint32_t dbits[4] = {d01[0], d01[1], d23[0], d23[1]};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int blk = 4 * i + t;
          v4i_d blo, bhi;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (Q80) { blo[e] = (int)b.q[2 * i][e]; bhi[e] = (int)b.q[2 * i + 1][e]; }
            else { blo[e] = (int)(b.q[i][e] & 0x0F0F0F0Fu); bhi[e] = (int)((b.q[i][e] >> 4) & 0x0F0F0F0Fu); }
          }
          const float w = valid ? (float)__builtin_bit_cast(_Float16, (uint16_t)dbits[t]) : 0.0f;
          const float nsw = -kSeed * w, nm = -8.0f * w;   // Q4_0: d * (q - 8), the 8 on the stored block sum (vecdotq.cuh:46-66)
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            const v4i_d alo = *(const v4i_d*)(xsel[rt][t] + 128 * i);
            const v4i_d ahi = *(const v4i_d*)(xsel[rt][t] + 128 * i + 16);
            v4i_d S = __builtin_amdgcn_mfma_i32_16x16x64_i8(alo, blo, seed, 0, 0, 0);
            S = __builtin_amdgcn_mfma_i32_16x16x64_i8(ahi, bhi, S, 0, 0, 0);
            const uint4 x4 = *(const uint4*)(xsc + (s * 8 + blk) * XR + 16 * rt + 4 * lgrp);
            const uint32_t scw[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const h2_d hh = __builtin_bit_cast(h2_d, scw[r]);
              acc[rt][q][r] = __builtin_fmaf(seeded_times(S[r], w, nsw), (float)hh[0], acc[rt][q][r]);
              if constexpr (Q40) acc[rt][q][r] = __builtin_fmaf((float)hh[1], nm, acc[rt][q][r]);
            }
          }
        }
      }
    } else if constexpr (Q6) {
      // the activations of k group t for the lanes of that group, the row of zeros for the others
      const int8_t* xsel[RT][4];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int t = 0; t < 4; ++t) xsel[rt][t] = xq + (lgrp == t ? 16 * rt + lcol : XR) * pitch + s * 256 + 16 * lgrp;
      const float d = valid ? (float)__builtin_bit_cast(_Float16, (uint16_t)b.d) : 0.0f;
      // Each of the four lanes of a column fetched one 16-byte piece of qh and four of the 16 scales; lane swaps hand
      // every lane the two pieces (g % 2 of either half) and all the scales it needs: rows of 16 lanes g0 g1 g2 g3 ->
      // g0 g1 g0 g1 and g2 g3 g2 g3, and once more -> one k group's register in every lane.
      u4_d qh[2];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const auto sw = __builtin_amdgcn_permlane32_swap(b.qh[e], b.qh[e], false, false);
        qh[0][e] = sw[0];
        qh[1][e] = sw[1];
      }
      const auto sc_h = __builtin_amdgcn_permlane32_swap(b.sc, b.sc, false, false);
      const auto sc01 = __builtin_amdgcn_permlane16_swap(sc_h[0], sc_h[0], false, false);
      const auto sc23 = __builtin_amdgcn_permlane16_swap(sc_h[1], sc_h[1], false, false);
      const uint32_t scs[4] = {sc01[0], sc01[1], sc23[0], sc23[1]};
#pragma unroll
      for (int n = 0; n < 2; ++n)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          v4i_d bv;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t lo = (h ? b.ql[n][e] >> 4 : b.ql[n][e]) & 0x0F0F0F0Fu;
            const uint32_t hi = (qh[n][e] >> (4 * h + 2 * (lgrp >> 1))) & 0x03030303u;
            bv[e] = (int)sub_bytes(lo | (hi << 4), 0x20202020u);
          }
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            const uint4 sc4 = *(const uint4*)(xsc + (s * 8 + 4 * n + 2 * h) * XR + 16 * rt + 4 * lgrp);       // block 4 n + 2 h
            const uint4 sc5 = *(const uint4*)(xsc + (s * 8 + 4 * n + 2 * h + 1) * XR + 16 * rt + 4 * lgrp);   // and the next
            const uint32_t d8w[2][4] = {{sc4.x, sc4.y, sc4.z, sc4.w}, {sc5.x, sc5.y, sc5.z, sc5.w}};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
              const int grp = 8 * n + 4 * h + t;             // 16 values 128 n + 64 h + 16 t .. of the super-block
              const v4i_d av = *(const v4i_d*)(xsel[rt][t] + 128 * n + 64 * h);
              const v4i_d S = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, seed, 0, 0, 0);
              const int sc = (int)(int8_t)((scs[grp >> 2] >> (8 * (grp & 3))) & 0xFF);
              const float w = d * (float)sc, nsw = -kSeed * w;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const h2_d hh = __builtin_bit_cast(h2_d, d8w[t >> 1][r]);
                acc[rt][q][r] = __builtin_fmaf(seeded_times(S[r], w, nsw), (float)hh[0], acc[rt][q][r]);
              }
            }
          }
        }
    } else {
      const int8_t* xrow[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) xrow[rt] = xq + (16 * rt + lcol) * pitch + s * 256 + 64 * (lgrp >> 1) + 16 * (lgrp & 1);
      // 6-bit scales and mins of the 8 sub-blocks (dequantize.cuh:156-163), times d and dmin
      float dw[8], mw[8];
      const uint32_t dm = valid ? b.hdr.x : 0u;
      const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(dm & 0xFFFF));
      const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(dm >> 16));
      // the twelve scale bytes: sc, m of blocks 0..3 in the low six bits of bytes 0..3, 4..7; of blocks 4..7 the
      // low four bits in the nibbles of bytes 8..11 and the high two in the top bits of bytes 0..3, 4..7
      const uint32_t s_lo = b.hdr.y, s_mid = b.hdr.z, s_hi = b.hdr.w;
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
          const v4i_d zero = {0, 0, 0, 0};
          v4i_d bv;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            uint32_t v = (h ? b.q[i][e] >> 4 : b.q[i][e]) & 0x0F0F0F0Fu;
            if constexpr (Q5) v |= ((b.qh[e] >> (4 * i + h + 2 * (lgrp >> 1))) & 0x01010101u) << 4;
            bv[e] = (int)v;
          }
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            // this lane's 16 activations of block 4 i + 2 (lgrp / 2) + h
            const v4i_d av = *(const v4i_d*)(xrow[rt] + (4 * i + h) * 32);
#pragma unroll
            for (int sel = 0; sel < 2; ++sel) {
              const int blkno = 4 * i + 2 * sel + h;
              const v4i_d asel = (lgrp >> 1) == sel ? av : zero;
              const v4i_d S = __builtin_amdgcn_mfma_i32_16x16x64_i8(asel, bv, seed, 0, 0, 0);
              const uint4 x4 = *(const uint4*)(xsc + (s * 8 + blkno) * XR + 16 * rt + 4 * lgrp);
              const uint32_t scw[4] = {x4.x, x4.y, x4.z, x4.w};
              const float w = dw[blkno], nsw = -kSeed * w, nm = -mw[blkno];
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const h2_d hh = __builtin_bit_cast(h2_d, scw[r]);
                if constexpr (GSUM) {   // d8 * (S * dw - m * sum(q8)): the offset joins the block sum before d8 is applied
                  const float qsum = (float)((int)scw[r] >> 16);   // the 16-bit integer staged in place of the second half
                  const float u = __builtin_fmaf(qsum, nm, seeded_times(S[r], w, nsw));
                  acc[rt][q][r] = __builtin_fmaf(u, (float)hh[0], acc[rt][q][r]);
                } else {
                  acc[rt][q][r] = __builtin_fmaf(seeded_times(S[r], w, nsw), (float)hh[0], acc[rt][q][r]);
                  acc[rt][q][r] = __builtin_fmaf((float)hh[1], nm, acc[rt][q][r]);
                }
              }
            }
          }
        }
    }
  };
  static_assert(MAX_SB <= 2 * KSPL, "a wave holds at most two super-blocks");
  // (both super-blocks unconditionally: a load whose only use is guarded is moved into the guard, behind the barrier)
#pragma unroll
  for (int q = 0; q < NP; ++q) {
    // the next tile is requested as soon as a super-block's registers are free (the fences keep the compiler from
    // starting those loads before that, which would need the registers of both tiles)
    consume(q, min(my0, nmine - 1), cur, my0 < my1);
    if (q + 1 < NP) {
      __builtin_amdgcn_sched_barrier(0);
      fetch(q + 1, min(my0, nmine - 1), cur);
      __builtin_amdgcn_sched_barrier(0);
    }
    consume(q, min(my0 + 1, nmine - 1), nxt, my0 + 1 < my1);
    if (q + 1 < NP) {
      __builtin_amdgcn_sched_barrier(0);
      fetch(q + 1, min(my0 + 1, nmine - 1), nxt);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- the KSPL partial tiles are added in the order of K
  __syncthreads();                                        // every wave is done with the activations
  float* red = (float*)smem;                              // [KSPL][XR][N_T]
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int q = 0; q < NP; ++q) red[(ks * XR + 16 * rt + 4 * lgrp + r) * N_T + 16 * q + lcol] = acc[rt][q][r];
  __syncthreads();
  float* const mine = a.gsplits > 1 ? a.partial + ((int64_t)tile * a.gsplits + gs) * (XR * N_T) : nullptr;
  for (int e = tid; e < XR * N_T; e += NT) {
    float sum = red[e];
#pragma unroll
    for (int z = 1; z < KSPL; ++z) sum += red[z * XR * N_T + e];
    const int m = e / N_T, nn = n_base + e % N_T;
    if (mine) mine[e] = sum;
    else if (m < a.M && nn < a.N) Y[(int64_t)m * a.ldy + nn] = finish<T>(sum, bias, nn);
  }
}

// How a call is laid out.  Up to 16 rows: 16 columns per workgroup until that gives 640 workgroups, 32 above (measured on Q4_K,
// K = 4096 at 16 rows: N = 4096 8.9 against 13.5 us, N = 8192 11.3, N = 14336 15.3 against 17.5 us).  Workgroups split K
// between them when a stretch would not fit LDS (K > 4096), or down to one super-block per wave when the output has
// fewer than 192 column groups.
struct Direct16Plan {
  int np, rt, tiles, gsplits, per_wg;   // np: 16-column tiles per workgroup; rt: 16-row tiles of X (1 or 2)
  int64_t partial_bytes() const { return gsplits > 1 ? (int64_t)tiles * gsplits * (16 * rt * 16 * np * 4) : 0; }
};
static Direct16Plan direct16_plan(int M, int N, int K, int64_t partial_bytes_available) {
  Direct16Plan p;
  p.rt = M > 16 ? 2 : 1;
  const int tiles16 = (N + 15) / 16;
  // 32 rows of X fill LDS, so one workgroup runs per CU: columns per workgroup so that one round of workgroups covers
  // the output where it can (Q4_K [14336,4096] at 32 rows: 64 columns 22 us, 32 columns 26 us)
  if (p.rt == 2) p.np = tiles16 <= 256 ? 1 : tiles16 <= 512 ? 2 : 4;
  else p.np = (N + 31) / 32 >= 320 ? 2 : 1;
  p.tiles = (N + 16 * p.np - 1) / (16 * p.np);
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
int64_t rows16_direct_partial_bytes(int M, int N, int K) { return K % 256 || M > 32 ? 0 : direct16_plan(M, N, K, INT64_MAX).partial_bytes(); }

// bytes of 256 values
static inline int direct_block_bytes(int type) {
  return type == T_Q6_K ? 210 : type == T_Q5_K ? 176 : type == T_Q4_0 ? 8 * 18 : type == T_Q8_0 ? 8 * 34 : 144;
}

template <typename T, int NP, int FMT, bool GSUM, int RT = 1>
static int rows16_direct_launch(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, const Direct16Plan& p,
                                hipStream_t stream, const LinearArgs& la) {
  constexpr int KSPL = kDirectKspl, N_T = 16 * NP, XROWS = FMT == DIRECT_Q4_K || FMT == DIRECT_Q5_K ? 16 * RT : 16 * RT + 1;
  constexpr int BS = FMT == DIRECT_Q6_K ? 210 : FMT == DIRECT_Q5_K ? 176 : FMT == DIRECT_Q4_0 ? 8 * 18 : FMT == DIRECT_Q8_0 ? 8 * 34 : 144;
  const size_t act = (size_t)XROWS * (p.per_wg * 256 + 16) + (size_t)p.per_wg * 8 * 16 * RT * 4, red = (size_t)KSPL * 16 * RT * N_T * 4;
  const size_t lds = act > red ? act : red;
  auto kern = rows16_direct_kernel<T, KSPL, NP, FMT, GSUM, RT>;
  if (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    allow_large_lds(kern, RT * 80 * 1024, done);
  }
  Direct16Args a = {M, N, K, (int)q8_kp(K), p.gsplits, p.per_wg, q8_row_bytes(K), la.w_pitch ? la.w_pitch : (int64_t)(K / 256) * BS,
                    la.ldy ? la.ldy : (int64_t)N, partial};
  hipLaunchKernelGGL(kern, dim3(p.tiles * p.gsplits), dim3(64 * KSPL), lds, stream, (const uint8_t*)W, (const char*)ws, (T*)Y,
                     (const T*)la.bias, a);
  if (p.gsplits > 1)
    hipLaunchKernelGGL((mmqi_reduce_kernel<16 * RT, N_T, T>), dim3(p.tiles, 1), dim3(256), 0, stream, partial, (T*)Y, M, N, 1, 0,
                       p.gsplits, a.ldy, (const T*)la.bias);
  return launch_status();
}

template <typename T, int FMT>
static int rows16_direct_typed(const void* W, const void* ws, void* Y, int M, int N, int K, float* partial, const Direct16Plan& p,
                               hipStream_t stream, const LinearArgs& la, bool gemv_sums) {
  if constexpr (FMT == DIRECT_Q4_K || FMT == DIRECT_Q5_K) {   // (the two operators agree on the other formats)
    if (gemv_sums) {
      if (p.rt == 2) {   // 17 .. 32 rows
        if (p.np == 4) return rows16_direct_launch<T, 4, FMT, true, 2>(W, ws, Y, M, N, K, partial, p, stream, la);
        if (p.np == 2) return rows16_direct_launch<T, 2, FMT, true, 2>(W, ws, Y, M, N, K, partial, p, stream, la);
        return rows16_direct_launch<T, 1, FMT, true, 2>(W, ws, Y, M, N, K, partial, p, stream, la);
      }
      if (p.np == 2) return rows16_direct_launch<T, 2, FMT, true>(W, ws, Y, M, N, K, partial, p, stream, la);
      return rows16_direct_launch<T, 1, FMT, true>(W, ws, Y, M, N, K, partial, p, stream, la);
    }
  }
  if constexpr (FMT == DIRECT_Q4_K || FMT == DIRECT_Q5_K || FMT == DIRECT_Q6_K) {
    if (p.rt == 2) {   // 17 .. 32 rows
      if (p.np == 4) return rows16_direct_launch<T, 4, FMT, false, 2>(W, ws, Y, M, N, K, partial, p, stream, la);
      if (p.np == 2) return rows16_direct_launch<T, 2, FMT, false, 2>(W, ws, Y, M, N, K, partial, p, stream, la);
      return rows16_direct_launch<T, 1, FMT, false, 2>(W, ws, Y, M, N, K, partial, p, stream, la);
    }
  }
  if (p.np == 2) return rows16_direct_launch<T, 2, FMT, false>(W, ws, Y, M, N, K, partial, p, stream, la);
  return rows16_direct_launch<T, 1, FMT, false>(W, ws, Y, M, N, K, partial, p, stream, la);
}

// Whether rows16_direct() would run this call.
bool rows16_direct_takes(const void* W, int64_t w_pitch, int type, int M, int N, int K, int64_t partial_bytes) {
  const bool kquant = type == T_Q4_K || type == T_Q5_K || type == T_Q6_K;
  if ((!kquant && type != T_Q4_0 && type != T_Q8_0) || M > (kquant ? 32 : 16) || K % 256) return false;
  const int64_t pitch = w_pitch ? w_pitch : (int64_t)(K / 256) * direct_block_bytes(type);
  // (the blocks of the other formats are at even addresses anyway)
  if ((type == T_Q4_K || type == T_Q5_K) && (((uintptr_t)W & 15) || (pitch & 15))) return false;
  return direct16_plan(M, N, K, partial_bytes).gsplits != 0;
}

// Whether the kernel is the faster route for a call it can run.  The K-quants: always on the tile operator's side
// (against the staged 16-row tiles), and from five rows on against the streaming GEMV when the matrix has at least 8M
// weights (below that the GEMV's single launch wins: [1024,4096] 8 against 10 us).  Q4_0 and Q8_0, whose blocks make
// every 16-byte load unaligned, stream at 2.3 TB/s only: from nine rows on against the GEMV (eight rows of
// [14336,4096] take it 18 us, this kernel 22 and 30 us; sixteen rows 36 and 35 us), and against the staged tiles while
// K is not split over workgroups (Q4_0 [14336,4096] 21.8 against 24.0 us, [4096,4096] 10.6 against 13.7 us, but
// [28672,8192] 65 against 50 us) and, for Q8_0, up to 32M weights ([4096,4096] 12.1 against 14.2 us; [14336,4096] 30
// against 27 us).
bool rows16_direct_pays(int type, int M, int64_t N, int64_t K, bool against_gemv) {
  const bool kquant = type == T_Q4_K || type == T_Q5_K || type == T_Q6_K;
  if (against_gemv) return M >= (kquant ? 5 : 9) && N * K >= (8 << 20);
  if (kquant) return true;
  return M >= 9 && K <= 256 * kDirectMaxSb && (type != T_Q8_0 || N * K <= (32 << 20));
}

// Q4_K, Q5_K (W and its row pitch 16-byte aligned), Q6_K with at most 32 rows of X, Q4_0 or Q8_0 with at most 16;
// GGUF_NOT_TAKEN otherwise.
// gemv_sums: the GEMV operator's offset term (see GSUM) instead of the tile operator's.
int rows16_direct(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial, int64_t partial_bytes,
                  hipStream_t s, const LinearArgs& la, bool gemv_sums) {
  if (!rows16_direct_takes(W, la.w_pitch, type, M, N, K, partial_bytes)) return GGUF_NOT_TAKEN;
  const Direct16Plan p = direct16_plan(M, N, K, partial_bytes);
  if (type == T_Q6_K) {
    GGUF_DISPATCH_DTYPE(dtype, return (rows16_direct_typed<scalar_t, DIRECT_Q6_K>(W, ws, Y, M, N, K, partial, p, s, la, gemv_sums)));
    return GGUF_ERR_DTYPE;
  }
  if (type == T_Q4_0) {
    GGUF_DISPATCH_DTYPE(dtype, return (rows16_direct_typed<scalar_t, DIRECT_Q4_0>(W, ws, Y, M, N, K, partial, p, s, la, gemv_sums)));
    return GGUF_ERR_DTYPE;
  }
  if (type == T_Q8_0) {
    GGUF_DISPATCH_DTYPE(dtype, return (rows16_direct_typed<scalar_t, DIRECT_Q8_0>(W, ws, Y, M, N, K, partial, p, s, la, gemv_sums)));
    return GGUF_ERR_DTYPE;
  }
  if (type == T_Q5_K) {
    GGUF_DISPATCH_DTYPE(dtype, return (rows16_direct_typed<scalar_t, DIRECT_Q5_K>(W, ws, Y, M, N, K, partial, p, s, la, gemv_sums)));
    return GGUF_ERR_DTYPE;
  }
  GGUF_DISPATCH_DTYPE(dtype, return (rows16_direct_typed<scalar_t, DIRECT_Q4_K>(W, ws, Y, M, N, K, partial, p, s, la, gemv_sums)));
  return GGUF_ERR_DTYPE;
}

}  // namespace gguf
