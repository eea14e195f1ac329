// The a8 prefill GEMM on the half-precision MFMA engine: q8_1-quantized activations times GGUF weights, the
// reference's ggml_mul_mat_a8 semantics (gguf_kernel.cu:220-290) to within the operand roundings.  Kernel: mmq_h_core.h.
#include "mmq_h_core.h"

namespace gguf {

// Tile size and the hand-out of tiles to workgroups for one launch (see MmqhPlan).
//   * The largest tile that still gives most CUs a workgroup: large tiles decode each weight block for more token
//     rows and read less LDS per MFMA; small ones fill the chip when M or N is small.
//   * When even the large tile leaves most CUs idle and K is long, the large tile is kept and every tile is split
//     along K instead.
//   * When the tiles fill the chip once or more but the last round of workgroups would be mostly empty, the tiles of
//     that round are split along K, so that the round is short instead of sparse.
// Splitting needs fp32 scratch in the workspace; without it the plan falls back to whole tiles.
MmqhPlan mmq_half_plan(int M, int N, int K, int64_t avail) {
  constexpr int CUS = 256;
  static const int MT[4] = {256, 128, 128, 64}, NT[4] = {128, 128, 64, 64};
  const auto tiles = [&](int c) { return (int64_t)((M + MT[c] - 1) / MT[c]) * ((N + NT[c] - 1) / NT[c]); };
  const int nsteps = (K + 63) / 64;
  const int big = M > 128 ? 0 : 1;
  MmqhPlan p = {3, 0, 0, 1};
  if (M <= 64) {
    // A handful of tokens: the weights are read once and little is computed, so what counts is how many independent
    // streams of weight blocks are in flight.  Small tiles, four workgroups per CU, K split as far as that fills them.
    const int64_t t = tiles(3);
    int s = t > 0 ? (int)(4 * CUS / t) : 1;
    if (s > nsteps / 4) s = nsteps / 4;
    if (s > 8) s = 8;
    p = MmqhPlan{3, 0, (int)t, s};
    if (s >= 2 && p.partial_bytes() <= avail) return p;
    return MmqhPlan{3, (int)t, 0, 1};
  }
  const int64_t tb = tiles(big);
  if (tb < 180 && tb > 0) {                     // too few tiles: split them all
    int s = (int)(CUS / tb);
    if (s > nsteps / 16) s = nsteps / 16;
    if (s > 8) s = 8;
    p = MmqhPlan{big, 0, (int)tb, s};
    if (s >= 2 && p.partial_bytes() <= avail) return p;
  }
  int cfg = 3;
  for (int c = big; c < 4; ++c)
    if (tiles(c) >= 180) { cfg = c; break; }
  const int64_t t = tiles(cfg);
  p = MmqhPlan{cfg, (int)t, 0, 1};
  const int slots = cfg == 0 ? CUS : 2 * CUS;   // workgroups the chip holds at once: one 256x128 tile per CU, two of 128x128
  if (cfg <= 1 && t > slots) {                  // look at the last round
    const int rest = (int)(t % slots);
    int s = rest ? slots / rest : 1;
    if (s > nsteps / 8) s = nsteps / 8;
    if (s > 8) s = 8;
    if (s >= 2) {
      const MmqhPlan q = {cfg, (int)(t - rest), rest, s};
      if (q.partial_bytes() <= avail) return q;
    }
  }
  return p;
}

template <class F>
static int mmqh_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, float* partial, int64_t partial_bytes,
                    hipStream_t s, const LinearArgs& la) {
  if (dtype == GGUF_DTYPE_F16) return mmqh_typed<A8Codes<F>, _Float16>(W, ws, Y, M, N, K, partial, partial_bytes, s, la);
  if (dtype == GGUF_DTYPE_BF16) return mmqh_typed<A8Codes<F>, bf16_t>(W, ws, Y, M, N, K, partial, partial_bytes, s, la);
  return GGUF_ERR_DTYPE;
}

// The half-MFMA engine for one call; the workspace already holds the quantized rows and, behind them, their half plane.
int mmq_half(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial,
             int64_t partial_bytes, hipStream_t s, const LinearArgs& la) {
  switch (type) {
    case T_Q4_0: return mmqh_fmt<MQ4_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_0: return mmqh_fmt<MQ5_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q8_0: return mmqh_fmt<MQ8_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q2_K: return mmqh_fmt<MQ2_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q3_K: return mmqh_fmt<MQ3_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q4_K: return mmqh_fmt<MQ4_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_K: return mmqh_fmt<MQ5_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_IQ4_XS: return mmqh_fmt<MIQ4_XS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_IQ2_XXS: return mmqh_fmt<MIQ2_XXS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q6_K: return mmqh_fmt<MQ6_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
  }
  return GGUF_ERR_TYPE;
}

// fp32 scratch the plan for this shape would use, given all the room it wants
int64_t mmq_half_partial_bytes(int M, int N, int K) { return mmq_half_plan(M, N, K, INT64_MAX).partial_bytes(); }

bool mmq_half_supported(int type) {
  switch (type) {
    case T_Q4_0: case T_Q5_0: case T_Q8_0: case T_Q2_K: case T_Q3_K: case T_Q4_K: case T_Q5_K: case T_Q6_K: case T_IQ4_XS:
    case T_IQ2_XXS: return true;
    default: return false;  // Q4_1 / Q5_1 round their scale products to half in the reference; they stay on the int8 engine
  }
}

}  // namespace gguf
