// The a8 prefill GEMM on the integer engine: q8_1-quantized activations times GGUF weights with exact int8 dot
// products and fp32 block scales, the reference's ggml_mul_mat_a8 arithmetic (gguf_kernel.cu:220-290, mmq.cuh:2-104).
// Kernel: mmq_i_core.h.
#include "mmq_i_core.h"

namespace gguf {

// Tile shape and the hand-out of tiles to workgroups for one launch (see MmqiPlan).  Two workgroups fit a CU, so the
// chip holds 512 at once.
//   * 128 x 64 tiles (the packed blocks of 64 weight rows are decoded once per 128 token rows); 64 x 128 for M <= 64.
//   * Fewer tiles than the chip holds: every tile is split along K as far as that fills it (three ways when the
//     tiles fill between half and two thirds of it).
//   * More: whole rounds of tiles run unsplit, and the tiles of the last, partly filled round are split so that the
//     round is short instead of sparse.
// Splitting needs fp32 scratch behind the quantized rows; without it the plan falls back to whole tiles.
MmqiPlan mmq_int_plan(int M, int N, int K, int64_t avail) {
  constexpr int SLOTS = 512;
  const int cfg = M > 64 ? 0 : 1;
  const int mt = cfg == 0 ? 128 : 64, nt = cfg == 0 ? 64 : 128;
  const int64_t t = (int64_t)((M + mt - 1) / mt) * ((N + nt - 1) / nt);
  const int nsteps = (K + MMQI_KS - 1) / MMQI_KS;
  const MmqiPlan whole = {cfg, (int)t, 0, 1};
  const int rest = (int)(t % SLOTS);
  if (rest == 0 || t <= 0) return whole;
  int s = SLOTS / rest;
  // a round between half and two thirds full: split three ways it becomes two full rounds of a third the length
  // (Q6_K [18944,3584] at 128 rows, 296 tiles: 85.5 -> 78 us; four ways 77, five 82 us)
  if (s == 1 && 3 * rest <= 2 * SLOTS) s = 3;
  if (s > nsteps / 4) s = nsteps / 4;   // a stretch of K shorter than four steps is mostly prologue
  if (s > 8) s = 8;
  if (s < 2) return whole;
  const MmqiPlan p = {cfg, (int)(t - rest), rest, s};
  return p.partial_bytes() <= avail ? p : whole;
}

int64_t mmq_int_partial_bytes(int M, int N, int K) { return mmq_int_plan(M, N, K, INT64_MAX).partial_bytes(); }

template <class F>
static int mmqi_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, float* partial, int64_t partial_bytes,
                    hipStream_t s, const LinearArgs& la) {
  GGUF_DISPATCH_DTYPE(dtype, return (mmqi_typed<F, scalar_t>(W, ws, Y, M, N, K, partial, partial_bytes, s, la)));
  return GGUF_ERR_DTYPE;
}

// The integer engine for one call; the workspace already holds the quantized rows.  GGUF_NOT_TAKEN for the formats
// whose scale products follow other rules (Q4_1 / Q5_1: rounded to half; Q2_K: offsets per 16 values).
int mmq_int(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial,
            int64_t partial_bytes, hipStream_t s, const LinearArgs& la) {
  switch (type) {
    case T_Q4_0: return mmqi_fmt<MQ4_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_0: return mmqi_fmt<MQ5_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q8_0: return mmqi_fmt<MQ8_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q3_K: return mmqi_fmt<MQ3_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q4_K: return mmqi_fmt<MQ4_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_K: return mmqi_fmt<MQ5_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q6_K: return mmqi_fmt<MQ6_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_IQ4_XS: return mmqi_fmt<MIQ4_XS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_IQ2_XXS: return mmqi_fmt<MIQ2_XXS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
  }
  return GGUF_NOT_TAKEN;
}

}  // namespace gguf

