// The a8 prefill GEMM on the integer engine: q8_1-quantized activations times GGUF weights with exact int8 dot
// products and fp32 block scales, the reference's ggml_mul_mat_a8 arithmetic (gguf_kernel.cu:220-290, mmq.cuh:2-104).
// Kernel: mmq_i_core.h.
#include "mmq_i_core.h"

namespace gguf {

// Tile shape and the hand-out of tiles to workgroups for one launch (see MmqiPlan).
//   * Four shapes.  128 x 64 on four waves, two workgroups per CU (the packed blocks of 64 weight rows are decoded once
//     per 128 token rows); 64 x 128 for M <= 64; 256 x 128 on eight waves, one workgroup per CU, a wave owning 32 x 128:
//     the activation scales a wave reads from LDS per block serve four column tiles instead of two and the weights are
//     decoded once per 256 rows (Q6_K [18944,3584] at 512 rows 229 -> 207 us, Q8_0 [14336,4096] 129 -> 112 us, IQ4_XS
//     130 -> 108 us; Q5_K's kernel of that shape spills and is left out); 128 x 64 on eight waves, one workgroup per CU,
//     for 65 .. 128 rows, where the larger tiles leave CUs without work.
//   * How a shape's tiles fall into rounds of the workgroups the chip holds decides between them: fewer tiles than the
//     chip holds are split along K as far as that fills it (three ways when they fill between half and two thirds of
//     it); with more, whole rounds of tiles run unsplit and the tiles of the last, partly filled round are split so
//     that the round is short instead of sparse.  The estimate is rounds x (steps of K + a start-up of about a step
//     and a half), weighted by what a step of the shape was measured to take.
// Splitting needs fp32 scratch behind the quantized rows; without it a plan falls back to whole tiles.
static MmqiPlan plan_for(int cfg, int slots, int M, int N, int K, int64_t avail) {
  MmqiPlan whole = {cfg, 0, 0, 1};
  const int64_t t = (int64_t)((M + whole.mt() - 1) / whole.mt()) * ((N + whole.nt() - 1) / whole.nt());
  const int nsteps = (K + MMQI_KS - 1) / MMQI_KS;
  whole.whole = (int)t;
  const int rest = (int)(t % slots);
  if (rest == 0 || t <= 0) return whole;
  int s = slots / rest;
  // a round between half and two thirds full: split three ways it becomes two full rounds of a third the length
  // (Q6_K [18944,3584] at 128 rows, 296 tiles of 128 x 64: 85.5 -> 78 us; four ways 77, five 82 us)
  if (s == 1 && 3 * rest <= 2 * slots) s = 3;
  if (s > nsteps / 4) s = nsteps / 4;   // a stretch of K shorter than four steps is mostly prologue
  if (s > 8) s = 8;
  if (s < 2) return whole;
  const MmqiPlan p = {cfg, (int)(t - rest), rest, s};
  return p.partial_bytes() <= avail ? p : whole;
}

static double plan_cost(const MmqiPlan& p, int slots, double step_cost, int K) {
  const int nsteps = (K + MMQI_KS - 1) / MMQI_KS;
  constexpr double START = 1.5;   // pipeline fill, result or partial-tile store: in steps
  double c = (double)((p.whole + slots - 1) / slots) * (nsteps + START);
  if (p.shared > 0) c += (double)((p.shared * p.splits + slots - 1) / slots) * ((nsteps + p.splits - 1) / p.splits + START) + 1.0;
  return c * step_cost;
}

MmqiPlan mmq_int_plan(int M, int N, int K, int64_t avail, bool wide_ok) {
  // workgroups the chip holds, and what a step of K costs relative to the 128 x 64 tiles (two workgroups share a CU
  // there: the figure is per round of workgroups)
  struct Shape { int cfg, slots; double step_cost; };
  if (M <= 64) return plan_for(1, 512, M, N, K, avail);
  MmqiPlan best = plan_for(0, 512, M, N, K, avail);
  double best_cost = plan_cost(best, 512, 1.0, K);
  auto consider = [&](const Shape& sh) {
    const MmqiPlan p = plan_for(sh.cfg, sh.slots, M, N, K, avail);
    const double c = plan_cost(p, sh.slots, sh.step_cost, K);
    if (c < 0.97 * best_cost) { best = p; best_cost = c; }
  };
  if (M <= 128) consider({3, 256, 0.6});
  // 256-row tiles when the rows fill them (M = 384 would multiply 128 rows of padding)
  if (wide_ok && M >= 448 && 20 * M >= 17 * ((M + 255) / 256 * 256)) consider({2, 256, 1.8});
  return best;
}

// (the workspace is sized without knowing the format: room for whichever shape a format may take)
int64_t mmq_int_partial_bytes(int M, int N, int K) {
  const int64_t a = mmq_int_plan(M, N, K, INT64_MAX, true).partial_bytes(), b = mmq_int_plan(M, N, K, INT64_MAX, false).partial_bytes();
  return a > b ? a : b;
}

template <class F>
static int mmqi_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, float* partial, int64_t partial_bytes,
                    hipStream_t s, const LinearArgs& la) {
  GGUF_DISPATCH_DTYPE(dtype, return (mmqi_typed<F, scalar_t>(W, ws, Y, M, N, K, partial, partial_bytes, s, la)));
  return GGUF_ERR_DTYPE;
}

// The integer engine for one call; the workspace already holds the quantized rows.  GGUF_NOT_TAKEN for types without
// tiles.  (Q4_1 / Q5_1 round their scale products to half, Q2_K subtracts an offset per 16 values: see rescale.)
int mmq_int(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial,
            int64_t partial_bytes, hipStream_t s, const LinearArgs& la) {
  switch (type) {
    case T_Q4_0: return mmqi_fmt<MQ4_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q4_1: return mmqi_fmt<MQ4_1>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q5_1: return mmqi_fmt<MQ5_1>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
    case T_Q2_K: return mmqi_fmt<MQ2_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s, la);
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

// The grouped MoE contraction on the integer engine, rows in slot order (mmq_i_core.h, MmqiMoe); blocks of 64 slots.
int mmq_int_moe(const void* W, const void* ws, void* Y, int dtype, int type, int slots, int N, int K, const int32_t* expert_ids,
                const int32_t* num_tokens_post_padded, int64_t expert_stride, int block, hipStream_t s) {
  if (block != 64) return GGUF_ERR_SHAPE;
  const MmqiMoe moe = {expert_ids, num_tokens_post_padded, expert_stride, block};
  switch (type) {
#define MMQI_MOE_CASE(ID, FMT) \
  case ID: GGUF_DISPATCH_DTYPE(dtype, return (mmqi_moe_typed<FMT, scalar_t>(W, ws, Y, slots, N, K, moe, s))); return GGUF_ERR_DTYPE;
    MMQI_MOE_CASE(T_Q4_0, MQ4_0) MMQI_MOE_CASE(T_Q4_1, MQ4_1) MMQI_MOE_CASE(T_Q5_0, MQ5_0) MMQI_MOE_CASE(T_Q5_1, MQ5_1)
    MMQI_MOE_CASE(T_Q8_0, MQ8_0) MMQI_MOE_CASE(T_Q2_K, MQ2_K) MMQI_MOE_CASE(T_Q3_K, MQ3_K) MMQI_MOE_CASE(T_Q4_K, MQ4_K)
    MMQI_MOE_CASE(T_Q5_K, MQ5_K) MMQI_MOE_CASE(T_Q6_K, MQ6_K) MMQI_MOE_CASE(T_IQ4_XS, MIQ4_XS) MMQI_MOE_CASE(T_IQ2_XXS, MIQ2_XXS)
#undef MMQI_MOE_CASE
  }
  return GGUF_NOT_TAKEN;
}

}  // namespace gguf

