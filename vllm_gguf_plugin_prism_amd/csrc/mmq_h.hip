// The a8 prefill GEMM on the half-precision MFMA engine: q8_1-quantized activations times GGUF weights, the
// reference's ggml_mul_mat_a8 semantics (gguf_kernel.cu:220-290) to within the operand roundings.  Kernel: mmq_h_core.h.
#include "mmq_h_core.h"

namespace gguf {

// Number of K splits the half engine would like for this shape (1 = none): enough to give every CU a workgroup of the
// large tile, every split keeping at least 16 steps of 64 elements.
int mmq_half_splits(int M, int N, int K) {
  const int mt = M > 128 ? 256 : 128;
  const int64_t tiles = (int64_t)((M + mt - 1) / mt) * ((N + 127) / 128);
  if (tiles >= 180 || tiles == 0) return 1;
  int s = (int)(256 / tiles);
  const int by_k = (K / 64) / 16;
  if (s > by_k) s = by_k;
  if (s > 8) s = 8;
  return s < 2 ? 1 : s;
}

template <class F>
static int mmqh_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, float* partial, int64_t partial_bytes,
                    hipStream_t s) {
  if (dtype == GGUF_DTYPE_F16) return mmqh_typed<A8Codes<F>, _Float16>(W, ws, Y, M, N, K, partial, partial_bytes, s);
#ifndef GGUF_MMQ_TUNE
  if (dtype == GGUF_DTYPE_BF16) return mmqh_typed<A8Codes<F>, bf16_t>(W, ws, Y, M, N, K, partial, partial_bytes, s);
#endif
  return GGUF_ERR_DTYPE;
}

// The half-MFMA engine for one call; the workspace already holds the quantized rows and, behind them, their half plane.
int mmq_half(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial,
             int64_t partial_bytes, hipStream_t s) {
  switch (type) {
#ifndef GGUF_MMQ_TUNE
    case T_Q4_0: return mmqh_fmt<MQ4_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_Q5_0: return mmqh_fmt<MQ5_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_Q8_0: return mmqh_fmt<MQ8_0>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_Q2_K: return mmqh_fmt<MQ2_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_Q3_K: return mmqh_fmt<MQ3_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_Q4_K: return mmqh_fmt<MQ4_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_Q5_K: return mmqh_fmt<MQ5_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_IQ4_XS: return mmqh_fmt<MIQ4_XS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
    case T_IQ2_XXS: return mmqh_fmt<MIQ2_XXS>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
#endif
    case T_Q6_K: return mmqh_fmt<MQ6_K>(W, ws, Y, dtype, M, N, K, partial, partial_bytes, s);
  }
  return GGUF_ERR_TYPE;
}

bool mmq_half_supported(int type) {
  switch (type) {
    case T_Q4_0: case T_Q5_0: case T_Q8_0: case T_Q2_K: case T_Q3_K: case T_Q4_K: case T_Q5_K: case T_Q6_K: case T_IQ4_XS:
    case T_IQ2_XXS: return true;
    default: return false;  // Q4_1 / Q5_1 round their scale products to half in the reference; they stay on the int8 engine
  }
}

}  // namespace gguf
