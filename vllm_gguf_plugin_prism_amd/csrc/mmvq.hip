// C entry points of the decode-path GEMV and of the per-pair MoE GEMV.  The kernels live in mmvq_core.h and are
// instantiated per group of formats in the mmvq_<group>.hip files; this file validates and routes by ggml type.
#include "gguf_common.h"

namespace gguf {

int mmvq_group_std_a(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);
int mmvq_group_std_b(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);
int mmvq_group_k_a(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);
int mmvq_group_k_b(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);
int mmvq_group_iq_a(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);
int mmvq_group_iq_b(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);
int mmvq_group_iq_c(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la);

int moe_vec_group_std_a(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);
int moe_vec_group_std_b(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);
int moe_vec_group_k_a(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);
int moe_vec_group_k_b(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);
int moe_vec_group_iq_a(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);
int moe_vec_group_iq_b(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);
int moe_vec_group_iq_c(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s);

}  // namespace gguf

namespace gguf {
// one GEMV call after validation; with la.tile_sums the result is GGUF_NOT_TAKEN where the streaming kernel does not apply
// rows16_direct.hip: 16-row MFMA tiles read straight from the packed blocks (Q4_K, Q5_K, Q6_K)
bool rows16_direct_takes(const void* W, int64_t w_pitch, int type, int M, int N, int K, int64_t partial_bytes);
bool rows16_direct_pays(int type, int M, int64_t N, int64_t K, bool against_gemv);
int rows16_direct(const void* W, const void* ws, void* Y, int dtype, int type, int M, int N, int K, float* partial, int64_t partial_bytes,
                  hipStream_t s, const LinearArgs& la, bool gemv_sums);

int mmvq_any(int type, const void* W, const void* x, void* q8_workspace, void* Y, int xdtype, int64_t N, int64_t K, int64_t M,
             hipStream_t s, const LinearArgs& la) {
  // Five rows or more (nine for Q4_0 / Q8_0) of a matrix of at least 8M weights: the tile kernel's time does not grow
  // with the rows (up to 16 or 32 per launch), the streaming kernel's does (Q4_K [14336,4096] at 8 / 16 rows 22 / 42 us
  // against 17 us, Q6_K 36 / 71 against 27 us, Q4_0 at 16 rows 36 against 22 us).  The operator's workspace holds the quantized rows and nothing else, so K up to 4096 (beyond that
  // the tile kernel wants room for partial tiles).  The arithmetic stays the GEMV's (offset term on d8 * sum(q8)).
  if (!la.tile_sums && N <= 0x7FFFFFF0LL && K <= 0x7FFFFFF0LL && rows16_direct_pays(type, (int)(M < 16 ? M : 16), N, K, true) &&
      rows16_direct_takes(W, la.w_pitch, type, 16, (int)N, (int)K, 0)) {
    int rc = quantize_q8_1(x, xdtype, q8_workspace, M, K, s);
    if (rc != GGUF_OK) return rc;
    const int64_t ldy = la.ldy ? la.ldy : N, esz = xdtype == GGUF_DTYPE_F32 ? 4 : 2;
    const int step = rows16_direct_takes(W, la.w_pitch, type, 32, (int)N, (int)K, 0) ? 32 : 16;   // (the K-quants take 32 rows per launch)
    for (int64_t m0 = 0; m0 < M; m0 += step) {
      const int rows = (int)(M - m0 < step ? M - m0 : step);
      rc = rows16_direct(W, (const char*)q8_workspace + m0 * q8_row_bytes(K), (char*)Y + m0 * ldy * esz, xdtype, type, rows, (int)N, (int)K,
                         nullptr, 0, s, la, true);
      // takes() was asked for a full chunk above; a chunk the tile kernel then declines is a planning error, never a
      // result the caller should see as the internal "not taken" code with part of Y written
      if (rc == GGUF_NOT_TAKEN) return GGUF_ERR_LAUNCH;
      if (rc != GGUF_OK) return rc;
    }
    return GGUF_OK;
  }
  switch (type) {
    case T_Q4_0: return mmvq_group_std_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q4_1: return mmvq_group_std_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q8_0: return mmvq_group_std_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q5_0: return mmvq_group_std_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q5_1: return mmvq_group_std_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ4_NL: return mmvq_group_std_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q2_K: return mmvq_group_k_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q3_K: return mmvq_group_k_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q6_K: return mmvq_group_k_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q4_K: return mmvq_group_k_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_Q5_K: return mmvq_group_k_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ4_XS: return mmvq_group_iq_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ2_XXS: return mmvq_group_iq_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ3_XXS: return mmvq_group_iq_a(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ2_XS: return mmvq_group_iq_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ2_S: return mmvq_group_iq_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ3_S: return mmvq_group_iq_b(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ1_S: return mmvq_group_iq_c(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
    case T_IQ1_M: return mmvq_group_iq_c(type, W, x, q8_workspace, Y, xdtype, N, K, M, s, la);
  }
  return GGUF_ERR_TYPE;
}
}  // namespace gguf

extern "C" int gguf_mmvq_linear(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                                int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M,
                                gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (N < 0 || M < 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  if (w_row_pitch_bytes < K / qk * block_bytes(type) || y_row_pitch < N) return GGUF_ERR_SHAPE;
  LinearArgs la;
  la.w_pitch = w_row_pitch_bytes;
  la.ldy = y_row_pitch;
  la.bias = bias;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || M == 0) return GGUF_OK;
  if (!W || !x || !q8_workspace || !Y) return GGUF_ERR_NULL;
  // packed blocks sit at even addresses (every block size is even): the GEMV's block loads rely on it
  if (((uintptr_t)W & 1) || (w_row_pitch_bytes & 1)) return GGUF_ERR_SHAPE;
  return mmvq_any(type, W, x, q8_workspace, Y, xdtype, N, K, M, (hipStream_t)stream, la);
}

extern "C" int gguf_mmvq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N,
                         int64_t K, int64_t M, gguf_stream_t stream) {
  const int qk = gguf::block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (K <= 0 || K % qk != 0) return GGUF_ERR_SHAPE;
  return gguf_mmvq_linear(W, K / qk * gguf::block_bytes(type), x, xdtype, q8_workspace, Y, N, nullptr, type, N, K, M, stream);
}

extern "C" int gguf_moe_vec_act(const void* X, int xdtype, void* q8_workspace, const void* W, const int32_t* topk_ids,
                                void* Y, int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens, int act,
                                int64_t num_experts, int64_t workspace_bytes, gguf_stream_t stream);

namespace gguf {
// mmq.hip: the same operator on the grouped tile kernel, for calls whose experts are shared by enough pairs
bool moe_vec_tiles_ok(int type, int64_t pairs, int64_t num_experts, int64_t expert_bytes);
int64_t moe_vec_tiles_workspace(int64_t tokens, int64_t top_k, int64_t K, int64_t num_experts);
int moe_vec_tiles(const void* X, int xdtype, void* workspace, const void* W, const int32_t* topk_ids, void* Y, int type, int N,
                  int K, int top_k, int tokens, int act, int num_experts, hipStream_t s);
}  // namespace gguf

extern "C" int64_t gguf_moe_vec_workspace_bytes(int64_t tokens, int64_t top_k, int64_t K, int64_t num_experts) {
  if (tokens < 0 || top_k <= 0 || K <= 0 || num_experts < 0) return 0;
  const int64_t sorted_cap = tokens * top_k + num_experts * 7;  // room for groups of up to eight pairs per expert block
  const int64_t vec = tokens * gguf::q8_row_bytes(K) + (sorted_cap + (sorted_cap + 3) / 4 + 1) * 4;
  const int64_t tiles = gguf::moe_vec_tiles_workspace(tokens, top_k, K, num_experts);   // blocks of 32 pairs per expert
  return vec > tiles ? vec : tiles;
}

extern "C" int gguf_moe_vec(const void* X, int xdtype, void* q8_workspace, const void* W, const int32_t* topk_ids, void* Y,
                            int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens, gguf_stream_t stream) {
  return gguf_moe_vec_act(X, xdtype, q8_workspace, W, topk_ids, Y, type, N, K, top_k, tokens, 0, 0, 0, stream);
}

extern "C" int gguf_moe_vec_act(const void* X, int xdtype, void* q8_workspace, const void* W, const int32_t* topk_ids,
                                void* Y, int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens, int act,
                                int64_t num_experts, int64_t workspace_bytes, gguf_stream_t stream) {
  using namespace gguf;
  if (act < 0 || act > 2) return GGUF_ERR_SHAPE;
  const int qk = block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (N < 0 || tokens < 0 || top_k <= 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL ||
      tokens * top_k > 0x7FFFFFF0LL)
    return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || tokens == 0) return GGUF_OK;
  if (!X || !q8_workspace || !W || !topk_ids || !Y) return GGUF_ERR_NULL;
  if ((uintptr_t)W & 1) return GGUF_ERR_SHAPE;  // packed blocks sit at even addresses
  hipStream_t s = (hipStream_t)stream;
  const int pairs = (int)(tokens * top_k);
  const int ne = num_experts > 0 && num_experts <= 1024 ? (int)num_experts : 0;
  // the workspace holds at least the quantized activations; a caller that provides more says so
  const int64_t scratch_bytes = workspace_bytes > tokens * q8_row_bytes(K) ? workspace_bytes : tokens * q8_row_bytes(K);
  if (ne > 0 && moe_vec_tiles_ok(type, pairs, ne, N * (K / qk) * block_bytes(type)) &&
      scratch_bytes >= moe_vec_tiles_workspace(tokens, top_k, K, ne))
    return moe_vec_tiles(X, xdtype, q8_workspace, W, topk_ids, Y, type, (int)N, (int)K, (int)top_k, (int)tokens, act, ne, s);
  switch (type) {
    case T_Q4_0: return moe_vec_group_std_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q4_1: return moe_vec_group_std_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q8_0: return moe_vec_group_std_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q5_0: return moe_vec_group_std_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q5_1: return moe_vec_group_std_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ4_NL: return moe_vec_group_std_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q2_K: return moe_vec_group_k_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q3_K: return moe_vec_group_k_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q6_K: return moe_vec_group_k_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q4_K: return moe_vec_group_k_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_Q5_K: return moe_vec_group_k_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ4_XS: return moe_vec_group_iq_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ2_XXS: return moe_vec_group_iq_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ3_XXS: return moe_vec_group_iq_a(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ2_XS: return moe_vec_group_iq_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ2_S: return moe_vec_group_iq_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ3_S: return moe_vec_group_iq_b(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ1_S: return moe_vec_group_iq_c(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
    case T_IQ1_M: return moe_vec_group_iq_c(type, W, X, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, act, ne, q8_workspace, scratch_bytes, s);
  }
  return GGUF_ERR_TYPE;
}
