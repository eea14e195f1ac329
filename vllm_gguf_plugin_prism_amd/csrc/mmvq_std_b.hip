// GEMV and per-pair MoE GEMV instantiations for Q5_0, Q5_1, IQ4_NL (one translation unit per group of formats so
// that the groups compile in parallel).  Returns GGUF_ERR_TYPE for a type outside the group.
#include "mmvq_core.h"

namespace gguf {

int mmvq_group_std_b(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la) {
  switch (type) {
    case T_Q5_0: return mmvq_fmt<FmtQ5_0>(W, x, ws, Y, dtype, N, K, M, s, la);
    case T_Q5_1: return mmvq_fmt<FmtQ5_1>(W, x, ws, Y, dtype, N, K, M, s, la);
    case T_IQ4_NL: return mmvq_fmt<FmtIQ4_NL>(W, x, ws, Y, dtype, N, K, M, s, la);
    default: return GGUF_ERR_TYPE;
  }
}

int moe_vec_group_std_b(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s) {
  switch (type) {
    case T_Q5_0: return moe_vec_fmt<FmtQ5_0>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    case T_Q5_1: return moe_vec_fmt<FmtQ5_1>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    case T_IQ4_NL: return moe_vec_fmt<FmtIQ4_NL>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    default: return GGUF_ERR_TYPE;
  }
}

}  // namespace gguf
