// GEMV and per-pair MoE GEMV instantiations for Q4_0, Q4_1, Q8_0 (one translation unit per group of formats so
// that the groups compile in parallel).  Returns GGUF_ERR_TYPE for a type outside the group.
#include "mmvq_core.h"

namespace gguf {

int mmvq_group_std_a(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la) {
  switch (type) {
    case T_Q4_0: return mmvq_fmt<FmtQ4_0>(W, x, ws, Y, dtype, N, K, M, s, la);
    case T_Q4_1: return mmvq_fmt<FmtQ4_1>(W, x, ws, Y, dtype, N, K, M, s, la);
    case T_Q8_0: return mmvq_fmt<FmtQ8_0>(W, x, ws, Y, dtype, N, K, M, s, la);
    default: return GGUF_ERR_TYPE;
  }
}

int moe_vec_group_std_a(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s) {
  switch (type) {
    case T_Q4_0: return moe_vec_fmt<FmtQ4_0>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    case T_Q4_1: return moe_vec_fmt<FmtQ4_1>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    case T_Q8_0: return moe_vec_fmt<FmtQ8_0>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    default: return GGUF_ERR_TYPE;
  }
}

}  // namespace gguf
