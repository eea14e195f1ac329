// GEMV and per-pair MoE GEMV instantiations for IQ1_S, IQ1_M (one translation unit per group of formats so
// that the groups compile in parallel).  Returns GGUF_ERR_TYPE for a type outside the group.
#include "mmvq_core.h"

namespace gguf {

int mmvq_group_iq_c(int type, const void* W, const void* x, void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M,
                   hipStream_t s, const LinearArgs& la) {
  switch (type) {
    case T_IQ1_S: return mmvq_fmt<FmtIQ1_S>(W, x, ws, Y, dtype, N, K, M, s, la);
    case T_IQ1_M: return mmvq_fmt<FmtIQ1_M>(W, x, ws, Y, dtype, N, K, M, s, la);
    default: return GGUF_ERR_TYPE;
  }
}

int moe_vec_group_iq_c(int type, const void* W, const void* x, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                      int pairs, int act, int num_experts, void* scratch, int64_t scratch_bytes, hipStream_t s) {
  switch (type) {
    case T_IQ1_S: return moe_vec_fmt<FmtIQ1_S>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    case T_IQ1_M: return moe_vec_fmt<FmtIQ1_M>(W, x, Y, dtype, N, K, ids, top_k, pairs, act, num_experts, scratch, scratch_bytes, s);
    default: return GGUF_ERR_TYPE;
  }
}

}  // namespace gguf
