// The torch operator library `_C_gguf` over the C ABI of libgguf_hip.so, compiled: the six schemas of the reference's
// csrc/torch_bindings.cpp:22-40 with its dispatch keys (:42-53: CUDA, which HIP tensors dispatch on, and
// CompositeExplicitAutograd for the block-size query).  Per call it allocates the result and the workspace with torch,
// takes torch's current stream and passes raw pointers on -- what vllm_gguf_plugin_prism_amd/ops.py does in Python, minus
// the interpreter (about 4 us of host time per call).  Host code only: built with the C++ compiler against torch's
// headers, linked against libgguf_hip.so beside it.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <algorithm>
#include <optional>

#include "gguf_hip.h"

namespace {

int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return GGUF_DTYPE_F32;
    case at::kHalf: return GGUF_DTYPE_F16;
    case at::kBFloat16: return GGUF_DTYPE_BF16;
    default: TORCH_CHECK(false, "unsupported dtype ", t, "; need float32, float16 or bfloat16");
  }
}

void check(int rc, const char* what) {
  if (rc == GGUF_OK) return;
  TORCH_CHECK_NOT_IMPLEMENTED(rc != GGUF_ERR_TYPE, what, ": ggml type not supported by this entry point");
  TORCH_CHECK(false, what, ": error ", rc, " from libgguf_hip (see gguf_hip.h)");
}

void need_contiguous(const at::Tensor& t, const char* name) { TORCH_CHECK(t.is_contiguous(), "GGUF ops need contiguous tensors: ", name); }

gguf_stream_t stream_of(const at::Tensor& t) { return (gguf_stream_t)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.get_device()).stream(); }

at::Tensor workspace(const at::Tensor& like, int64_t bytes) {
  return at::empty({std::max<int64_t>(bytes, 16)}, like.options().dtype(at::kByte));
}

at::Tensor ggml_dequantize(const at::Tensor& W, int64_t type, int64_t m, int64_t n, std::optional<at::ScalarType> dtype) {
  need_contiguous(W, "W");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(W.device());
  const at::ScalarType out_dtype = dtype.value_or(at::kHalf);
  at::Tensor out = at::empty({m, n}, W.options().dtype(out_dtype));
  check(gguf_dequantize(W.data_ptr(), (int)type, out.data_ptr(), dtype_code(out_dtype), m * n, stream_of(W)), "ggml_dequantize");
  return out;
}

at::Tensor ggml_mul_mat_vec_a8(const at::Tensor& W, const at::Tensor& X, int64_t type, int64_t row) {
  need_contiguous(W, "W");
  need_contiguous(X, "X");
  TORCH_CHECK(X.dim() == 2, "X must be [vectors, K]");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(X.device());
  const int64_t vecs = X.size(0), col = X.size(1);
  at::Tensor out = at::empty({vecs, row}, X.options());
  at::Tensor ws = workspace(X, vecs * gguf_q8_1_row_bytes(col));
  check(gguf_mmvq(W.data_ptr(), X.data_ptr(), dtype_code(X.scalar_type()), ws.data_ptr(), out.data_ptr(), (int)type, row, col, vecs, stream_of(X)),
        "ggml_mul_mat_vec_a8");
  return out;
}

at::Tensor ggml_mul_mat_a8(const at::Tensor& W, const at::Tensor& X, int64_t type, int64_t row) {
  need_contiguous(W, "W");
  need_contiguous(X, "X");
  TORCH_CHECK(X.dim() == 2, "X must be [tokens, K]");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(X.device());
  const int64_t vecs = X.size(0), col = X.size(1);
  at::Tensor out = at::empty({vecs, row}, X.options());
  const int64_t bytes = std::max<int64_t>(gguf_mmq_workspace_bytes_engine(vecs, row, col, GGUF_MMQ_AUTO), 16);
  at::Tensor ws = workspace(X, bytes);
  check(gguf_mmq_engine(W.data_ptr(), X.data_ptr(), dtype_code(X.scalar_type()), ws.data_ptr(), out.data_ptr(), (int)type, row, col, vecs,
                        GGUF_MMQ_AUTO, bytes, stream_of(X)),
        "ggml_mul_mat_a8");
  return out;
}

at::Tensor ggml_moe_a8(const at::Tensor& X, const at::Tensor& W, const at::Tensor& sorted_token_ids, const at::Tensor& expert_ids,
                       const at::Tensor& num_tokens_post_padded, int64_t type, int64_t row, int64_t top_k, int64_t tokens) {
  for (const at::Tensor* t : {&X, &W, &sorted_token_ids, &expert_ids, &num_tokens_post_padded}) need_contiguous(*t, "an argument of ggml_moe_a8");
  for (const at::Tensor* t : {&sorted_token_ids, &expert_ids, &num_tokens_post_padded})
    TORCH_CHECK(t->scalar_type() == at::kInt, "MoE index tensors must be int32");
  TORCH_CHECK(X.dim() == 2 && W.dim() == 3, "X must be [tokens, K] and W [experts, row, bytes]");
  // the kernel keeps the reference's guard on expert ids (moe.cuh:33): refuse rather than return a result with holes
  TORCH_CHECK_NOT_IMPLEMENTED(W.size(0) <= 256, "ggml_moe_a8 takes at most 256 experts, got ", W.size(0));
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(X.device());
  const int64_t col = X.size(1);
  at::Tensor out = at::empty({tokens * top_k, row}, X.options());
  at::Tensor ws = workspace(X, tokens * gguf_q8_1_row_bytes(col));
  check(gguf_moe_mmq_block(X.data_ptr(), dtype_code(X.scalar_type()), ws.data_ptr(), W.data_ptr(), W.stride(0) * (int64_t)W.element_size(),
                           sorted_token_ids.data_ptr<int32_t>(), expert_ids.data_ptr<int32_t>(), num_tokens_post_padded.data_ptr<int32_t>(),
                           sorted_token_ids.size(0), out.data_ptr(), (int)type, row, col, top_k, tokens, 0, gguf_moe_block_size((int)type),
                           W.size(0), stream_of(X)),
        "ggml_moe_a8");
  return out;
}

at::Tensor ggml_moe_a8_vec(const at::Tensor& X, const at::Tensor& W, const at::Tensor& topk_ids, int64_t top_k, int64_t type, int64_t row,
                           int64_t tokens) {
  for (const at::Tensor* t : {&X, &W, &topk_ids}) need_contiguous(*t, "an argument of ggml_moe_a8_vec");
  TORCH_CHECK(topk_ids.scalar_type() == at::kInt, "topk_ids must be int32");
  TORCH_CHECK(X.dim() == 2 && W.dim() == 3, "X must be [tokens, K] and W [experts, row, bytes]");
  const c10::hip::HIPGuardMasqueradingAsCUDA guard(X.device());
  const int64_t col = X.size(1);
  at::Tensor out = at::empty({tokens * top_k, row}, X.options());
  const int64_t bytes = std::max<int64_t>(gguf_moe_vec_workspace_bytes(tokens, top_k, col, W.size(0)), 16);   // quantized rows + routing sort
  at::Tensor ws = workspace(X, bytes);
  check(gguf_moe_vec_act(X.data_ptr(), dtype_code(X.scalar_type()), ws.data_ptr(), W.data_ptr(), topk_ids.data_ptr<int32_t>(), out.data_ptr(),
                         (int)type, row, col, top_k, tokens, 0, W.size(0), bytes, stream_of(X)),
        "ggml_moe_a8_vec");
  return out;
}

int64_t ggml_moe_get_block_size(int64_t type) { return gguf_moe_block_size((int)type); }

}  // namespace

TORCH_LIBRARY(_C_gguf, m) {
  m.def("ggml_dequantize(Tensor W, int type, SymInt m, SymInt n, ScalarType? dtype) -> Tensor");
  m.def("ggml_mul_mat_vec_a8(Tensor W, Tensor X, int type, SymInt row) -> Tensor");
  m.def("ggml_mul_mat_a8(Tensor W, Tensor X, int type, SymInt row) -> Tensor");
  m.def(
      "ggml_moe_a8(Tensor X, Tensor W, Tensor sorted_token_ids, Tensor expert_ids, Tensor num_tokens_post_padded, "
      "int type, SymInt row, SymInt top_k, SymInt tokens) -> Tensor");
  m.def("ggml_moe_a8_vec(Tensor X, Tensor W, Tensor topk_ids, int top_k, int type, SymInt row, SymInt tokens) -> Tensor");
  m.def("ggml_moe_get_block_size(int type) -> int");
}

TORCH_LIBRARY_IMPL(_C_gguf, CUDA, m) {
  m.impl("ggml_dequantize", &ggml_dequantize);
  m.impl("ggml_mul_mat_vec_a8", &ggml_mul_mat_vec_a8);
  m.impl("ggml_mul_mat_a8", &ggml_mul_mat_a8);
  m.impl("ggml_moe_a8", &ggml_moe_a8);
  m.impl("ggml_moe_a8_vec", &ggml_moe_a8_vec);
}

TORCH_LIBRARY_IMPL(_C_gguf, CompositeExplicitAutograd, m) { m.impl("ggml_moe_get_block_size", &ggml_moe_get_block_size); }
