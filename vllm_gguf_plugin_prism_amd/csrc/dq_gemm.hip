// Y = X . dequant(W)^T without materialising the dense weights: the reference's fallback for formats and batch
// sizes that have no a8 kernel, `ggml_dequantize` followed by `x @ weight.T` (quantization/linear.py:50-58,
// diffusion_config.py:21-30), as one GEMM that decodes the packed blocks on the fly.  The activations are not
// quantized: X is multiplied as it is (converted to half precision), the weights are the half-precision values the
// reference's dequantize kernels produce.  Kernel: mmq_h_core.h with DqCodes.
#include "mmq_h_core.h"

namespace gguf {

// X[M][K] of any dtype -> half rows [M][pitch], zero beyond K (pitch = q8_half_pitch(K)); values past the half range saturate
template <typename T>
__global__ __launch_bounds__(256) void to_half_rows_kernel(const T* __restrict__ x, _Float16* __restrict__ xh, int K, int pitch) {
  const int64_t m = blockIdx.y;
  const int e0 = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (e0 >= pitch) return;
  v8h o;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int e = e0 + i;
    const float v = e < K ? to_f32<T>(x[m * K + e]) : 0.0f;
    o[i] = (_Float16)fminf(fmaxf(v, -65504.0f), 65504.0f);
  }
  *(v8h*)(xh + m * pitch + e0) = o;
}

template <class F>
static int dq_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, float* partial, int64_t partial_bytes,
                  hipStream_t s) {
  if (dtype == GGUF_DTYPE_F16) return mmqh_typed<DqCodes<F>, _Float16>(W, ws, Y, M, N, K, partial, partial_bytes, s);
  if (dtype == GGUF_DTYPE_BF16) return mmqh_typed<DqCodes<F>, bf16_t>(W, ws, Y, M, N, K, partial, partial_bytes, s);
  return GGUF_ERR_DTYPE;
}

static bool dq_type_ok(int type) {
  switch (type) {
    case T_Q4_0: case T_Q4_1: case T_Q5_0: case T_Q5_1: case T_Q8_0: case T_Q2_K: case T_Q3_K: case T_Q4_K: case T_Q5_K:
    case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: return true;
    default: return false;
  }
}

}  // namespace gguf

extern "C" int gguf_dequant_gemm(const void* W, const void* x, int xdtype, void* workspace, void* Y, int type, int64_t N,
                                 int64_t K, int64_t M, int64_t workspace_bytes, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0 || !dq_type_ok(type)) return GGUF_ERR_TYPE;
  if (N < 0 || M < 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL || M > 0x7FFFFFF0LL || workspace_bytes < 0)
    return GGUF_ERR_SHAPE;
  if (xdtype != GGUF_DTYPE_F16 && xdtype != GGUF_DTYPE_BF16) return GGUF_ERR_DTYPE;  // fp32 products are not what this engine forms
  if (N == 0 || M == 0) return GGUF_OK;
  if (!W || !x || !workspace || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  // same workspace layout as the a8 operator: the half rows sit behind the (here unused) quantized rows
  const int64_t rows_bytes = (M * (q8_row_bytes(K) + 2 * q8_half_pitch(K)) + 255) / 256 * 256;
  if (workspace_bytes < M * (q8_row_bytes(K) + 2 * q8_half_pitch(K))) return GGUF_ERR_WORKSPACE;
  _Float16* xh = (_Float16*)((char*)workspace + M * q8_row_bytes(K));
  const int pitch = (int)q8_half_pitch(K);
  const unsigned gx = (unsigned)((pitch / 8 + 255) / 256);
  for (int64_t off = 0; off < M; off += 65535) {
    const unsigned rows = (unsigned)((M - off) < 65535 ? (M - off) : 65535);
    if (xdtype == GGUF_DTYPE_F16)
      hipLaunchKernelGGL(to_half_rows_kernel<_Float16>, dim3(gx, rows), dim3(256), 0, s, (const _Float16*)x + off * K, xh + off * pitch, (int)K, pitch);
    else
      hipLaunchKernelGGL(to_half_rows_kernel<bf16_t>, dim3(gx, rows), dim3(256), 0, s, (const bf16_t*)x + off * K, xh + off * pitch, (int)K, pitch);
  }
  float* partial = (float*)((char*)workspace + rows_bytes);
  const int64_t partial_bytes = workspace_bytes > rows_bytes ? workspace_bytes - rows_bytes : 0;
  const int m = (int)M, n = (int)N, k = (int)K;
  switch (type) {
    case T_Q4_0: return dq_fmt<MQ4_0>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q4_1: return dq_fmt<MQ4_1>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q5_0: return dq_fmt<MQ5_0>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q5_1: return dq_fmt<MQ5_1>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q8_0: return dq_fmt<MQ8_0>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q2_K: return dq_fmt<MQ2_K>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q3_K: return dq_fmt<MQ3_K>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q4_K: return dq_fmt<MQ4_K>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q5_K: return dq_fmt<MQ5_K>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_Q6_K: return dq_fmt<MQ6_K>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_IQ4_XS: return dq_fmt<MIQ4_XS>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
    case T_IQ2_XXS: return dq_fmt<MIQ2_XXS>(W, workspace, Y, xdtype, m, n, k, partial, partial_bytes, s);
  }
  return GGUF_ERR_TYPE;
}
