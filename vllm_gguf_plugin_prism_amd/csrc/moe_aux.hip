// Helpers at the caller seam of the MoE path: the routing sort that feeds the grouped kernel, and the
// top-k weighting + sum that follows the second expert GEMM.
//
// The reference takes both from vLLM (quantization/fused_moe.py:53-66: moe_align_block_size;
// :87-95: out.mul_(topk_weights) then ops.moe_sum); they are not part of its own native code.
#include "gguf_common.h"

namespace gguf {

constexpr int ALIGN_THREADS = 1024;
constexpr int ALIGN_WAVES = ALIGN_THREADS / 64;
constexpr int ALIGN_MAX_EXPERTS = 1024;

// One workgroup sorts the flat (token, choice) pairs by expert, stably, and pads every expert's run to a multiple
// of `block`:
//   sorted_ids[pos]  flat pair index, or `numel` in padding and unused slots
//   expert_ids[b]    expert of block b, -1 past the padded total
//   num_post_padded  padded total
// Stable order (ascending pair index inside a run) makes the result a pure function of the input.  Pairs are taken
// 1024 at a time; inside a chunk a pair's rank among equal experts is (same-expert pairs in earlier waves) +
// (same-expert lanes below it in its wave), the first from a per-wave histogram in LDS, the second from ballots.
__global__ __launch_bounds__(ALIGN_THREADS) void moe_align_kernel(const int32_t* __restrict__ topk_ids, int numel,
                                                                  int num_experts, int block,
                                                                  int32_t* __restrict__ sorted_ids, int sorted_capacity,
                                                                  int32_t* __restrict__ expert_ids, int expert_capacity,
                                                                  int32_t* __restrict__ num_post_padded) {
  extern __shared__ int lds[];
  int* start = lds;                          // [E] first slot of the expert's run, then its running cursor
  int* wave_cnt = lds + num_experts;         // [ALIGN_WAVES][E] per-wave histogram of the current chunk
  __shared__ int total_padded;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  for (int i = tid; i < sorted_capacity; i += ALIGN_THREADS) sorted_ids[i] = numel;
  for (int e = tid; e < num_experts; e += ALIGN_THREADS) start[e] = 0;
  __syncthreads();
  for (int i = tid; i < numel; i += ALIGN_THREADS) {
    const int e = topk_ids[i];
    if (e >= 0 && e < num_experts) atomicAdd(&start[e], 1);  // counts: the sum does not depend on the order of adds
  }
  __syncthreads();
  if (tid == 0) {
    int pos = 0;
    for (int e = 0; e < num_experts; ++e) {
      const int padded = (start[e] + block - 1) / block * block;
      start[e] = pos;
      pos += padded;
    }
    total_padded = pos;
    num_post_padded[0] = pos;
  }
  __syncthreads();
  // expert of every block: expert e owns blocks [start[e], start[e+1]) / block
  for (int e = tid; e < num_experts; e += ALIGN_THREADS) {
    const int end = e + 1 < num_experts ? start[e + 1] : total_padded;
    for (int b = start[e] / block; b < end / block && b < expert_capacity; ++b) expert_ids[b] = e;
  }
  for (int b = total_padded / block + tid; b < expert_capacity; b += ALIGN_THREADS) expert_ids[b] = -1;

  for (int c0 = 0; c0 < numel; c0 += ALIGN_THREADS) {
    for (int i = tid; i < ALIGN_WAVES * num_experts; i += ALIGN_THREADS) wave_cnt[i] = 0;
    __syncthreads();
    const int i = c0 + tid;
    int e = i < numel ? topk_ids[i] : -1;
    if (e >= num_experts) e = -1;
    // rank among the lanes of this wave with the same expert, and this wave's count of it
    int rank_in_wave = 0;
    unsigned long long todo = __ballot(e >= 0);
    while (todo) {
      const int leader = __ffsll((long long)todo) - 1;
      const int e0 = __shfl(e, leader);
      const unsigned long long same = __ballot(e == e0);
      if (e == e0) {
        rank_in_wave = __popcll(same & ((1ull << lane) - 1));
        if (lane == leader) wave_cnt[wave * num_experts + e0] = __popcll(same);
      }
      todo &= ~same;
    }
    __syncthreads();
    if (e >= 0) {
      int before = 0;
      for (int w = 0; w < wave; ++w) before += wave_cnt[w * num_experts + e];
      const int pos = start[e] + before + rank_in_wave;
      if (pos < sorted_capacity) sorted_ids[pos] = i;
    }
    __syncthreads();
    for (int ee = tid; ee < num_experts; ee += ALIGN_THREADS) {
      int sum = 0;
      for (int w = 0; w < ALIGN_WAVES; ++w) sum += wave_cnt[w * num_experts + ee];
      start[ee] += sum;
    }
    __syncthreads();
  }
}

// out[t, n] = sum_k  T( float(Y[t, k, n]) * w[t, k] )   accumulated in fp32 in the order k = 0 .. top_k-1 and rounded
// once: the in-place multiply by the routing weights followed by the sum over the top-k axis.
template <typename T>
__global__ __launch_bounds__(256) void moe_weighted_sum_kernel(const T* __restrict__ Y, const float* __restrict__ w,
                                                               T* __restrict__ out, int top_k, int64_t N) {
  const int64_t t = blockIdx.y;
  for (int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x; n < N; n += (int64_t)gridDim.x * 256) {
    float acc = 0.0f;
    for (int k = 0; k < top_k; ++k) {
      const T p = from_f32<T>(to_f32<T>(Y[(t * top_k + k) * N + n]) * w[t * top_k + k]);
      acc += to_f32<T>(p);
    }
    out[t * N + n] = from_f32<T>(acc);
  }
}

}  // namespace gguf

extern "C" int gguf_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int64_t num_experts, int64_t block,
                                         int32_t* sorted_token_ids, int64_t sorted_capacity, int32_t* expert_ids,
                                         int64_t expert_capacity, int32_t* num_tokens_post_padded, gguf_stream_t stream) {
  using namespace gguf;
  if (numel < 0 || num_experts <= 0 || num_experts > ALIGN_MAX_EXPERTS || block <= 0 || numel > 0x3FFFFFFFLL) return GGUF_ERR_SHAPE;
  // every expert may need up to block-1 padding slots
  const int64_t need = numel + num_experts * (block - 1);
  if (sorted_capacity < need || sorted_capacity > 0x7FFFFFF0LL || expert_capacity < (need + block - 1) / block ||
      expert_capacity > 0x7FFFFFF0LL)
    return GGUF_ERR_SHAPE;
  if (!sorted_token_ids || !expert_ids || !num_tokens_post_padded || (numel > 0 && !topk_ids)) return GGUF_ERR_NULL;
  const size_t lds = (size_t)(1 + ALIGN_WAVES) * num_experts * sizeof(int);
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(ALIGN_THREADS), lds, (hipStream_t)stream, topk_ids, (int)numel,
                     (int)num_experts, (int)block, sorted_token_ids, (int)sorted_capacity, expert_ids, (int)expert_capacity,
                     num_tokens_post_padded);
  return launch_status();
}

extern "C" int gguf_moe_weighted_sum(const void* Y, const float* topk_weights, void* out, int dtype, int64_t tokens,
                                     int64_t top_k, int64_t N, gguf_stream_t stream) {
  using namespace gguf;
  if (tokens < 0 || top_k <= 0 || N < 0 || tokens > 0x7FFFFFF0LL || top_k > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  if (dtype < 0 || dtype > 2) return GGUF_ERR_DTYPE;
  if (tokens == 0 || N == 0) return GGUF_OK;
  if (!Y || !topk_weights || !out) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const unsigned gx = (unsigned)((N + 255) / 256 < 64 ? (N + 255) / 256 : 64);
  for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
    const unsigned gy = (unsigned)(tokens - t0 < 65535 ? tokens - t0 : 65535);
    GGUF_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((moe_weighted_sum_kernel<scalar_t>), dim3(gx, gy), dim3(256), 0, s,
                                                  (const scalar_t*)Y + t0 * top_k * N, topk_weights + t0 * top_k,
                                                  (scalar_t*)out + t0 * N, (int)top_k, N));
  }
  return launch_status();
}
