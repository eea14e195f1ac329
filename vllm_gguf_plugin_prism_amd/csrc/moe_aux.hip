// Helpers at the caller seam of the MoE path: the routing sort that feeds the grouped kernel, and the
// top-k weighting + sum that follows the second expert GEMM.
//
// The reference takes both from vLLM (quantization/fused_moe.py:53-66: moe_align_block_size;
// :87-95: out.mul_(topk_weights) then ops.moe_sum); they are not part of its own native code.
#include "q8_1_device.h"

namespace gguf {

constexpr int ALIGN_THREADS = 1024;
constexpr int ALIGN_WAVES = ALIGN_THREADS / 64;
constexpr int ALIGN_MAX_EXPERTS = 1024;

// One workgroup sorts the flat (token, choice) pairs by expert, stably, and pads every expert's run to a multiple
// of `block`:
//   sorted_ids[pos]  flat pair index, or `numel` in padding and unused slots
//   expert_ids[b]    expert of block b, -1 past the padded total
//   num_post_padded  padded total
// Stable order (ascending pair index inside a run) makes the result a pure function of the input.
// Every wave owns a contiguous stretch of the pairs.  Pass 1 counts experts per wave (a private histogram row in LDS);
// a scan over experts and, per expert, over waves turns the rows into the first slot of each (wave, expert); pass 2
// walks the stretch again 64 pairs at a time, places every pair at its row's cursor plus the number of lanes below it
// with the same expert, and moves the cursor on.  The lanes that share an expert are found with one ballot per bit
// of the expert id.  A wave's LDS operations complete in order, so its row needs no barrier inside a pass.
__device__ __forceinline__ void moe_align_body(const int32_t* __restrict__ topk_ids, int numel, int num_experts, int block,
                                               int32_t* __restrict__ sorted_ids, int sorted_capacity,
                                               int32_t* __restrict__ expert_ids, int expert_capacity,
                                               int32_t* __restrict__ num_post_padded, int* lds,
                                               int32_t* __restrict__ slot_of_pair = nullptr) {
  int* start = lds;                          // [E] pairs of the expert, then the first slot of its run
  int* cursor = lds + num_experts;           // [ALIGN_WAVES][E] per-wave counts, then per-wave cursors
  __shared__ int total_padded;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per_wave = ((numel + ALIGN_WAVES - 1) / ALIGN_WAVES + 63) / 64 * 64;
  const int w_begin = min(wave * per_wave, numel), w_end = min(w_begin + per_wave, numel);
  int* mine = cursor + wave * num_experts;

  for (int i = tid; i < sorted_capacity; i += ALIGN_THREADS) sorted_ids[i] = numel;
  if (slot_of_pair)   // the inverse of the sort: -1 for a pair whose expert id names no expert
    for (int i = tid; i < numel; i += ALIGN_THREADS) slot_of_pair[i] = -1;
  for (int e = lane; e < num_experts; e += 64) mine[e] = 0;
  for (int i = w_begin + lane; i < w_end; i += 64) {
    const int e = topk_ids[i];
    if (e >= 0 && e < num_experts) atomicAdd(&mine[e], 1);  // counts: the sum does not depend on the order of adds
  }
  __syncthreads();
  for (int e = tid; e < num_experts; e += ALIGN_THREADS) {
    int sum = 0;
    for (int w = 0; w < ALIGN_WAVES; ++w) sum += cursor[w * num_experts + e];
    start[e] = sum;
  }
  __syncthreads();
  if (wave == 0) {  // exclusive scan of the padded counts, 64 experts at a time
    int running = 0;
    for (int e0 = 0; e0 < num_experts; e0 += 64) {
      const int e = e0 + lane;
      const int padded = e < num_experts ? (start[e] + block - 1) / block * block : 0;
      int incl = padded;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int below = __shfl_up(incl, d);
        if (lane >= d) incl += below;
      }
      if (e < num_experts) start[e] = running + incl - padded;
      running += __shfl(incl, 63);
    }
    if (lane == 0) {
      total_padded = running;
      num_post_padded[0] = running;
    }
  }
  __syncthreads();
  for (int e = tid; e < num_experts; e += ALIGN_THREADS) {
    // expert e owns blocks [start[e], start[e+1]) / block; its waves' cursors follow each other inside the run
    const int end = e + 1 < num_experts ? start[e + 1] : total_padded;
    for (int b = start[e] / block; b < end / block && b < expert_capacity; ++b) expert_ids[b] = e;
    int pos = start[e];
    for (int w = 0; w < ALIGN_WAVES; ++w) {
      const int c = cursor[w * num_experts + e];
      cursor[w * num_experts + e] = pos;
      pos += c;
    }
  }
  for (int b = total_padded / block + tid; b < expert_capacity; b += ALIGN_THREADS) expert_ids[b] = -1;
  __syncthreads();

  const int bits = 32 - __clz(max(num_experts - 1, 1));
  for (int i0 = w_begin; i0 < w_end; i0 += 64) {
    const int i = i0 + lane;
    int e = i < w_end ? topk_ids[i] : -1;
    if (e >= num_experts) e = -1;
    unsigned long long same = __ballot(e >= 0);   // lanes with this lane's expert
    for (int b = 0; b < bits; ++b) {
      const unsigned long long set = __ballot((e >> b) & 1);
      same &= ((e >> b) & 1) ? set : ~set;
    }
    if (e >= 0) {
      const int below = __popcll(same & ((1ull << lane) - 1));
      const int pos = mine[e] + below;
      if (pos < sorted_capacity) sorted_ids[pos] = i;
      if (slot_of_pair && pos < sorted_capacity) slot_of_pair[i] = pos;
      if (below == 0) mine[e] = pos + __popcll(same);   // one lane per expert moves the cursor; read above, written here
    }
  }
}

__global__ __launch_bounds__(ALIGN_THREADS) void moe_align_kernel(const int32_t* __restrict__ topk_ids, int numel,
                                                                  int num_experts, int block,
                                                                  int32_t* __restrict__ sorted_ids, int sorted_capacity,
                                                                  int32_t* __restrict__ expert_ids, int expert_capacity,
                                                                  int32_t* __restrict__ num_post_padded) {
  extern __shared__ int lds[];
  moe_align_body(topk_ids, numel, num_experts, block, sorted_ids, sorted_capacity, expert_ids, expert_capacity, num_post_padded, lds);
}

__global__ __launch_bounds__(ALIGN_THREADS) void moe_align_inverse_kernel(const int32_t* __restrict__ topk_ids, int numel, int num_experts,
                                                                          int block, int32_t* __restrict__ sorted_ids, int sorted_capacity,
                                                                          int32_t* __restrict__ expert_ids, int expert_capacity,
                                                                          int32_t* __restrict__ num_post_padded,
                                                                          int32_t* __restrict__ slot_of_pair) {
  extern __shared__ int lds[];
  moe_align_body(topk_ids, numel, num_experts, block, sorted_ids, sorted_capacity, expert_ids, expert_capacity, num_post_padded, lds,
                 slot_of_pair);
}

// Row s of the workspace = the q8_1 quantisation of the token row behind slot s of the sort (zeros in padding slots; slots
// past the padded total are left alone): the activations in the order in which the grouped contraction walks them.
template <typename T>
__global__ __launch_bounds__(256) void moe_gather_quantize_kernel(const T* __restrict__ x, char* __restrict__ ws, int K, int Kp,
                                                                  int64_t row_bytes, const int32_t* __restrict__ sorted_ids,
                                                                  const int32_t* __restrict__ num_post_padded, int numel, int top_k) {
  const int t = blockIdx.x * 256 + threadIdx.x;   // one thread per 8 values of the padded row
  const int s = blockIdx.y;
  if (t * 8 >= Kp || s >= num_post_padded[0]) return;
  const int pair = sorted_ids[s];
  if (pair < numel) {
    q8_1_quantize_thread<T>(x + (int64_t)(pair / top_k) * K, ws + (int64_t)s * row_bytes, K, Kp, row_bytes, ACT_NONE, 0, t, nullptr);
  } else {
    char* row = ws + (int64_t)s * row_bytes;
    *(uint2*)(row + 8 * t) = make_uint2(0, 0);
    if ((t & 3) == 0) {
      float* fd = (float*)(row + Kp);
      const int b = t >> 2, nb = Kp / 32;
      fd[b] = 0.0f; fd[nb + b] = 0.0f; fd[2 * nb + b] = 0.0f;
    }
  }
}

// The two preparations of a MoE layer on tiles in one launch: workgroup 0 sorts the routing, the others quantize the
// rows of X (1024 threads, eight values each: 8192 values of the padded rows per workgroup, rows in turn).
template <typename T>
__global__ __launch_bounds__(ALIGN_THREADS) void moe_prepare_kernel(const T* __restrict__ x, char* __restrict__ ws, int K, int Kp,
                                                                    int64_t row_bytes, int tokens, const int32_t* __restrict__ topk_ids,
                                                                    int numel, int num_experts, int block,
                                                                    int32_t* __restrict__ sorted_ids, int sorted_capacity,
                                                                    int32_t* __restrict__ expert_ids, int expert_capacity,
                                                                    int32_t* __restrict__ num_post_padded) {
  extern __shared__ int lds[];
  if (blockIdx.x == 0) {
    moe_align_body(topk_ids, numel, num_experts, block, sorted_ids, sorted_capacity, expert_ids, expert_capacity, num_post_padded, lds);
    return;
  }
  const int per_row = Kp / 8;                                   // threads a row takes
  const int64_t g = (int64_t)(blockIdx.x - 1) * ALIGN_THREADS + threadIdx.x;
  const int64_t m = g / per_row;
  if (m >= tokens) return;                                      // (per_row is a multiple of 64: whole waves leave)
  q8_1_quantize_thread<T>(x, ws, K, Kp, row_bytes, ACT_NONE, m, (int)(g % per_row), nullptr);
}

// out[t, n] = sum_k  T( float(Y[t, k, n]) * w[t, k] )   accumulated in fp32 in the order k = 0 .. top_k-1 and rounded
// once: the in-place multiply by the routing weights followed by the sum over the top-k axis.
template <typename T>
__global__ __launch_bounds__(256) void moe_weighted_sum_kernel(const T* __restrict__ Y, const float* __restrict__ w,
                                                               T* __restrict__ out, int top_k, int64_t N,
                                                               const int32_t* __restrict__ ids, int num_experts,
                                                               const int32_t* __restrict__ slot_of_pair) {
  const int64_t t = blockIdx.y;
  for (int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x; n < N; n += (int64_t)gridDim.x * 256) {
    float acc = 0.0f;
    for (int k = 0; k < top_k; ++k) {
      // (ids given: a pair whose id names no expert has a row of zeros, whatever Y holds there)
      // (slot_of_pair given: the rows of Y are in the order of the routing sort; -1 = the pair was dropped)
      const int64_t row = slot_of_pair ? (int64_t)slot_of_pair[t * top_k + k] : t * top_k + k;
      const bool live = row >= 0 && (!ids || (unsigned)ids[t * top_k + k] < (unsigned)num_experts);
      const T p = from_f32<T>((live ? to_f32<T>(Y[row * N + n]) : 0.0f) * w[t * top_k + k]);
      acc += to_f32<T>(p);
    }
    out[t * N + n] = from_f32<T>(acc);
  }
}

int moe_weighted_sum_live(const void* Y, const float* topk_weights, const int32_t* topk_ids, int num_experts, void* out, int dtype,
                          int64_t tokens, int64_t top_k, int64_t N, hipStream_t s, const int32_t* slot_of_pair) {
  const unsigned gx = (unsigned)((N + 255) / 256 < 64 ? (N + 255) / 256 : 64);
  for (int64_t t0 = 0; t0 < tokens; t0 += 65535) {
    const unsigned gy = (unsigned)(tokens - t0 < 65535 ? tokens - t0 : 65535);
    GGUF_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL((moe_weighted_sum_kernel<scalar_t>), dim3(gx, gy), dim3(256), 0, s,
                                                  (const scalar_t*)Y + (slot_of_pair ? 0 : t0 * top_k * N), topk_weights + t0 * top_k,
                                                  (scalar_t*)out + t0 * N, (int)top_k, N, topk_ids ? topk_ids + t0 * top_k : nullptr,
                                                  num_experts, slot_of_pair ? slot_of_pair + t0 * top_k : nullptr));
  }
  return launch_status();
}

// quantize_q8_1(X) and gguf_moe_align_block_size(topk_ids) in one launch (sizes checked by the caller)
int moe_prepare(const void* X, int xdtype, void* q8x, int tokens, int K, const int32_t* topk_ids, int numel, int num_experts, int block,
                int32_t* sorted_ids, int sorted_capacity, int32_t* expert_ids, int expert_capacity, int32_t* num_post_padded,
                hipStream_t s) {
  const int Kp = (int)q8_kp(K);
  const size_t lds = (size_t)(1 + ALIGN_WAVES) * num_experts * sizeof(int);
  if (lds > 65536) return GGUF_NOT_TAKEN;
  const int64_t threads = (int64_t)tokens * (Kp / 8);
  const unsigned grid = 1 + (unsigned)((threads + ALIGN_THREADS - 1) / ALIGN_THREADS);
  GGUF_DISPATCH_DTYPE(xdtype, hipLaunchKernelGGL(moe_prepare_kernel<scalar_t>, dim3(grid), dim3(ALIGN_THREADS), lds, s, (const scalar_t*)X,
                                                 (char*)q8x, K, Kp, q8_row_bytes(K), tokens, topk_ids, numel, num_experts, block, sorted_ids,
                                                 sorted_capacity, expert_ids, expert_capacity, num_post_padded));
  return launch_status();
}

// The routing sort with its inverse, then the rows of X quantized into slot order (two launches; sizes checked by the caller)
int moe_prepare_sorted(const void* X, int xdtype, void* q8x_sorted, int K, const int32_t* topk_ids, int numel, int top_k, int num_experts,
                       int block, int32_t* sorted_ids, int sorted_capacity, int32_t* expert_ids, int expert_capacity,
                       int32_t* num_post_padded, int32_t* slot_of_pair, hipStream_t s) {
  const size_t lds = (size_t)(1 + ALIGN_WAVES) * num_experts * sizeof(int);
  if (lds > 65536) return GGUF_NOT_TAKEN;
  hipLaunchKernelGGL(moe_align_inverse_kernel, dim3(1), dim3(ALIGN_THREADS), lds, s, topk_ids, numel, num_experts, block, sorted_ids,
                     sorted_capacity, expert_ids, expert_capacity, num_post_padded, slot_of_pair);
  const int Kp = (int)q8_kp(K);
  const int slots = sorted_capacity / block * block;
  if (slots > 65535) return GGUF_ERR_SHAPE;
  GGUF_DISPATCH_DTYPE(xdtype, hipLaunchKernelGGL(moe_gather_quantize_kernel<scalar_t>, dim3((Kp / 8 + 255) / 256, slots), dim3(256), 0, s,
                                                 (const scalar_t*)X, (char*)q8x_sorted, K, Kp, q8_row_bytes(K), sorted_ids, num_post_padded,
                                                 numel, top_k));
  return launch_status();
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
  if (lds > 65536) {
    static std::atomic<uint64_t> done{0};
    gguf::allow_large_lds(moe_align_kernel, (1 + ALIGN_WAVES) * ALIGN_MAX_EXPERTS * sizeof(int), done);
  }
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
  return moe_weighted_sum_live(Y, topk_weights, nullptr, 0, out, dtype, tokens, top_k, N, (hipStream_t)stream, nullptr);
}
