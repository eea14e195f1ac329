// Measurement probes, built into their own library (libgguf_probes.so) and loaded by bench.py only; nothing here is
// on the operator path.
//   * plain streaming reads of a buffer, by launch geometry: what one launch over a matrix-sized buffer can reach on
//     this machine before any arithmetic is added (the ceiling the GEMV kernels are held against);
//   * a plain copy of known size, to scale the FETCH_SIZE / WRITE_SIZE hardware counters;
//   * the streaming GEMV kernel of the library compiled with its phase trace on (Q4_K, batch 1, fp16).
#ifndef GGUF_PROBE_NO_TRACE   // (the untraced build of this file is for timing the same kernel without the trace's stores)
#define GGUF_TRACE_PHASES 1
#endif
#include "../mmvq_core.h"

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// workgroup w reads the contiguous range [w * per, (w + 1) * per) of 16-byte words, UNROLL loads in flight per lane
template <int UNROLL, bool NONTEMPORAL>
__global__ void read_kernel(const u32x4* __restrict__ src, int64_t n16, int* sink) {
  const int64_t per = (n16 + gridDim.x - 1) / gridDim.x;
  const int64_t lo = blockIdx.x * per, hi = lo + per < n16 ? lo + per : n16;
  u32x4 acc = {0, 0, 0, 0};
  int64_t i = lo + threadIdx.x;
  for (; i + (int64_t)(UNROLL - 1) * blockDim.x < hi; i += (int64_t)UNROLL * blockDim.x) {
    u32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const u32x4* p = src + i + (int64_t)u * blockDim.x;
      v[u] = NONTEMPORAL ? __builtin_nontemporal_load(p) : *p;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
  }
  for (; i < hi; i += blockDim.x) acc ^= src[i];
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1;   // keeps the loads alive; practically never true
}

__global__ void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (int64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

}  // namespace

extern "C" int gguf_probe_read(const void* buf, int64_t bytes, int threads, int workgroups, int unroll, int nontemporal, int* sink,
                               void* stream) {
  if (!buf || !sink || bytes <= 0 || bytes % 16 != 0 || threads <= 0 || threads > 1024 || workgroups <= 0) return -3;
  const dim3 g(workgroups), b(threads);
  hipStream_t s = (hipStream_t)stream;
  const u32x4* p = (const u32x4*)buf;
  const int64_t n16 = bytes / 16;
#define GGUF_PROBE_CASE(U, NT) \
  if (unroll == U && (nontemporal != 0) == NT) { hipLaunchKernelGGL((read_kernel<U, NT>), g, b, 0, s, p, n16, sink); return gguf::launch_status(); }
  GGUF_PROBE_CASE(2, false) GGUF_PROBE_CASE(4, false) GGUF_PROBE_CASE(8, false)
  GGUF_PROBE_CASE(2, true) GGUF_PROBE_CASE(4, true) GGUF_PROBE_CASE(8, true)
#undef GGUF_PROBE_CASE
  return -3;
}

extern "C" int gguf_probe_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  if (!src || !dst || bytes <= 0 || bytes % 16 != 0) return -3;
  hipLaunchKernelGGL(copy_kernel, dim3(2048), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, (u32x4*)dst, bytes / 16);
  return gguf::launch_status();
}

// Y[1, N] = q8_1(X[1, K]) . W[N, K]^T for Q4_K and fp16, the library's streaming kernel with its phase trace on.
extern "C" int gguf_probe_mmvq_q4_k(const void* W, const void* x, void* Y, int64_t N, int64_t K, void* stream) {
  using namespace gguf;
  if (!W || !x || !Y || N <= 0 || K <= 0 || K % 256 != 0) return -3;
  const LinearArgs la;
  bool ok;
  if (K <= 4096 && N <= 16 * num_cus()) ok = launch_stream<FmtQ4_K, 1, _Float16, false, 8>(W, (const _Float16*)x, (_Float16*)Y, (int)N, (int)K, (hipStream_t)stream, la);
  else ok = launch_stream<FmtQ4_K, 1, _Float16>(W, (const _Float16*)x, (_Float16*)Y, (int)N, (int)K, (hipStream_t)stream, la);
  return ok ? launch_status() : -3;
}

// The trace of the last gguf_probe_mmvq_q4_k launch: per workgroup, for its first and its last wave, the wall-clock
// ticks (10 ns) at entry, own activations quantized, all activations in LDS, own rows walked, results stored.
extern "C" int gguf_probe_mmvq_trace(unsigned long long* host, int workgroups) {
  if (!host || workgroups <= 0 || workgroups > 1024) return -3;
#ifdef GGUF_TRACE_PHASES
  return hipMemcpyFromSymbol(host, HIP_SYMBOL(gguf::g_mmvq_phases), (size_t)workgroups * 2 * 8 * sizeof(unsigned long long)) == hipSuccess ? 0 : -5;
#else
  return -1;
#endif
}
