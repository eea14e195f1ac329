// q8_1 activation quantizer for gfx950.
//
// Semantics follow the reference's quantize_q8_1 (csrc/gguf/gguf_kernel.cu:32-69):
// per 32 values, amax and sum are reduced by an xor butterfly over lane masks
// 16, 8, 4, 2, 1; d = amax / 127 in fp32; q = roundf(x / d) (0 when amax == 0);
// d and sum are stored rounded to half; columns [K, roundup(K, 512)) count as 0.
//
// Layout here: four lanes own one block, eight consecutive values each, so
// lane^2 / lane^1 are the butterfly partners for masks 16 / 8 (DPP quad
// permutes) and masks 4, 2, 1 are in-register.  The fp32 addition tree is
// therefore the same tree the reference evaluates.
#include "q8_1_device.h"

namespace gguf {

template <typename T>
__global__ __launch_bounds__(256) void quantize_q8_1_kernel(const T* __restrict__ x, char* __restrict__ ws, int K,
                                                           int Kp, int64_t row_bytes, int act,
                                                           _Float16* __restrict__ xh) {
  const int t = blockIdx.x * 256 + threadIdx.x;  // one thread per 8 values of the padded row
  if (t * 8 >= Kp) return;
  q8_1_quantize_thread<T>(x, ws, K, Kp, row_bytes, act, blockIdx.y, t, xh);
}

__global__ void q8_1_unpack_kernel(const char* __restrict__ ws, int8_t* __restrict__ q, float* __restrict__ ds, int Kp,
                                   int64_t row_bytes) {
  const int64_t m = blockIdx.y;
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= Kp) return;
  const char* row = ws + m * row_bytes;
  q[m * Kp + i] = ((const int8_t*)row)[i];
  if ((i & 31) == 0) {
    const float* fd = (const float*)(row + Kp);
    const int nb = Kp / 32, b = i >> 5;
    ds[(m * nb + b) * 2] = fd[b];
    ds[(m * nb + b) * 2 + 1] = fd[nb + b];
  }
}

int quantize_q8_1(const void* x, int xdtype, void* ws, int64_t M, int64_t K, hipStream_t stream, int act, void* half_plane) {
  if (M == 0) return GGUF_OK;
  const int Kp = (int)q8_kp(K);
  const int64_t rb = q8_row_bytes(K);
  const int gx = (Kp / 8 + 255) / 256;
  for (int64_t off = 0; off < M; off += 65535) {
    const int rows = (int)((M - off) < 65535 ? (M - off) : 65535);
    GGUF_DISPATCH_DTYPE(xdtype, hipLaunchKernelGGL(quantize_q8_1_kernel<scalar_t>, dim3(gx, rows), dim3(256), 0, stream,
                                                   (const scalar_t*)x + off * K * (act == ACT_NONE ? 1 : 2), (char*)ws + off * rb, (int)K, Kp, rb, act,
                                                   half_plane ? (_Float16*)half_plane + off * q8_half_pitch(K) : (_Float16*)nullptr));
  }
  return launch_status();
}

}  // namespace gguf

extern "C" int64_t gguf_q8_1_row_bytes(int64_t K) { return K <= 0 ? 0 : gguf::q8_row_bytes(K); }

extern "C" int gguf_quantize_q8_1(const void* x, int xdtype, void* ws, int64_t M, int64_t K, gguf_stream_t stream) {
  if (M < 0 || K <= 0 || K % 32 != 0) return GGUF_ERR_SHAPE;
  if (M > 0 && (!x || !ws)) return GGUF_ERR_NULL;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  return gguf::quantize_q8_1(x, xdtype, ws, M, K, (hipStream_t)stream, gguf::ACT_NONE, nullptr);
}

extern "C" int gguf_q8_1_unpack(const void* ws, int8_t* q, float* ds, int64_t M, int64_t K, gguf_stream_t stream) {
  if (M < 0 || K <= 0 || K % 32 != 0) return GGUF_ERR_SHAPE;
  if (M == 0) return GGUF_OK;
  if (!ws || !q || !ds) return GGUF_ERR_NULL;
  const int Kp = (int)gguf::q8_kp(K);
  for (int64_t off = 0; off < M; off += 65535) {
    const int rows = (int)((M - off) < 65535 ? (M - off) : 65535);
    hipLaunchKernelGGL(gguf::q8_1_unpack_kernel, dim3((Kp + 255) / 256, rows), dim3(256), 0, (hipStream_t)stream,
                       (const char*)ws + off * gguf::q8_row_bytes(K), q + off * Kp, ds + off * (Kp / 32) * 2, Kp,
                       gguf::q8_row_bytes(K));
  }
  return gguf::launch_status();
}
