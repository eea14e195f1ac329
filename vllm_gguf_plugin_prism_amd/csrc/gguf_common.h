// Shared device helpers for the gfx950 GGUF kernels: block geometry, unaligned
// loads, int8 dot products, wave64 reductions and dtype conversion.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <atomic>

#include "../../include/gguf_hip.h"

namespace gguf {

// ggml type ids (reference: csrc/gguf/gguf_kernel.cu:119-215)
enum : int {
  T_Q4_0 = 2, T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q8_0 = 8,
  T_Q2_K = 10, T_Q3_K = 11, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14,
  T_IQ2_XXS = 16, T_IQ2_XS = 17, T_IQ3_XXS = 18, T_IQ1_S = 19, T_IQ4_NL = 20,
  T_IQ3_S = 21, T_IQ2_S = 22, T_IQ4_XS = 23, T_IQ1_M = 29,
};

__host__ __device__ constexpr int block_elems(int t) {
  return (t == T_Q4_0 || t == T_Q4_1 || t == T_Q5_0 || t == T_Q5_1 || t == T_Q8_0 || t == T_IQ4_NL) ? 32
       : (t == T_Q2_K || t == T_Q3_K || t == T_Q4_K || t == T_Q5_K || t == T_Q6_K || t == T_IQ2_XXS ||
          t == T_IQ2_XS || t == T_IQ3_XXS || t == T_IQ1_S || t == T_IQ3_S || t == T_IQ2_S || t == T_IQ4_XS ||
          t == T_IQ1_M) ? 256 : 0;
}
__host__ __device__ constexpr int block_bytes(int t) {
  switch (t) {
    case T_Q4_0: return 18;  case T_Q4_1: return 20;  case T_Q5_0: return 22;  case T_Q5_1: return 24;
    case T_Q8_0: return 34;  case T_Q2_K: return 84;  case T_Q3_K: return 110; case T_Q4_K: return 144;
    case T_Q5_K: return 176; case T_Q6_K: return 210; case T_IQ2_XXS: return 66; case T_IQ2_XS: return 74;
    case T_IQ3_XXS: return 98; case T_IQ1_S: return 50; case T_IQ4_NL: return 18; case T_IQ3_S: return 110;
    case T_IQ2_S: return 82; case T_IQ4_XS: return 136; case T_IQ1_M: return 56;
    default: return 0;
  }
}

// ---------------------------------------------------------------------------
// q8_1 workspace: per row of X (Kp = K rounded up to 512, nb = Kp / 32)
//   int8  qs[Kp]   quants
//   float d [nb]   block scale, the half-rounded value widened to fp32
//   float s [nb]   block sum of the unquantized values, half-rounded, widened
//   float du[nb]   d * sum(qs) of the block (exact in fp32)
// ---------------------------------------------------------------------------
__host__ __device__ inline int64_t q8_kp(int64_t K) { return (K + 511) / 512 * 512; }
__host__ __device__ inline int64_t q8_row_bytes(int64_t K) { return q8_kp(K) / 32 * 44; }
// Behind the M quantized rows the half-MFMA GEMM keeps the dequantized rows in half precision, [M][q8_half_pitch(K)].
// The pitch is not a multiple of 4096 bytes: a tile reads the same columns of many rows at once, and rows a power of
// two apart would all fall into the same memory channel.
__host__ __device__ inline int64_t q8_half_pitch(int64_t K) { return q8_kp(K) + 128; }

struct Q8Row {
  const int8_t* qs;
  const float* d;
  const float* s;
  const float* du;
};
__host__ __device__ inline Q8Row q8_row(const void* ws, int64_t K, int64_t row) {
  const int64_t kp = q8_kp(K);
  const char* base = (const char*)ws + row * q8_row_bytes(K);
  Q8Row r;
  r.qs = (const int8_t*)base;
  r.d = (const float*)(base + kp);
  r.s = r.d + kp / 32;
  r.du = r.s + kp / 32;
  return r;
}

// ---------------------------------------------------------------------------
// loads at arbitrary byte alignment (GGUF blocks are only 2-byte aligned)
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ T ld(const void* p) {
  T v;
  __builtin_memcpy(&v, p, sizeof(T));
  return v;
}
// A block whose size is 2 modulo 4 (18, 22, 34 bytes) starts at an even address that is a multiple of 4 for every
// other block only.  A 16-byte load from such an address costs the memory pipeline about twice an aligned one, so
// the block is fetched as the ND = (size + 2) / 4 whole dwords that cover it from the dword boundary at or below it
// -- the first and the last of them hold at least one byte of the block, so nothing outside the dwords the block
// touches is read -- and the fields are cut out with funnel shifts.  Returns the bit offset (0 or 16) of the block
// inside w[0].
template <int ND>
__device__ __forceinline__ uint32_t ld_block_dwords(const uint8_t* p, uint32_t (&w)[ND]) {
  const uintptr_t a = (uintptr_t)p;
  const __attribute__((address_space(1))) uint32_t* q = (const __attribute__((address_space(1))) uint32_t*)(a & ~(uintptr_t)3);
#pragma unroll
  for (int i = 0; i < ND; ++i) w[i] = q[i];
  return (uint32_t)(a & 2) * 8;
}
// bits [bits, bits + 32) of the 64-bit value hi:lo, bits in 0..32
__device__ __forceinline__ uint32_t funnel(uint32_t lo, uint32_t hi, uint32_t bits) {
  return (uint32_t)((((uint64_t)hi << 32) | lo) >> bits);
}
// The same cut from a copy of the blocks in LDS: the ND dwords from the dword boundary at or below byte off (even) of
// base (16-byte aligned); returns the bit offset of that byte inside w[0].
template <int ND>
__device__ __forceinline__ uint32_t lds_block_dwords(const char* base, int off, uint32_t (&w)[ND]) {
  const uint32_t* q = (const uint32_t*)(base + (off & ~3));
#pragma unroll
  for (int i = 0; i < ND; ++i) w[i] = q[i];
  return (uint32_t)(off & 2) * 8;
}
// eight bytes at an even offset of such a copy (touches the dword behind them when the offset is a multiple of four)
__device__ __forceinline__ uint2 lds_cut8(const char* base, int off) {
  uint32_t w[3];
  const uint32_t sh = lds_block_dwords(base, off, w);
  return make_uint2(funnel(w[0], w[1], sh), funnel(w[1], w[2], sh));
}
__device__ __forceinline__ float ld_f16(const void* p) { return (float)ld<_Float16>(p); }
__device__ __forceinline__ _Float16 ld_h(const void* p) { return ld<_Float16>(p); }

__device__ __forceinline__ int dot4(int a, int b, int c) { return __builtin_amdgcn_sdot4(a, b, c, false); }

// byte-wise negate of the bytes of g selected by the 0x00/0xff byte mask m (all bytes of g are in 1..127)
__device__ __forceinline__ uint32_t neg_bytes(uint32_t g, uint32_t m) { return (g ^ m) + (m & 0x01010101u); }

// ---------------------------------------------------------------------------
// wave64 sum: DPP inside rows of 16 lanes, then four row totals by readlane
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_mov<0x141>(v);  // row_half_mirror
  v += dpp_mov<0x140>(v);  // row_mirror
  const int b = __builtin_bit_cast(int, v);
  const float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (r0 + r1) + (r2 + r3);
}

// ---------------------------------------------------------------------------
// dtype plumbing.  bf16 is carried as its 16-bit pattern.
// ---------------------------------------------------------------------------
struct bf16_t {
  uint16_t bits;
};
__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __builtin_bit_cast(float, (uint32_t)v.bits << 16); }
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {  // round to nearest even, quiet NaN
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  bf16_t r;
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
    r.bits = 0x7FC0;
  } else {
    r.bits = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
  }
  return r;
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<_Float16>(_Float16 v) { return (float)v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ _Float16 from_f32<_Float16>(float v) { return (_Float16)v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// half result of the half-math dequant kernels -> output dtype (reference: ggml-common.h:1079-1096)
template <typename T> __device__ __forceinline__ T from_half(_Float16 v);
template <> __device__ __forceinline__ float from_half<float>(_Float16 v) { return (float)v; }
template <> __device__ __forceinline__ _Float16 from_half<_Float16>(_Float16 v) { return v; }
template <> __device__ __forceinline__ bf16_t from_half<bf16_t>(_Float16 v) { return f32_to_bf16((float)v); }

#define GGUF_DISPATCH_DTYPE(code, ...)                                   \
  switch (code) {                                                        \
    case GGUF_DTYPE_F32: { using scalar_t = float; __VA_ARGS__; break; } \
    case GGUF_DTYPE_F16: { using scalar_t = _Float16; __VA_ARGS__; break; } \
    case GGUF_DTYPE_BF16: { using scalar_t = gguf::bf16_t; __VA_ARGS__; break; } \
    default: return GGUF_ERR_DTYPE;                                      \
  }

// How one call addresses a shard of a merged linear layer (quantization/linear.py:229-262): the rows of W may sit in a
// wider, padded tensor, the result may be a column range of a wider output, and the layer's bias may be added.
struct LinearArgs {
  int64_t w_pitch = 0;         // bytes between rows of W; 0 = rows are dense
  int64_t ldy = 0;             // elements between rows of Y; 0 = N
  const void* bias = nullptr;  // N values of Y's dtype, added to every row of the result after it is rounded; or null
  bool tile_sums = false;      // GEMV kernels only: form the offset term as the reference's tile kernels do (see TileSums)
};
// out = round(round(v) + bias): the reference rounds the product to the output dtype and then adds in that dtype
template <typename T>
__device__ __forceinline__ T finish(float v, const T* bias, int64_t n) {
  const T r = from_f32<T>(v);
  return bias ? from_f32<T>(to_f32<T>(r) + to_f32<T>(bias[n])) : r;
}

// q8_1 quantisation of M rows into the workspace (q8_1.hip).  act: gated activation applied while loading (see
// q8_1_device.h).  half_plane: if not null, also the dequantized rows in half precision, [M][q8_kp(K)].
// From how many pairs on the per-pair MoE operator sorts its pairs by expert and reads a shared expert once per group
// of them: two pairs per expert on average.  While all the experts together fit the last-level cache the per-pair
// kernel, which has no sort and no second launch, reads shared experts from there and stays ahead a little longer
// (Q4_0, 64 experts [2048,2048] top-8: 65 against 95 us at 16 tokens, 91 against 96 at 20, 101 against 95 at 24;
// the whole layer on the tile kernels takes 85 us from there on).
static inline bool moe_share_pays(int64_t pairs, int64_t num_experts, int64_t expert_bytes) {
  const bool cached = num_experts * expert_bytes <= (192ll << 20);
  return cached ? 2 * pairs >= 5 * num_experts : pairs >= 2 * num_experts;
}
int quantize_q8_1(const void* x, int xdtype, void* ws, int64_t M, int64_t K, hipStream_t stream, int act = 0,
                  void* half_plane = nullptr);

// Opt a kernel in to more than 64 KB of dynamic LDS, once per device: `done` is the caller's bit set of the devices
// already served (one static per kernel instantiation).  The attribute belongs to the device the kernel's code object
// is loaded on, so a second GPU in the same process needs its own call.
template <typename K>
static inline void allow_large_lds(K kern, size_t lds, std::atomic<uint64_t>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) dev = 0;
  const uint64_t bit = 1ull << dev;
  if (done.load(std::memory_order_relaxed) & bit) return;
  (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  done.fetch_or(bit, std::memory_order_relaxed);
}

// compute units of the current device (asked once per device)
static inline int num_cus() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev > 63) dev = 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    hipDeviceProp_t prop;
    n = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

constexpr int GGUF_NOT_TAKEN = 1;  // internal: a route that declined the call (never returned through the C ABI)
inline int launch_status() { return hipGetLastError() == hipSuccess ? GGUF_OK : GGUF_ERR_LAUNCH; }

}  // namespace gguf
