// q8_1 quantisation of eight consecutive activation values per lane, four lanes (one DPP quad)
// per 32-value block.  Shared by the stand-alone quantizer and by the GEMV prologue that
// quantizes straight into LDS.
//
// Reference semantics (csrc/gguf/gguf_kernel.cu:32-69): amax and sum by an xor butterfly over
// lane masks 16, 8, 4, 2, 1; d = amax / 127 (fp32, IEEE division); q = roundf(x / d), 0 when
// amax == 0; d and sum stored rounded to half.  With eight values per lane, masks 16 and 8 are
// the quad partners lane^2 and lane^1 and masks 4, 2, 1 are in-register, which evaluates the
// same fp32 addition tree.
#pragma once
#include "gguf_common.h"

namespace gguf {

// Eight consecutive activation values: raw8<T>::load only issues the global load (so it can be hoisted
// above other loads without forcing a wait), cvt widens to fp32.
template <typename T> struct raw8;
typedef float raw_f32x4 __attribute__((ext_vector_type(4)));      // (plain vector types: a register tuple the inline
typedef uint32_t raw_u32x4 __attribute__((ext_vector_type(4)));   //  assembly below can name as one operand)
template <> struct raw8<float> {
  raw_f32x4 a, b;
  __device__ __forceinline__ void load(const float* p) { a = *(const raw_f32x4*)p; b = *(const raw_f32x4*)(p + 4); }
  // The same load kept from the compiler's count of loads in flight, for a kernel that has loads outstanding which the
  // values need not wait for: landed() waits until at most `behind` younger loads are outstanding (loads return in order).
  __device__ __forceinline__ void load_uncounted(const float* p) {
    asm volatile("global_load_dwordx4 %0, %2, off\n\tglobal_load_dwordx4 %1, %2, off offset:16" : "=&v"(a), "=&v"(b) : "v"(p) : "memory");
  }
  template <int BEHIND> __device__ __forceinline__ void landed() {
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(BEHIND) : "memory");
  }
  // Nothing that uses the loaded values may be scheduled before this point (and the wait for them comes here).
  __device__ __forceinline__ void hold() {
    asm volatile("" : "+v"(a.x), "+v"(a.y), "+v"(a.z), "+v"(a.w), "+v"(b.x), "+v"(b.y), "+v"(b.z), "+v"(b.w));
  }
  __device__ __forceinline__ void cvt(float (&v)[8]) const {
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};
template <> struct raw8<_Float16> {
  raw_u32x4 a;
  __device__ __forceinline__ void load(const _Float16* p) { a = *(const raw_u32x4*)p; }
  __device__ __forceinline__ void load_uncounted(const _Float16* p) { asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(a) : "v"(p) : "memory"); }
  template <int BEHIND> __device__ __forceinline__ void landed() { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(BEHIND) : "memory"); }
  __device__ __forceinline__ void hold() { asm volatile("" : "+v"(a.x), "+v"(a.y), "+v"(a.z), "+v"(a.w)); }
  __device__ __forceinline__ void cvt(float (&v)[8]) const {
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] & 0xFFFF));
      v[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (uint16_t)(w[i] >> 16));
    }
  }
};
template <> struct raw8<bf16_t> {
  raw_u32x4 a;
  __device__ __forceinline__ void load(const bf16_t* p) { a = *(const raw_u32x4*)p; }
  __device__ __forceinline__ void load_uncounted(const bf16_t* p) { asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(a) : "v"(p) : "memory"); }
  template <int BEHIND> __device__ __forceinline__ void landed() { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(BEHIND) : "memory"); }
  __device__ __forceinline__ void hold() { asm volatile("" : "+v"(a.x), "+v"(a.y), "+v"(a.z), "+v"(a.w)); }
  __device__ __forceinline__ void cvt(float (&v)[8]) const {
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
      v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xFFFF0000u);
    }
  }
};
template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
  raw8<T> r;
  r.load(p);
  r.cvt(v);
}

// Gated activation applied while loading: v = T(act(gate)) * up with the product rounded to T again, i.e. the values a
// separate act-and-multiply kernel would have stored in dtype T (the MoE layer applies it between its two GEMMs,
// quantization/fused_moe.py:44-51,80).  act: 1 = SiLU, 2 = GELU (erf form).
enum { ACT_NONE = 0, ACT_SILU = 1, ACT_GELU = 2 };
// g <- T(T(act(g)) * u) for eight values already widened to fp32
template <typename T>
__device__ __forceinline__ float gate1(float g, float u, int act) {
  const float a = act == ACT_SILU ? g / (1.0f + expf(-g)) : g * 0.5f * (1.0f + erff(g * 0.70710678118654752440f));
  return to_f32<T>(from_f32<T>(to_f32<T>(from_f32<T>(a)) * u));  // T x T products are exact in fp32, so one rounding each
}
template <typename T>
__device__ __forceinline__ void gate8(float (&g)[8], const float (&u)[8], int act) {
#pragma unroll
  for (int i = 0; i < 8; ++i) g[i] = gate1<T>(g[i], u[i], act);
}
template <typename T>
__device__ __forceinline__ void load8_gated(const T* gate, const T* up, int act, float (&v)[8]) {
  float u[8];
  load8<T>(gate, v);
  load8<T>(up, u);
  gate8<T>(v, u, act);
}

template <int CTRL>
__device__ __forceinline__ int dpp_mov_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

struct Q8Quad {
  uint2 q;      // this lane's eight quants
  float d;      // block scale, half-rounded           (same in all four lanes)
  float s;      // block sum of the inputs, half-rounded
  float du;     // d * sum of the block's quants
};

// All four lanes of a quad must call this together.
__device__ __forceinline__ Q8Quad q8_1_quantize8(const float (&v)[8]) {
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
  amax = fmaxf(amax, dpp_mov<0x4E>(amax));
  amax = fmaxf(amax, dpp_mov<0xB1>(amax));

  float s[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = v[i] + dpp_mov<0x4E>(v[i]);  // mask 16: lane ^ 2
#pragma unroll
  for (int i = 0; i < 8; ++i) s[i] = s[i] + dpp_mov<0xB1>(s[i]);  // mask 8:  lane ^ 1
  const float t0 = s[0] + s[4], t1 = s[1] + s[5], t2 = s[2] + s[6], t3 = s[3] + s[7];  // mask 4
  const float u0 = t0 + t2, u1 = t1 + t3;                                             // mask 2
  const float sum = u0 + u1;                                                          // mask 1

  const float d = amax / 127.0f;
  const float dd = amax == 0.0f ? 1.0f : d;  // an all-zero block divides 0 by 1: q = 0 without a branch
  // q = roundf(x / dd), ties away from zero, bit-for-bit what the IEEE quotient gives.  The hardware reciprocal
  // (one ulp) replaces eight divisions: x * rcp(dd) is within 127 * 2^-22 of the true quotient, so it rounds the same
  // way unless its fraction lies within 2^-14 of a tie, and away from a tie adding half a unit and truncating is the
  // rounding.  A lane that meets a near-tie among its eight values, or a scale so small that its reciprocal
  // overflows, forms the exact quotients for all eight instead.
  const float rd = __builtin_amdgcn_rcpf(dd);
  float t[8];
  bool exact = !(rd < 3.0e38f);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    t[i] = v[i] * rd;
    const float fr = __builtin_amdgcn_fractf(fabsf(t[i]));
    exact = exact || fabsf(fr - 0.5f) < 6.1035156e-5f;
  }
  if (exact) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float e = v[i] / dd;
      const float tr = truncf(e);
      // the quotient rounded half away from zero, as a value that the add-half-and-truncate below maps to itself
      t[i] = tr + (fabsf(e - tr) >= 0.5f ? copysignf(1.0f, e) : 0.0f);
    }
  }
  int q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = (int)(t[i] + copysignf(0.5f, t[i]));   // (the conversion truncates)
  Q8Quad r;
  r.q.x = __builtin_amdgcn_perm(__builtin_amdgcn_perm(q[3], q[2], 0x0c0c0400), __builtin_amdgcn_perm(q[1], q[0], 0x0c0c0400), 0x05040100);
  r.q.y = __builtin_amdgcn_perm(__builtin_amdgcn_perm(q[7], q[6], 0x0c0c0400), __builtin_amdgcn_perm(q[5], q[4], 0x0c0c0400), 0x05040100);
  int isum = __builtin_amdgcn_sdot4((int)r.q.x, 0x01010101, 0, false);
  isum = __builtin_amdgcn_sdot4((int)r.q.y, 0x01010101, isum, false);
  isum += dpp_mov_i<0x4E>(isum);
  isum += dpp_mov_i<0xB1>(isum);
  r.d = (float)(_Float16)d;
  r.s = (float)(_Float16)sum;
  r.du = r.d * (float)isum;
  return r;
}

// One thread of the row quantizer: the eight values [8 t, 8 t + 8) of padded row m -> eight quants, and from the first
// lane of each quad the block's d, s and d * sum(q) planes.  The four lanes of a quad must run together (the block's
// amax and sum cross them).  act: rows of x are [gate | up] and the gated activation is quantized; xh: also the
// dequantized row in half precision.
template <typename T>
__device__ __forceinline__ void q8_1_quantize_thread(const T* __restrict__ x, char* __restrict__ ws, int K, int Kp, int64_t row_bytes, int act,
                                                     int64_t m, int t, _Float16* __restrict__ xh) {
  const int e0 = t * 8;
  float v[8];
  if (e0 < K) {
    if (act == ACT_NONE) load8<T>(x + m * (int64_t)K + e0, v);
    else load8_gated<T>(x + m * (int64_t)(2 * K) + e0, x + m * (int64_t)(2 * K) + K + e0, act, v);  // rows are [gate | up]
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.0f;
  }
  const Q8Quad r = q8_1_quantize8(v);
  char* row = ws + m * row_bytes;
  *(uint2*)(row + e0) = r.q;
  if (xh) {
    // the dequantized row in half precision for the half-MFMA GEMM: RN16(d * q), d being the half-rounded scale.
    // d * q is exact in fp32; magnitudes past the half range saturate (only reachable from bf16 / fp32 inputs).
    union { _Float16 h[8]; uint4 v; } o;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int q = (int)(int8_t)((i < 4 ? r.q.x >> (8 * i) : r.q.y >> (8 * (i - 4))) & 0xFF);
      o.h[i] = (_Float16)fminf(fmaxf(r.d * (float)q, -65504.0f), 65504.0f);
    }
    *(uint4*)(xh + m * (int64_t)(Kp + 128) + e0) = o.v;   // row pitch: q8_half_pitch
  }
  if ((t & 3) == 0) {
    const int b = t >> 2;
    const int nb = Kp / 32;
    float* fd = (float*)(row + Kp);
    fd[b] = r.d;
    fd[nb + b] = r.s;
    fd[2 * nb + b] = r.du;
  }
}


}  // namespace gguf
