// Decode-path GEMV on packed GGUF weights with q8_1 activations (gfx950).
//
//   Y[m, n] = sum over blocks of  dot(W block of row n, q8_1 block(s) of X[m])
//
// with the per-format block formulas of the reference's vec_dot_<fmt>_q8_1
// functions (csrc/gguf/vecdotq.cuh; cited at each format below).  The work
// split is not the reference's "one 64-lane wave per (row, vector)" grid
// (csrc/gguf/mmvq.cuh:2-50): here
//   * a workgroup of four waves owns 4*RPW consecutive rows, so its weight bytes
//     are one contiguous span of HBM, and every lane pulls 16 bytes per load;
//   * the quantized activations of up to eight vectors are staged once per
//     workgroup in LDS (quants + block scales), and every weight byte loaded is
//     used for all of them, so weights cross HBM once per call for M <= 8;
//   * a "unit" is the 32 weights one lane turns into int8 dot products per step;
//     partial sums stay in fp32 registers and are reduced with DPP at the end.
#include "gguf_common.h"
#include "grid_codes.h"

namespace gguf {

enum { AUX_NONE = 0, AUX_S8 = 1, AUX_DU = 2 };

struct Act {            // LDS views of one staged activation vector
  const int8_t* q;      // [kc]
  const float* d;       // [kc/32] block scales
  const float* a;       // [kc/32] block sums (AUX_S8) or d*sum(q) (AUX_DU)
};

// ------------------------------------------------------------------ Q4_0 (vecdotq.cuh:46-66,493-509)
struct FmtQ4_0 {
  static constexpr int QK = 32, BS = 18, AUX = AUX_S8, TABLE_BYTES = 0;
  struct Regs { float d; uint4 q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const uint8_t* b = row + (int64_t)(u0 + u) * BS;
    Regs r; r.d = ld_f16(b); r.q = ld<uint4>(b + 2); return r;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    const int4 lo = *(const int4*)(x.q + 32 * u), hi = *(const int4*)(x.q + 32 * u + 16);
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {lo.x, lo.y, lo.z, lo.w}, ah[4] = {hi.x, hi.y, hi.z, hi.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = dot4((int)(q[i] & 0x0F0F0F0Fu), al[i], s);
      s = dot4((int)((q[i] >> 4) & 0x0F0F0F0Fu), ah[i], s);
    }
    return r.d * ((float)s * x.d[u] - 8.0f * x.a[u]);
  }
};

// ------------------------------------------------------------------ Q8_0 (vecdotq.cuh:165-177,852-867)
struct FmtQ8_0 {
  static constexpr int QK = 32, BS = 34, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { float d; uint4 q0, q1; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const uint8_t* b = row + (int64_t)(u0 + u) * BS;
    Regs r; r.d = ld_f16(b); r.q0 = ld<uint4>(b + 2); r.q1 = ld<uint4>(b + 18); return r;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    const int4 a0 = *(const int4*)(x.q + 32 * u), a1 = *(const int4*)(x.q + 32 * u + 16);
    int s = 0;
    s = dot4((int)r.q0.x, a0.x, s); s = dot4((int)r.q0.y, a0.y, s); s = dot4((int)r.q0.z, a0.z, s); s = dot4((int)r.q0.w, a0.w, s);
    s = dot4((int)r.q1.x, a1.x, s); s = dot4((int)r.q1.y, a1.y, s); s = dot4((int)r.q1.z, a1.z, s); s = dot4((int)r.q1.w, a1.w, s);
    return r.d * x.d[u] * (float)s;
  }
};

// ------------------------------------------------------------------ Q4_K (vecdotq.cuh:328-351,1159-1202)
// unit c of a super-block: 16 bytes of qs = 16 low nibbles of sub-block 2g and 16 high nibbles of 2g+1
struct FmtQ4_K {
  static constexpr int QK = 256, BS = 144, AUX = AUX_DU, TABLE_BYTES = 0;
  struct Regs { float d, dmin; int sc0, sc1, m0, m1; uint4 q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7, g = c >> 1;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint4 hdr = ld<uint4>(b);
    Regs r;
    r.q = ld<uint4>(b + 16 + 16 * c);
    r.d = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x & 0xFFFF));
    r.dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x >> 16));
    const int sh = 16 * (g & 1);
    const uint32_t A = (hdr.y >> sh) & 0xFFFF, B = (hdr.z >> sh) & 0xFFFF, C = (hdr.w >> sh) & 0xFFFF;
    uint32_t a0, a1;
    if (g < 2) {
      a0 = A & 0x3F3F; a1 = B & 0x3F3F;
    } else {
      a0 = (C & 0x0F0F) | ((A & 0xC0C0) >> 2);
      a1 = ((C >> 4) & 0x0F0F) | ((B & 0xC0C0) >> 2);
    }
    r.sc0 = a0 & 0xFF; r.sc1 = a0 >> 8; r.m0 = a1 & 0xFF; r.m1 = a1 >> 8;
    if (c & 1) { r.m0 = 0; r.m1 = 0; }  // the offset term of a sub-block pair is added once, by its first unit
    return r;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    const int sb = u >> 3, c = u & 7, g = c >> 1, h = c & 1;
    const int8_t* qa = x.q + 256 * sb + 64 * g + 16 * h;
    const int4 lo = *(const int4*)qa, hi = *(const int4*)(qa + 32);
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {lo.x, lo.y, lo.z, lo.w}, ah[4] = {hi.x, hi.y, hi.z, hi.w};
    int s0 = 0, s1 = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s0 = dot4((int)(q[i] & 0x0F0F0F0Fu), al[i], s0);
      s1 = dot4((int)((q[i] >> 4) & 0x0F0F0F0Fu), ah[i], s1);
    }
    const float2 d8 = *(const float2*)(x.d + 8 * sb + 2 * g);
    const float2 du = *(const float2*)(x.a + 8 * sb + 2 * g);
    const float pos = d8.x * (float)(s0 * r.sc0) + d8.y * (float)(s1 * r.sc1);
    const float neg = du.x * (float)r.m0 + du.y * (float)r.m1;
    return r.d * pos - r.dmin * neg;
  }
};

// ------------------------------------------------------------------ Q6_K (vecdotq.cuh:447-465,1417-1441)
// unit c of a super-block: half h = c>>2, columns l in [8*(c&3), +8) of that half; covers elements
// 128h + 32t + l for t = 0..3, i.e. eight values in each of four q8_1 blocks.
struct FmtQ6_K {
  static constexpr int QK = 256, BS = 210, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { float d; uint2 qla, qlb, qh; int sc[4]; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7, h = c >> 2, cc = c & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r;
    r.qla = ld<uint2>(b + 64 * h + 8 * cc);
    r.qlb = ld<uint2>(b + 64 * h + 32 + 8 * cc);
    r.qh = ld<uint2>(b + 128 + 32 * h + 8 * cc);
    const uint2 s8 = ld<uint2>(b + 192 + 8 * h);
    const uint64_t sw = ((uint64_t)s8.y << 32) | s8.x;
    const int so = 8 * (cc >> 1);
#pragma unroll
    for (int t = 0; t < 4; ++t) r.sc[t] = (int)(int8_t)(sw >> (16 * t + so));
    r.d = ld_f16(b + 208);
    return r;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    const int sb = u >> 3, c = u & 7, h = c >> 2, cc = c & 3;
    const int8_t* qa = x.q + 256 * sb + 128 * h + 8 * cc;
    const float* d8 = x.d + 8 * sb + 4 * h;
    float acc = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int2 a = *(const int2*)(qa + 32 * t);
      const uint2 ql = (t & 1) ? r.qlb : r.qla;
      const int shl = (t >> 1) ? 4 : 0;
      const int vx = (int)(((ql.x >> shl) & 0x0F0F0F0Fu) | (((r.qh.x >> (2 * t)) & 0x03030303u) << 4));
      const int vy = (int)(((ql.y >> shl) & 0x0F0F0F0Fu) | (((r.qh.y >> (2 * t)) & 0x03030303u) << 4));
      const int s = dot4(vx, a.x, dot4(vy, a.y, 0));
      const int ones = dot4(0x01010101, a.x, dot4(0x01010101, a.y, 0));
      acc += d8[t] * (float)(r.sc[t] * (s - 32 * ones));
    }
    return r.d * acc;
  }
};

// 16-entry signed byte table lookup of four 4-bit indices held one per byte
__device__ __forceinline__ int lut16(uint32_t idx, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
  const uint32_t sel = idx & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
  const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
  return (int)((hi & m) | (lo & ~m));
}

// ------------------------------------------------------------------ IQ4_XS (vecdotq.cuh:1791-1811)
struct FmtIQ4_XS {
  static constexpr int QK = 256, BS = 136, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { float dl; int vlo[4], vhi[4]; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint2 hdr = ld<uint2>(b);
    const uint4 q = ld<uint4>(b + 8 + 16 * ib);
    const int ls = (int)(((hdr.y >> (4 * ib)) & 0xF) | ((((hdr.x >> 16) >> (2 * ib)) & 3) << 4));
    Regs r;
    r.dl = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x & 0xFFFF)) * (float)(ls - 32);
    // kvalues_iq4nl as four little-endian words
    constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
    const uint32_t qq[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      r.vlo[i] = lut16(qq[i] & 0x0F0F0F0Fu, T0, T1, T2, T3);
      r.vhi[i] = lut16((qq[i] >> 4) & 0x0F0F0F0Fu, T0, T1, T2, T3);
    }
    return r;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    const int4 lo = *(const int4*)(x.q + 32 * u), hi = *(const int4*)(x.q + 32 * u + 16);
    int s = 0;
    s = dot4(r.vlo[0], lo.x, s); s = dot4(r.vlo[1], lo.y, s); s = dot4(r.vlo[2], lo.z, s); s = dot4(r.vlo[3], lo.w, s);
    s = dot4(r.vhi[0], hi.x, s); s = dot4(r.vhi[1], hi.y, s); s = dot4(r.vhi[2], hi.z, s); s = dot4(r.vhi[3], hi.w, s);
    return r.dl * x.d[u] * (float)s;
  }
};

// ------------------------------------------------------------------ IQ2_XXS (vecdotq.cuh:1531-1552)
// LDS tables: the 256-entry grid expanded to 8 magnitudes per entry, and the 128 sign patterns as byte masks.
struct FmtIQ2_XXS {
  static constexpr int QK = 256, BS = 66, AUX = AUX_NONE, TABLE_BYTES = 256 * 8 + 128 * 8;
  struct Regs { float dl; uint2 g[4]; };
  static __device__ __forceinline__ void init_tables(char* tab) {
    const int t = threadIdx.x;
    uint2* grid = (uint2*)tab;
    uint2* sgn = grid + 256;
    const uint32_t code = k_iq2xxs_grid_codes[t];
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t c = (code >> (2 * j)) & 3;
      w[j >> 2] |= (8 + 17 * c + (c >> 1)) << (8 * (j & 3));
    }
    grid[t] = make_uint2(w[0], w[1]);
    if (t < 128) {
      const uint32_t s = t | ((__builtin_popcount(t) & 1) << 7);
      uint32_t m[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) m[j >> 2] |= ((s >> j) & 1 ? 0xFFu : 0u) << (8 * (j & 3));
      sgn[t] = make_uint2(m[0], m[1]);
    }
  }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char* tab) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint2 gq = ld<uint2>(b + 2 + 8 * ib);
    const uint2* grid = (const uint2*)tab;
    const uint2* sgn = grid + 256;
    Regs r;
    r.dl = ld_f16(b) * (0.5f + (float)(gq.y >> 28)) * 0.25f;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint2 mag = grid[(gq.x >> (8 * l)) & 0xFF];
      const uint2 m = sgn[(gq.y >> (7 * l)) & 127];
      r.g[l] = make_uint2(neg_bytes(mag.x, m.x), neg_bytes(mag.y, m.y));
    }
    return r;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    int s = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const int2 a = *(const int2*)(x.q + 32 * u + 8 * l);
      s = dot4((int)r.g[l].x, a.x, s);
      s = dot4((int)r.g[l].y, a.y, s);
    }
    return r.dl * x.d[u] * (float)s;
  }
};

// ------------------------------------------------------------------ kernel
// MOE selects the per-pair variant (reference: csrc/gguf/moe_vec.cuh:3-53): blockIdx.y is the flat
// (token, k) pair z; its expert topk_ids[z] picks the weight matrix (experts densely packed), its
// token z / top_k picks the activation row, and the result goes to row z of Y.
template <class F, int MT, int RPW, typename T, bool MOE>
__global__ __launch_bounds__(256) void mmvq_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                    T* __restrict__ Y, int N, int K, int kchunk, int64_t ws_row_bytes,
                                                    int64_t y_vec_stride, const int32_t* __restrict__ topk_ids,
                                                    int top_k) {
  extern __shared__ __align__(16) char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int Kp = (int)q8_kp(K);
  if (MOE) {
    const int z = blockIdx.y;
    const int e = topk_ids[z];
    W += (int64_t)e * N * ((int64_t)(K / F::QK) * F::BS);
    ws += (int64_t)(z / top_k) * ws_row_bytes;
    Y += (int64_t)z * N;
  }
  int8_t* lq = (int8_t*)smem;                         // [MT][kchunk]
  float* ldv = (float*)(smem + MT * kchunk);          // [MT][kchunk/32]
  float* lav = ldv + MT * (kchunk / 32);              // [MT][kchunk/32]
  char* tab = (char*)(lav + (F::AUX != AUX_NONE ? MT * (kchunk / 32) : 0));
  F::init_tables(tab);

  const int row0 = (blockIdx.x * 4 + wave) * RPW;
  const int64_t rowbytes = (int64_t)(K / F::QK) * F::BS;
  const uint8_t* rows[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) rows[r] = W + (int64_t)min(row0 + r, N - 1) * rowbytes;

  float acc[RPW][MT];
#pragma unroll
  for (int r = 0; r < RPW; ++r)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.0f;

  for (int k0 = 0; k0 < K; k0 += kchunk) {
    const int kc = min(kchunk, K - k0);
    if (k0 > 0) __syncthreads();
    // stage quants (16-byte granules) and block scales of the MT vectors
    const int g16 = kc >> 4;
    for (int i = tid; i < MT * g16; i += 256) {
      const int m = i / g16, j = i - m * g16;
      *(uint4*)(lq + m * kchunk + 16 * j) = *(const uint4*)(ws + m * ws_row_bytes + k0 + 16 * j);
    }
    const int nb = kc >> 5;
    for (int i = tid; i < MT * nb; i += 256) {
      const int m = i / nb, j = i - m * nb;
      const float* fd = (const float*)(ws + m * ws_row_bytes + Kp) + (k0 >> 5) + j;
      ldv[m * (kchunk / 32) + j] = fd[0];
      if (F::AUX == AUX_S8) lav[m * (kchunk / 32) + j] = fd[Kp / 32];
      if (F::AUX == AUX_DU) lav[m * (kchunk / 32) + j] = fd[2 * (Kp / 32)];
    }
    __syncthreads();

    const int u0 = k0 >> 5;  // first unit of this chunk within the row
    for (int u = lane; u < nb; u += 64) {
      typename F::Regs regs[RPW];
#pragma unroll
      for (int r = 0; r < RPW; ++r) regs[r] = F::load(rows[r], u0, u, tab);
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        Act x;
        x.q = lq + m * kchunk;
        x.d = ldv + m * (kchunk / 32);
        x.a = lav + m * (kchunk / 32);
#pragma unroll
        for (int r = 0; r < RPW; ++r) acc[r][m] += F::dot(regs[r], x, u, lane);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < RPW; ++r) {
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      const float v = wave_sum(acc[r][m]);
      if (lane == 0 && row0 + r < N) Y[m * y_vec_stride + row0 + r] = from_f32<T>(v);
    }
  }
}

static inline int kchunk_for(int mt) { return mt == 1 ? 32768 : mt == 2 ? 16384 : mt == 4 ? 8192 : 4096; }

template <class F, int MT, typename T>
static void launch_mt(const void* W, const char* ws, T* Y, int N, int K, hipStream_t stream) {
  constexpr int RPW = 2;
  int kchunk = kchunk_for(MT);
  const int kround = (K + 511) / 512 * 512;
  if (kchunk > kround) kchunk = kround;
  const size_t lds = (size_t)MT * kchunk + (size_t)MT * (kchunk / 32) * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES;
  const int grid = (N + 4 * RPW - 1) / (4 * RPW);
  hipLaunchKernelGGL((mmvq_kernel<F, MT, RPW, T, false>), dim3(grid), dim3(256), lds, stream, (const uint8_t*)W, ws, Y, N,
                     K, kchunk, q8_row_bytes(K), (int64_t)N, (const int32_t*)nullptr, 1);
}

template <class F, typename T>
static int moe_vec_typed(const void* W, const char* ws, void* Y, int N, int K, const int32_t* topk_ids, int top_k,
                         int pairs, hipStream_t stream) {
  constexpr int RPW = 2;
  int kchunk = kchunk_for(1);
  const int kround = (K + 511) / 512 * 512;
  if (kchunk > kround) kchunk = kround;
  const size_t lds = (size_t)kchunk + (size_t)(kchunk / 32) * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES;
  const int grid = (N + 4 * RPW - 1) / (4 * RPW);
  for (int z0 = 0; z0 < pairs; z0 += 65535) {
    const int nz = pairs - z0 < 65535 ? pairs - z0 : 65535;
    // the pair index is rebuilt from blockIdx.y, so later slabs shift the id and output bases by whole tokens
    if (z0 % top_k != 0) return GGUF_ERR_SHAPE;
    hipLaunchKernelGGL((mmvq_kernel<F, 1, RPW, T, true>), dim3(grid, nz), dim3(256), lds, stream, (const uint8_t*)W,
                       ws + (int64_t)(z0 / top_k) * q8_row_bytes(K), (T*)Y + (int64_t)z0 * N, N, K, kchunk, q8_row_bytes(K),
                       (int64_t)N, topk_ids + z0, top_k);
  }
  return launch_status();
}

template <class F>
static int moe_vec_fmt(const void* W, const void* ws, void* Y, int dtype, int N, int K, const int32_t* ids, int top_k,
                       int pairs, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_vec_typed<F, scalar_t>(W, (const char*)ws, Y, N, K, ids, top_k, pairs, s)));
  return GGUF_ERR_DTYPE;
}

template <class F, typename T>
static int mmvq_typed(const void* W, const void* ws, void* Y, int64_t N, int64_t K, int64_t M, hipStream_t stream) {
  const int64_t rb = q8_row_bytes(K);
  int64_t m0 = 0;
  while (m0 < M) {
    const int64_t left = M - m0;
    const char* wsm = (const char*)ws + m0 * rb;
    T* ym = (T*)Y + m0 * N;
    if (left >= 8) { launch_mt<F, 8, T>(W, wsm, ym, (int)N, (int)K, stream); m0 += 8; }
    else if (left >= 4) { launch_mt<F, 4, T>(W, wsm, ym, (int)N, (int)K, stream); m0 += 4; }
    else if (left >= 2) { launch_mt<F, 2, T>(W, wsm, ym, (int)N, (int)K, stream); m0 += 2; }
    else { launch_mt<F, 1, T>(W, wsm, ym, (int)N, (int)K, stream); m0 += 1; }
  }
  return launch_status();
}

int quantize_q8_1(const void* x, int xdtype, void* ws, int64_t M, int64_t K, hipStream_t stream);

template <class F>
static int mmvq_fmt(const void* W, const void* ws, void* Y, int dtype, int64_t N, int64_t K, int64_t M, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (mmvq_typed<F, scalar_t>(W, ws, Y, N, K, M, s)));
  return GGUF_ERR_DTYPE;
}

}  // namespace gguf

extern "C" int gguf_mmvq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N,
                         int64_t K, int64_t M, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (N < 0 || M < 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || M == 0) return GGUF_OK;
  if (!W || !x || !q8_workspace || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  switch (type) {
    case T_Q4_0: case T_Q8_0: case T_Q4_K: case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: break;
    default: return GGUF_ERR_TYPE;
  }
  int rc = quantize_q8_1(x, xdtype, q8_workspace, M, K, s);
  if (rc != GGUF_OK) return rc;
  switch (type) {
    case T_Q4_0: return mmvq_fmt<FmtQ4_0>(W, q8_workspace, Y, xdtype, N, K, M, s);
    case T_Q8_0: return mmvq_fmt<FmtQ8_0>(W, q8_workspace, Y, xdtype, N, K, M, s);
    case T_Q4_K: return mmvq_fmt<FmtQ4_K>(W, q8_workspace, Y, xdtype, N, K, M, s);
    case T_Q6_K: return mmvq_fmt<FmtQ6_K>(W, q8_workspace, Y, xdtype, N, K, M, s);
    case T_IQ4_XS: return mmvq_fmt<FmtIQ4_XS>(W, q8_workspace, Y, xdtype, N, K, M, s);
    case T_IQ2_XXS: return mmvq_fmt<FmtIQ2_XXS>(W, q8_workspace, Y, xdtype, N, K, M, s);
  }
  return GGUF_ERR_TYPE;
}

extern "C" int gguf_moe_vec(const void* X, int xdtype, void* q8_workspace, const void* W, const int32_t* topk_ids, void* Y,
                            int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0) return GGUF_ERR_TYPE;
  if (N < 0 || tokens < 0 || top_k <= 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL ||
      tokens * top_k > 0x7FFFFFF0LL)
    return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  switch (type) {
    case T_Q4_0: case T_Q8_0: case T_Q4_K: case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: break;
    default: return GGUF_ERR_TYPE;
  }
  if (N == 0 || tokens == 0) return GGUF_OK;
  if (!X || !q8_workspace || !W || !topk_ids || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const int rc = quantize_q8_1(X, xdtype, q8_workspace, tokens, K, s);
  if (rc != GGUF_OK) return rc;
  const int pairs = (int)(tokens * top_k);
  switch (type) {
    case T_Q4_0: return moe_vec_fmt<FmtQ4_0>(W, q8_workspace, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, s);
    case T_Q8_0: return moe_vec_fmt<FmtQ8_0>(W, q8_workspace, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, s);
    case T_Q4_K: return moe_vec_fmt<FmtQ4_K>(W, q8_workspace, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, s);
    case T_Q6_K: return moe_vec_fmt<FmtQ6_K>(W, q8_workspace, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, s);
    case T_IQ4_XS: return moe_vec_fmt<FmtIQ4_XS>(W, q8_workspace, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, s);
    case T_IQ2_XXS: return moe_vec_fmt<FmtIQ2_XXS>(W, q8_workspace, Y, xdtype, (int)N, (int)K, topk_ids, (int)top_k, pairs, s);
  }
  return GGUF_ERR_TYPE;
}
