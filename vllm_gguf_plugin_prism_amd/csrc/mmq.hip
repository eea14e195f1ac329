// Prefill-path GEMM on packed GGUF weights with q8_1 activations, on gfx950 int8 MFMA.
//
//   Y[m, n] = sum_kb  d8[m, kb] * dw[n, kb] * S[m, n, kb]  ( - offset terms )
//   S[m, n, kb] = sum over the 32 (or 16) elements of block kb of  xq[m, k] * wq[n, k]      (int32)
//
// The reference computes S with dp4a on the vector ALU from re-packed LDS tiles
// (csrc/gguf/mmq.cuh:2-104, vecdotq.cuh load_tiles_* / vec_dot_*_mul_mat).  Here S is
// one v_mfma_i32_32x32x32_i8 per 32x32 output tile and 32-element block (two
// v_mfma_i32_32x32x16_i8 for formats whose weight scale changes every 16 elements), and
// the vector ALU only rescales: convert, multiply by the activation scale, fused
// multiply-add with the weight scale into an fp32 accumulator.
//
// Work split: a workgroup of four waves owns an (M_T x N_T) output tile and walks K in
// steps of 128 elements.  Per step it stages the q8_1 activations (int8 + block scales)
// and unpacks the GGUF blocks of its N_T weight rows to plain int8 + per-block fp32
// scales in LDS; every wave then owns a (32*TM x 32*TN) sub-tile.  MFMA operands:
// A = activations (rows = tokens), B = weights (columns = output features), so a lane
// holds one output feature n and 16 token rows, the weight scale is a per-lane scalar
// and stores to Y are contiguous across lanes.
//
// The same kernel runs the grouped MoE contraction (reference: csrc/gguf/moe.cuh:5-129):
// token rows are gathered through sorted_token_ids, the weight base moves to the block's
// expert, and results scatter to the rows the slots name.
#include "gguf_common.h"
#include "grid_codes.h"

namespace gguf {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int KS = 128;     // K elements per step
constexpr int LDK = KS + 16; // LDS row pitch in bytes: 16-byte skew keeps b128 operand reads conflict-free

// --------------------------------------------------------------------------------------------
// Format policies: unpack one 32-element block of one weight row to int8 (8 dwords, element order)
// plus fp32 scale(s) and, where the format has one, the fp32 offset factor multiplied by the
// activation block's stored sum (the MMQ semantics, vecdotq.cuh:369-372, 61-64).
// --------------------------------------------------------------------------------------------
struct MQ4_0 {  // vecdotq.cuh:46-66, 511-571
  static constexpr int QK = 32, BS = 18, G = 32;
  static constexpr bool HAS_MIN = true;
  static __device__ __forceinline__ void unpack(const uint8_t* row, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const uint8_t* b = row + (int64_t)kb * BS;
    const uint4 v = ld<uint4>(b + 2);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = w[i] & 0x0F0F0F0Fu; q[4 + i] = (w[i] >> 4) & 0x0F0F0F0Fu; }
    s0 = ld_f16(b); s1 = s0; mn = 8.0f * s0;
  }
};

struct MQ8_0 {  // vecdotq.cuh:165-177, 869-921
  static constexpr int QK = 32, BS = 34, G = 32;
  static constexpr bool HAS_MIN = false;
  static __device__ __forceinline__ void unpack(const uint8_t* row, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const uint8_t* b = row + (int64_t)kb * BS;
    const uint4 v0 = ld<uint4>(b + 2), v1 = ld<uint4>(b + 18);
    q[0] = v0.x; q[1] = v0.y; q[2] = v0.z; q[3] = v0.w; q[4] = v1.x; q[5] = v1.y; q[6] = v1.z; q[7] = v1.w;
    s0 = ld_f16(b); s1 = s0; mn = 0.0f;
  }
};

struct MQ4_K {  // vecdotq.cuh:353-379, 1204-1277
  static constexpr int QK = 256, BS = 144, G = 32;
  static constexpr bool HAS_MIN = true;
  static __device__ __forceinline__ void unpack(const uint8_t* row, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const int sb = kb >> 3, j = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint4 hdr = ld<uint4>(b);
    const uint4 v0 = ld<uint4>(b + 16 + 32 * (j >> 1)), v1 = ld<uint4>(b + 32 + 32 * (j >> 1));
    const int sh = (j & 1) ? 4 : 0;
    const uint32_t w[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) q[i] = (w[i] >> sh) & 0x0F0F0F0Fu;
    const uint32_t sw[3] = {hdr.y, hdr.z, hdr.w};
    const uint8_t* s = (const uint8_t*)sw;
    int sc, m;
    if (j < 4) { sc = s[j] & 63; m = s[j + 4] & 63; }
    else { sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4); m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4); }
    const float d = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x & 0xFFFF));
    const float dmin = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x >> 16));
    s0 = d * (float)sc; s1 = s0; mn = dmin * (float)m;
  }
};

struct MQ6_K {  // vecdotq.cuh:467-491, 1443-1529: two int8 sub-scales per q8_1 block
  static constexpr int QK = 256, BS = 210, G = 16;
  static constexpr bool HAS_MIN = false;
  static __device__ __forceinline__ void unpack(const uint8_t* row, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const int sb = kb >> 3, h = (kb >> 2) & 1, t = kb & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint8_t* pl = b + 64 * h + 32 * (t & 1);
    const uint8_t* ph = b + 128 + 32 * h;
    const uint4 l0 = ld<uint4>(pl), l1 = ld<uint4>(pl + 16), h0 = ld<uint4>(ph), h1 = ld<uint4>(ph + 16);
    const uint32_t lw[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
    const uint32_t hw[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
    const int shl = (t >> 1) ? 4 : 0, shh = 2 * t;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t v = ((lw[i] >> shl) & 0x0F0F0F0Fu) | (((hw[i] >> shh) & 0x03030303u) << 4);
      q[i] = ((v | 0x80808080u) - 0x20202020u) ^ 0x80808080u;  // every byte minus 32, no borrow between bytes
    }
    const float d = ld_f16(b + 208);
    s0 = d * (float)(int8_t)b[192 + 8 * h + 2 * t];
    s1 = d * (float)(int8_t)b[192 + 8 * h + 2 * t + 1];
    mn = 0.0f;
  }
};

__device__ __forceinline__ int lut16q(uint32_t idx) {  // kvalues_iq4nl lookup of four indices, one per byte
  constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
  const uint32_t sel = idx & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(T1, T0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(T3, T2, sel);
  const uint32_t m = ((idx >> 3) & 0x01010101u) * 0xFFu;
  return (int)((hi & m) | (lo & ~m));
}

struct MIQ4_XS {  // extension: the reference has no MMQ tiles for i-quants (gguf_kernel.cu:236-287)
  static constexpr int QK = 256, BS = 136, G = 32;
  static constexpr bool HAS_MIN = false;
  static __device__ __forceinline__ void unpack(const uint8_t* row, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const int sb = kb >> 3, ib = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint2 hdr = ld<uint2>(b);
    const uint4 v = ld<uint4>(b + 8 + 16 * ib);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { q[i] = (uint32_t)lut16q(w[i] & 0x0F0F0F0Fu); q[4 + i] = (uint32_t)lut16q((w[i] >> 4) & 0x0F0F0F0Fu); }
    const int ls = (int)(((hdr.y >> (4 * ib)) & 0xF) | ((((hdr.x >> 16) >> (2 * ib)) & 3) << 4));
    s0 = (float)__builtin_bit_cast(_Float16, (uint16_t)(hdr.x & 0xFFFF)) * (float)(ls - 32);
    s1 = s0; mn = 0.0f;
  }
};

struct MIQ2_XXS {  // extension, see MIQ4_XS
  static constexpr int QK = 256, BS = 66, G = 32;
  static constexpr bool HAS_MIN = false;
  static __device__ __forceinline__ void unpack(const uint8_t* row, int kb, uint32_t (&q)[8], float& s0, float& s1, float& mn) {
    const int sb = kb >> 3, ib = kb & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    const uint2 g = ld<uint2>(b + 2 + 8 * ib);
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t code = k_iq2xxs_grid_codes[(g.x >> (8 * l)) & 0xFF];
      const uint32_t s7 = (g.y >> (7 * l)) & 127;
      const uint32_t sg = s7 | ((__builtin_popcount(s7) & 1) << 7);
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t c = (code >> (2 * j)) & 3;
        const uint32_t mag = 8 + 17 * c + (c >> 1);
        const uint32_t val = ((sg >> j) & 1) ? (0u - mag) & 0xFFu : mag;
        w[j >> 2] |= val << (8 * (j & 3));
      }
      q[2 * l] = w[0]; q[2 * l + 1] = w[1];
    }
    s0 = ld_f16(b) * (0.5f + (float)(g.y >> 28)) * 0.25f;
    s1 = s0; mn = 0.0f;
  }
};

// --------------------------------------------------------------------------------------------
struct MoeArgs {
  const int32_t* sorted_token_ids;
  const int32_t* expert_ids;
  const int32_t* num_tokens_post_padded;
  int64_t expert_stride;  // bytes
  int top_k;
  int num_pairs;          // tokens * top_k
};

template <class F, int WM, int WN, int TM, int TN, typename T, bool MOE>
__global__ __launch_bounds__(256, 2) void mmq_kernel(const uint8_t* __restrict__ W, const char* __restrict__ ws,
                                                       T* __restrict__ Y, int M, int N, int K, int64_t ws_row_bytes,
                                                       MoeArgs moe) {
  static_assert(WM * WN == 4, "four waves per workgroup");
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  constexpr int NG = KS / F::G;  // weight scales per row per step
  extern __shared__ __align__(16) char smem[];
  int8_t* xq = (int8_t*)smem;                       // [M_T][LDK]
  int8_t* wq = xq + M_T * LDK;                      // [N_T][LDK]
  float* xd = (float*)(wq + N_T * LDK);             // [4][M_T]
  float* xa = xd + 4 * M_T;                         // [4][M_T]   (HAS_MIN)
  float* wsc = xa + (F::HAS_MIN ? 4 * M_T : 0);     // [NG][N_T]
  float* wmn = wsc + NG * N_T;                      // [4][N_T]   (HAS_MIN)

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave / WN, wn = wave % WN;
  const int m_base = blockIdx.y * M_T, n_base = blockIdx.x * N_T;
  const int Kp = (int)q8_kp(K);
  const int64_t rowbytes = (int64_t)(K / F::QK) * F::BS;

  if (MOE) {
    if (m_base >= moe.num_tokens_post_padded[0]) return;
    static_assert(!MOE || M_T == 32, "one expert per 32 sorted slots");
    const int e = moe.expert_ids[blockIdx.y];
    if (e < 0 || e > 255) return;
    W += (int64_t)e * moe.expert_stride;
  }

  // source row of X (and destination row of Y) of every tile row this thread stages / stores
  float acc[TM][TN][16];
#pragma unroll
  for (int j = 0; j < TM; ++j)
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][i][r] = 0.0f;

  const int lrow = lane & 31, lhalf = lane >> 5;

  for (int k0 = 0; k0 < K; k0 += KS) {
    const int nkb = min(4, (K - k0) >> 5);
    __syncthreads();
    // ---- stage activations: 16-byte granules of int8, then block scales (transposed to [kb][m])
    for (int p = tid; p < M_T * 8; p += 256) {
      const int m = p >> 3, g = p & 7;
      int src = m_base + m;
      bool valid = true;
      if (MOE) {
        const int pair = moe.sorted_token_ids[src];
        valid = pair < moe.num_pairs;
        src = valid ? pair / moe.top_k : 0;
      } else {
        src = min(src, M - 1);
      }
      uint4 v = make_uint4(0, 0, 0, 0);
      if (valid && (g >> 1) < nkb) v = *(const uint4*)(ws + (int64_t)src * ws_row_bytes + k0 + 16 * g);
      *(uint4*)(xq + m * LDK + 16 * g) = v;
    }
    for (int p = tid; p < M_T * 4; p += 256) {
      const int m = p >> 2, kb = p & 3;
      int src = m_base + m;
      bool valid = kb < nkb;
      if (MOE) {
        const int pair = moe.sorted_token_ids[src];
        valid = valid && pair < moe.num_pairs;
        src = valid ? pair / moe.top_k : 0;
      } else {
        src = min(src, M - 1);
      }
      const float* fd = (const float*)(ws + (int64_t)src * ws_row_bytes + Kp) + (k0 >> 5) + kb;
      xd[kb * M_T + m] = valid ? fd[0] : 0.0f;
      if (F::HAS_MIN) xa[kb * M_T + m] = valid ? fd[Kp / 32] : 0.0f;
    }
    // ---- unpack weights: one (row, 32-block) pair per thread and pass
    for (int p = tid; p < N_T * 4; p += 256) {
      const int n = p >> 2, kb = p & 3;
      uint32_t q[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      float s0 = 0.0f, s1 = 0.0f, mn = 0.0f;
      if (kb < nkb) {
        const uint8_t* row = W + (int64_t)min(n_base + n, N - 1) * rowbytes;
        F::unpack(row, (k0 >> 5) + kb, q, s0, s1, mn);
      }
      *(uint4*)(wq + n * LDK + 32 * kb) = make_uint4(q[0], q[1], q[2], q[3]);
      *(uint4*)(wq + n * LDK + 32 * kb + 16) = make_uint4(q[4], q[5], q[6], q[7]);
      if (F::G == 32) {
        wsc[kb * N_T + n] = s0;
      } else {
        wsc[(2 * kb) * N_T + n] = s0;
        wsc[(2 * kb + 1) * N_T + n] = s1;
      }
      if (F::HAS_MIN) wmn[kb * N_T + n] = mn;
    }
    __syncthreads();

    // ---- contract
#pragma unroll 1
    for (int kb = 0; kb < nkb; ++kb) {
      float d8[TM][16];
      float a8[TM][16];
      v4i af[TM];
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        const int mrow = 32 * (wm * TM + j);
        af[j] = *(const v4i*)(xq + (mrow + lrow) * LDK + 32 * kb + 16 * lhalf);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float4 v = *(const float4*)(xd + kb * M_T + mrow + 8 * g + 4 * lhalf);
          d8[j][4 * g] = v.x; d8[j][4 * g + 1] = v.y; d8[j][4 * g + 2] = v.z; d8[j][4 * g + 3] = v.w;
          if (F::HAS_MIN) {
            const float4 u = *(const float4*)(xa + kb * M_T + mrow + 8 * g + 4 * lhalf);
            a8[j][4 * g] = u.x; a8[j][4 * g + 1] = u.y; a8[j][4 * g + 2] = u.z; a8[j][4 * g + 3] = u.w;
          }
        }
      }
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int ncol = 32 * (wn * TN + i) + lrow;
        const v4i bf = *(const v4i*)(wq + ncol * LDK + 32 * kb + 16 * lhalf);
        if (F::G == 32) {
          const float dw = wsc[kb * N_T + ncol];
          const float mw = F::HAS_MIN ? wmn[kb * N_T + ncol] : 0.0f;
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            v16i s = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            s = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[j], bf, s, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              acc[j][i][r] = __builtin_fmaf((float)s[r] * d8[j][r], dw, acc[j][i][r]);
              if (F::HAS_MIN) acc[j][i][r] = __builtin_fmaf(-a8[j][r], mw, acc[j][i][r]);
            }
          }
        } else {
          // weight scale changes every 16 elements: the K=16 MFMA takes the low / high 8 bytes of each lane's 16
          const float dwa = wsc[(2 * kb) * N_T + ncol], dwb = wsc[(2 * kb + 1) * N_T + ncol];
          // lane half h holds k = 16h..16h+15 of the block, but a 16-element group needs k = 8h'..8h'+7 from both
          // halves; re-read the operands with the K=16 addressing instead
          const long b0 = *(const long*)(wq + ncol * LDK + 32 * kb + 8 * lhalf);
          const long b1 = *(const long*)(wq + ncol * LDK + 32 * kb + 16 + 8 * lhalf);
#pragma unroll
          for (int j = 0; j < TM; ++j) {
            const int mrow = 32 * (wm * TM + j);
            const long a0 = *(const long*)(xq + (mrow + lrow) * LDK + 32 * kb + 8 * lhalf);
            const long a1 = *(const long*)(xq + (mrow + lrow) * LDK + 32 * kb + 16 + 8 * lhalf);
            v16i sa = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, sb2 = sa;
            sa = __builtin_amdgcn_mfma_i32_32x32x16_i8(a0, b0, sa, 0, 0, 0);
            sb2 = __builtin_amdgcn_mfma_i32_32x32x16_i8(a1, b1, sb2, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              const float t = __builtin_fmaf((float)sb2[r], dwb, (float)sa[r] * dwa);
              acc[j][i][r] = __builtin_fmaf(t, d8[j][r], acc[j][i][r]);
            }
          }
        }
      }
    }
  }

  // ---- store: lane = one output feature, 16 token rows per tile
#pragma unroll
  for (int j = 0; j < TM; ++j) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int mt = m_base + 32 * (wm * TM + j) + 8 * (r >> 2) + 4 * lhalf + (r & 3);
      int64_t dst;
      bool ok;
      if (MOE) {
        const int pair = moe.sorted_token_ids[mt];
        ok = pair < moe.num_pairs;
        dst = pair;
      } else {
        ok = mt < M;
        dst = mt;
      }
#pragma unroll
      for (int i = 0; i < TN; ++i) {
        const int n = n_base + 32 * (wn * TN + i) + lrow;
        if (ok && n < N) Y[dst * N + n] = from_f32<T>(acc[j][i][r]);
      }
    }
  }
}

template <class F, int WM, int WN, int TM, int TN, bool MOE>
static constexpr size_t mmq_lds_bytes() {
  constexpr int M_T = 32 * WM * TM, N_T = 32 * WN * TN;
  return (size_t)(M_T + N_T) * LDK + (size_t)4 * M_T * 4 * (F::HAS_MIN ? 2 : 1) + (size_t)(KS / F::G) * N_T * 4 +
         (F::HAS_MIN ? (size_t)4 * N_T * 4 : 0);
}

template <class F, int WM, int WN, int TM, int TN, typename T, bool MOE>
static void launch_mmq(const void* W, const void* ws, void* Y, int M, int N, int K, int m_tiles, const MoeArgs& moe,
                       hipStream_t stream) {
  constexpr int N_T = 32 * WN * TN;
  constexpr size_t lds = mmq_lds_bytes<F, WM, WN, TM, TN, MOE>();
  auto kern = mmq_kernel<F, WM, WN, TM, TN, T, MOE>;
  static bool configured = false;  // opt in to > 64 KB of dynamic LDS once per instantiation
  if (!configured) {
    (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    configured = true;
  }
  hipLaunchKernelGGL(kern, dim3((N + N_T - 1) / N_T, m_tiles), dim3(256), lds, stream, (const uint8_t*)W, (const char*)ws,
                     (T*)Y, M, N, K, q8_row_bytes(K), moe);
}

int quantize_q8_1(const void* x, int xdtype, void* ws, int64_t M, int64_t K, hipStream_t stream);

template <class F, typename T>
static int mmq_typed(const void* W, const void* ws, void* Y, int M, int N, int K, hipStream_t stream) {
  MoeArgs none = {};
  if (M <= 64) {
    launch_mmq<F, 2, 2, 1, 2, T, false>(W, ws, Y, M, N, K, (M + 63) / 64, none, stream);      // 64 x 128
  } else {
    launch_mmq<F, 2, 2, 2, 2, T, false>(W, ws, Y, M, N, K, (M + 127) / 128, none, stream);    // 128 x 128
  }
  return launch_status();
}

template <class F>
static int mmq_fmt(const void* W, const void* ws, void* Y, int dtype, int M, int N, int K, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (mmq_typed<F, scalar_t>(W, ws, Y, M, N, K, s)));
  return GGUF_ERR_DTYPE;
}

template <class F, typename T>
static int moe_typed(const void* W, const void* ws, void* Y, int N, int K, int num_sorted, const MoeArgs& moe,
                     hipStream_t stream) {
  launch_mmq<F, 1, 4, 1, 2, T, true>(W, ws, Y, 0, N, K, num_sorted / 32, moe, stream);  // 32 slots x 256
  return launch_status();
}

template <class F>
static int moe_fmt(const void* W, const void* ws, void* Y, int dtype, int N, int K, int num_sorted, const MoeArgs& moe,
                   hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_typed<F, scalar_t>(W, ws, Y, N, K, num_sorted, moe, s)));
  return GGUF_ERR_DTYPE;
}

__global__ void zero_rows_kernel(uint4* __restrict__ p, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) p[i] = make_uint4(0, 0, 0, 0);
}

static bool mmq_type_ok(int type) {
  switch (type) {
    case T_Q4_0: case T_Q8_0: case T_Q4_K: case T_Q6_K: case T_IQ4_XS: case T_IQ2_XXS: return true;
    default: return false;
  }
}

}  // namespace gguf

extern "C" int gguf_mmq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N,
                        int64_t K, int64_t M, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0 || !mmq_type_ok(type)) return GGUF_ERR_TYPE;
  if (N < 0 || M < 0 || K <= 0 || K % qk != 0 || N > 0x7FFFFFF0LL || K > 0x7FFFFFF0LL || M > 0x7FFFFFF0LL) return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || M == 0) return GGUF_OK;
  if (!W || !x || !q8_workspace || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const int rc = quantize_q8_1(x, xdtype, q8_workspace, M, K, s);
  if (rc != GGUF_OK) return rc;
  switch (type) {
    case T_Q4_0: return mmq_fmt<MQ4_0>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_Q8_0: return mmq_fmt<MQ8_0>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_Q4_K: return mmq_fmt<MQ4_K>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_Q6_K: return mmq_fmt<MQ6_K>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_IQ4_XS: return mmq_fmt<MIQ4_XS>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
    case T_IQ2_XXS: return mmq_fmt<MIQ2_XXS>(W, q8_workspace, Y, xdtype, (int)M, (int)N, (int)K, s);
  }
  return GGUF_ERR_TYPE;
}

extern "C" int gguf_moe_block_size(int type) { return gguf::block_elems(type) ? 32 : 0; }

extern "C" int gguf_moe_mmq(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                            const int32_t* sorted_token_ids, const int32_t* expert_ids,
                            const int32_t* num_tokens_post_padded, int64_t num_sorted, void* Y, int type, int64_t N,
                            int64_t K, int64_t top_k, int64_t tokens, gguf_stream_t stream) {
  using namespace gguf;
  const int qk = block_elems(type);
  if (qk == 0 || !mmq_type_ok(type)) return GGUF_ERR_TYPE;
  if (N < 0 || tokens < 0 || top_k <= 0 || num_sorted < 0 || K <= 0 || K % qk != 0 || expert_stride_bytes < 0 ||
      tokens * top_k > 0x7FFFFFF0LL || N > 0x7FFFFFF0LL)
    return GGUF_ERR_SHAPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (N == 0 || tokens == 0) return GGUF_OK;
  if (!X || !q8_workspace || !W || !sorted_token_ids || !expert_ids || !num_tokens_post_padded || !Y) return GGUF_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  // rows that no slot names stay zero, as with the reference's zero-filled output (gguf_kernel.cu:301-302)
  const int64_t ybytes = tokens * top_k * N * (xdtype == GGUF_DTYPE_F32 ? 4 : 2);
  const int64_t n16 = ybytes / 16;
  if (ybytes % 16 != 0) return GGUF_ERR_SHAPE;
  hipLaunchKernelGGL(zero_rows_kernel, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, s, (uint4*)Y, n16);
  const int rc = quantize_q8_1(X, xdtype, q8_workspace, tokens, K, s);
  if (rc != GGUF_OK) return rc;
  MoeArgs moe = {sorted_token_ids, expert_ids, num_tokens_post_padded, expert_stride_bytes, (int)top_k, (int)(tokens * top_k)};
  const int ns = (int)(num_sorted / 32 * 32);  // a trailing partial block is ignored, like the reference's integer division
  if (ns == 0) return launch_status();
  switch (type) {
    case T_Q4_0: return moe_fmt<MQ4_0>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_Q8_0: return moe_fmt<MQ8_0>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_Q4_K: return moe_fmt<MQ4_K>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_Q6_K: return moe_fmt<MQ6_K>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_IQ4_XS: return moe_fmt<MIQ4_XS>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
    case T_IQ2_XXS: return moe_fmt<MIQ2_XXS>(W, q8_workspace, Y, xdtype, (int)N, (int)K, ns, moe, s);
  }
  return GGUF_ERR_TYPE;
}
