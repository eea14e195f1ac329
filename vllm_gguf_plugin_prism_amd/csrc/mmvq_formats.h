// Per-format pieces of the GEMV kernels: how one lane fetches the 32 weights of a "unit", which quantized
// activations belong to them, and the block dot product of the reference's vec_dot_<fmt>_q8_1
// (csrc/gguf/vecdotq.cuh, cited at each format).  Included by mmvq_core.h inside its declarations.
#pragma once

namespace gguf {

// ------------------------------------------------------------------ Q4_0 (vecdotq.cuh:46-66,493-509)
struct FmtQ4_0 {
  static constexpr int QK = 32, BS = 18, AUX = AUX_S8, TABLE_BYTES = 0;
  struct Regs { uint16_t d; uint4 q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    uint32_t w[5];
    const uint32_t sh = ld_block_dwords(row + (int64_t)(u0 + u) * BS, w);
    return cut(w, sh);
  }
  static __device__ __forceinline__ Regs cut(const uint32_t (&w)[5], uint32_t sh) {
    const uint32_t shq = sh + 16;
    Regs r;
    r.d = (uint16_t)(w[0] >> sh);
    r.q = make_uint4(funnel(w[0], w[1], shq), funnel(w[1], w[2], shq), funnel(w[2], w[3], shq), funnel(w[3], w[4], shq));
    return r;
  }
  // The 64 blocks a wave covers, 1152 contiguous bytes, copied to LDS: lane l cuts block l out of the dwords that cover
  // it (the last block may touch the dword behind the span).
  static constexpr int SPAN = 64 * BS, SPAN_SLACK = 16;
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    uint32_t w[5];
    const uint32_t sh = lds_block_dwords(span, lane * BS, w);
    return cut(w, sh);
  }
  struct ActRegs { int4 lo, hi; float d, a; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    ActRegs a; a.lo = *(const int4*)(x.q + 32 * u); a.hi = *(const int4*)(x.q + 32 * u + 16); a.d = x.d[u]; a.a = x.a[u];
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = dot4((int)(q[i] & 0x0F0F0F0Fu), al[i], s);
      s = dot4((int)((q[i] >> 4) & 0x0F0F0F0Fu), ah[i], s);
    }
    return h2f(r.d) * ((float)s * x.d - 8.0f * x.a);
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    return dot(r, load_act(x, u), u);
  }
};

// ------------------------------------------------------------------ Q8_0 (vecdotq.cuh:165-177,852-867)
struct FmtQ8_0 {
  static constexpr int QK = 32, BS = 34, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { uint16_t d; uint4 q0, q1; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    uint32_t w[9];
    const uint32_t sh = ld_block_dwords(row + (int64_t)(u0 + u) * BS, w);
    return cut(w, sh);
  }
  static __device__ __forceinline__ Regs cut(const uint32_t (&w)[9], uint32_t sh) {
    const uint32_t shq = sh + 16;
    Regs r;
    r.d = (uint16_t)(w[0] >> sh);
    r.q0 = make_uint4(funnel(w[0], w[1], shq), funnel(w[1], w[2], shq), funnel(w[2], w[3], shq), funnel(w[3], w[4], shq));
    r.q1 = make_uint4(funnel(w[4], w[5], shq), funnel(w[5], w[6], shq), funnel(w[6], w[7], shq), funnel(w[7], w[8], shq));
    return r;
  }
  static constexpr int SPAN = 64 * BS, SPAN_SLACK = 16;   // 2176 bytes: three pieces for the first eight lanes
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    uint32_t w[9];
    const uint32_t sh = lds_block_dwords(span, lane * BS, w);
    return cut(w, sh);
  }
  struct ActRegs { int4 a0, a1; float d; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    ActRegs a; a.a0 = *(const int4*)(x.q + 32 * u); a.a1 = *(const int4*)(x.q + 32 * u + 16); a.d = x.d[u];
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    int s = 0;
    s = dot4((int)r.q0.x, x.a0.x, s); s = dot4((int)r.q0.y, x.a0.y, s); s = dot4((int)r.q0.z, x.a0.z, s); s = dot4((int)r.q0.w, x.a0.w, s);
    s = dot4((int)r.q1.x, x.a1.x, s); s = dot4((int)r.q1.y, x.a1.y, s); s = dot4((int)r.q1.z, x.a1.z, s); s = dot4((int)r.q1.w, x.a1.w, s);
    return h2f(r.d) * x.d * (float)s;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    return dot(r, load_act(x, u), u);
  }
};

// ------------------------------------------------------------------ Q4_K (vecdotq.cuh:328-351,1159-1202)
// unit c of a super-block: 16 bytes of qs = 16 low nibbles of sub-block 2g and 16 high nibbles of 2g+1
struct FmtQ4_K {
  static constexpr int QK = 256, BS = 144, AUX = AUX_DU, TABLE_BYTES = 0;
  struct Regs { uint4 hdr, q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.hdr = ld<uint4>(b); r.q = ld<uint4>(b + 16 + 16 * c); return r;
  }
  // The 64 units a wave covers are 8 whole blocks, 1152 contiguous bytes; from a copy of them in LDS lane l takes the
  // header of block l / 8 and its own 16 bytes of qs.
  static constexpr int SPAN = 8 * BS;
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    const char* b = span + (lane >> 3) * BS;
    Regs r; r.hdr = *(const uint4*)b; r.q = *(const uint4*)(b + 16 + 16 * (lane & 7)); return r;
  }
  struct ActRegs { int4 lo, hi; float2 d8, du; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    const int sb = u >> 3, c = u & 7, g = c >> 1, h = c & 1;
    const int8_t* qa = x.q + 256 * sb + 64 * g + 16 * h;
    ActRegs a;
    a.lo = *(const int4*)qa; a.hi = *(const int4*)(qa + 32);
    a.d8 = *(const float2*)(x.d + 8 * sb + 2 * g);
    a.du = *(const float2*)(x.a + 8 * sb + 2 * g);
    if (h) a.du = make_float2(0.0f, 0.0f);  // the offset term of a sub-block pair is added once, by its first unit
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const int g = (u & 7) >> 1;
    // 6-bit scales and mins of sub-blocks 2g and 2g+1 (dequantize.cuh:156-163 in 16-bit lanes)
    const int sh = 16 * (g & 1);
    const uint32_t A = (r.hdr.y >> sh) & 0xFFFF, B = (r.hdr.z >> sh) & 0xFFFF, C = (r.hdr.w >> sh) & 0xFFFF;
    uint32_t a0, a1;
    if (g < 2) {
      a0 = A & 0x3F3F; a1 = B & 0x3F3F;
    } else {
      a0 = (C & 0x0F0F) | ((A & 0xC0C0) >> 2);
      a1 = ((C >> 4) & 0x0F0F) | ((B & 0xC0C0) >> 2);
    }
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s0 = 0, s1 = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s0 = dot4((int)(q[i] & 0x0F0F0F0Fu), al[i], s0);
      s1 = dot4((int)((q[i] >> 4) & 0x0F0F0F0Fu), ah[i], s1);
    }
    // (|s| * scale < 2^21: the product of the two converted factors is the converted integer product, bit for bit, and
    //  a float multiply issues at four times the rate of a 32-bit integer one)
    const float pos = x.d8.x * ((float)s0 * (float)(a0 & 0xFF)) + x.d8.y * ((float)s1 * (float)(a0 >> 8));
    const float neg = x.du.x * (float)(a1 & 0xFF) + x.du.y * (float)(a1 >> 8);
    return h2f(r.hdr.x & 0xFFFF) * pos - h2f(r.hdr.x >> 16) * neg;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    return dot(r, load_act(x, u), u);
  }
};

// Selector of the byte permute that gathers bytes h, 2 + h, 4 + h, 6 + h of eight, h = bit 1 of the unit's column group:
// the per-group scale bytes of unit u in the Q6_K arrangement of units (also Q2_K's and Q3_K's)
__device__ __forceinline__ uint32_t k8_group_bytes(int u) { return (u & 2) ? 0x07050301u : 0x06040200u; }

// ------------------------------------------------------------------ Q6_K (vecdotq.cuh:447-465,1417-1441)
// unit c of a super-block: half h = c>>2, columns l in [8*(c&3), +8) of that half; covers elements
// 128h + 32t + l for t = 0..3, i.e. eight values in each of four q8_1 blocks.
struct FmtQ6_K {
  static constexpr int QK = 256, BS = 210, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { uint2 qla, qlb, qh, sc; uint16_t d; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7, h = c >> 2, cc = c & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r;
    r.qla = ld<uint2>(b + 64 * h + 8 * cc);
    r.qlb = ld<uint2>(b + 64 * h + 32 + 8 * cc);
    r.qh = ld<uint2>(b + 128 + 32 * h + 8 * cc);
    r.sc = ld<uint2>(b + 192 + 8 * h);
    r.d = ld<uint16_t>(b + 208);
    return r;
  }
  // The 64 units a wave covers are 8 whole blocks, 1680 contiguous bytes.  In the copy of them in LDS the blocks with
  // an odd number start two bytes into a dword (210 = 4 * 52 + 2): a lane reads the dwords that cover a field and
  // cuts it out with funnel shifts.  (The last field of the last block may touch the dword behind the span.)
  static constexpr int SPAN = 8 * BS, SPAN_SLACK = 16;
  static constexpr bool SPAN_ANY = true;   // the copy may start at any even offset `at` of its first 16 bytes
  static __device__ __forceinline__ Regs from_span(const char* span, int lane, int at = 0) {
    const int c = lane & 7, h = c >> 2, cc = c & 3, b = at + (lane >> 3) * BS;
    Regs r;
    r.qla = lds_cut8(span, b + 64 * h + 8 * cc);
    r.qlb = lds_cut8(span, b + 64 * h + 32 + 8 * cc);
    r.qh = lds_cut8(span, b + 128 + 32 * h + 8 * cc);
    r.sc = lds_cut8(span, b + 192 + 8 * h);
    uint32_t w[1];
    const uint32_t sh = lds_block_dwords(span, b + 208, w);
    r.d = (uint16_t)(w[0] >> sh);
    return r;
  }
  // `off`: the sum of the lane's eight quants of block t times the offset of the format's codes (32 here)
  struct ActRegs { int2 a[4]; float d8[4]; int off[4]; };
  template <int OFFSET>
  static __device__ __forceinline__ ActRegs load_act_off(const Act& x, int u) {
    const int sb = u >> 3, c = u & 7, h = c >> 2, cc = c & 3;
    const int8_t* qa = x.q + 256 * sb + 128 * h + 8 * cc;
    ActRegs a;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      a.a[t] = *(const int2*)(qa + 32 * t);
      a.d8[t] = x.d[8 * sb + 4 * h + t];
      a.off[t] = OFFSET * dot4(0x01010101, a.a[t].x, dot4(0x01010101, a.a[t].y, 0));
    }
    return a;
  }
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return load_act_off<32>(x, u); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    // the signed scales of the lane's four 16-value groups are bytes h, 2 + h, 4 + h, 6 + h of the eight it holds:
    // one byte permute gathers them (a 64-bit shift per group took three instructions each)
    const uint32_t sc4 = __builtin_amdgcn_perm(r.sc.y, r.sc.x, k8_group_bytes(u));
    float acc = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint2 ql = (t & 1) ? r.qlb : r.qla;
      const int shl = (t >> 1) ? 4 : 0;
      const int vx = (int)(((ql.x >> shl) & 0x0F0F0F0Fu) | (((r.qh.x >> (2 * t)) & 0x03030303u) << 4));
      const int vy = (int)(((ql.y >> shl) & 0x0F0F0F0Fu) | (((r.qh.y >> (2 * t)) & 0x03030303u) << 4));
      const int s = dot4(vx, x.a[t].x, dot4(vy, x.a[t].y, 0)) - x.off[t];
      const int sc = (int)(int8_t)(sc4 >> (8 * t));
      // (|sc * s| < 2^23: the product of the converted factors is the converted integer product, bit for bit, and a
      //  float multiply issues at four times the rate of a 32-bit integer one)
      acc += x.d8[t] * ((float)sc * (float)s);
    }
    return h2f(r.d) * acc;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    return dot(r, load_act(x, u), u);
  }
};

// 16-entry signed byte table lookup of four 4-bit indices held one per byte
// Bytes of `w`, shifted right by SH (0 or 4), hold four 4-bit table indices; the 16 table bytes are t0..t3.  Bits 0-2 pick a
// byte out of either half of the table, and a third byte permute takes byte i of the half that bit 3 of index i names:
// its selector is i, or 4 + i, which is (w >> (SH + 1)) & 4 in every byte on top of 0x03020100.
template <int SH>
__device__ __forceinline__ int lut16(uint32_t w, uint32_t t0, uint32_t t1, uint32_t t2, uint32_t t3) {
  const uint32_t sel = (SH ? w >> SH : w) & 0x07070707u;
  const uint32_t lo = __builtin_amdgcn_perm(t1, t0, sel);
  const uint32_t hi = __builtin_amdgcn_perm(t3, t2, sel);
  const uint32_t pick = ((w >> (SH + 1)) & 0x04040404u) | 0x03020100u;
  return (int)__builtin_amdgcn_perm(hi, lo, pick);
}

// ------------------------------------------------------------------ IQ4_XS (vecdotq.cuh:1791-1811)
struct FmtIQ4_XS {
  static constexpr int QK = 256, BS = 136, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { uint2 hdr; uint4 q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.hdr = ld<uint2>(b); r.q = ld<uint4>(b + 8 + 16 * ib); return r;
  }
  struct ActRegs { int4 lo, hi; float d; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    ActRegs a; a.lo = *(const int4*)(x.q + 32 * u); a.hi = *(const int4*)(x.q + 32 * u + 16); a.d = x.d[u];
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const int ib = u & 7;
    const int ls = (int)(((r.hdr.y >> (4 * ib)) & 0xF) | ((((r.hdr.x >> 16) >> (2 * ib)) & 3) << 4));
    const float dl = h2f(r.hdr.x & 0xFFFF) * (float)(ls - 32);
    // kvalues_iq4nl as four little-endian words
    constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
    const uint32_t qq[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = dot4(lut16<0>(qq[i], T0, T1, T2, T3), al[i], s);
      s = dot4(lut16<4>(qq[i], T0, T1, T2, T3), ah[i], s);
    }
    return dl * x.d * (float)s;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    return dot(r, load_act(x, u), u);
  }
};

// ------------------------------------------------------------------ IQ2_XXS (vecdotq.cuh:1531-1552)
// LDS tables: the 256-entry grid expanded to 8 magnitudes per entry, and the 128 sign patterns as byte masks.
struct FmtIQ2_XXS {
  static constexpr int QK = 256, BS = 66, AUX = AUX_NONE, TABLE_BYTES = 256 * 8 + 128 * 8;
  struct Regs { uint16_t d; uint2 g; };
  static __device__ __forceinline__ void init_tables(char* tab) {
    uint2* grid = (uint2*)tab;
    uint2* sgn = grid + 256;
    for (int t = threadIdx.x; t < 256; t += blockDim.x) {
      const uint32_t code = k_iq2xxs_grid_codes[t];
      uint32_t w[2] = {0, 0};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t c = (code >> (2 * j)) & 3;
        w[j >> 2] |= (8 + 17 * c + (c >> 1)) << (8 * (j & 3));
      }
      grid[t] = make_uint2(w[0], w[1]);
      if (t < 128) {
        const uint32_t sg = t | ((__builtin_popcount(t) & 1) << 7);
        uint32_t m[2] = {0, 0};
#pragma unroll
        for (int j = 0; j < 8; ++j) m[j >> 2] |= ((sg >> j) & 1 ? 0xFFu : 0u) << (8 * (j & 3));
        sgn[t] = make_uint2(m[0], m[1]);
      }
    }
  }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.d = ld<uint16_t>(b); r.g = ld<uint2>(b + 2 + 8 * ib); return r;
  }
  struct ActRegs { int2 a[4]; float d; const char* tab; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    ActRegs a;
#pragma unroll
    for (int l = 0; l < 4; ++l) a.a[l] = *(const int2*)(x.q + 32 * u + 8 * l);
    a.d = x.d[u]; a.tab = x.tab;
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint2* grid = (const uint2*)x.tab;
    const uint2* sgn = grid + 256;
    const float dl = h2f(r.d) * (0.5f + (float)(r.g.y >> 28)) * 0.25f;
    int s = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint2 mag = grid[(r.g.x >> (8 * l)) & 0xFF];
      const uint2 m = sgn[(r.g.y >> (7 * l)) & 127];
      s = dot4((int)neg_bytes(mag.x, m.x), x.a[l].x, s);
      s = dot4((int)neg_bytes(mag.y, m.y), x.a[l].y, s);
    }
    return dl * x.d * (float)s;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) {
    return dot(r, load_act(x, u), u);
  }
};


// ================================================================== the other thirteen formats
// bits 0..3 of b -> bit 0 of bytes 0..3 (the four partial products never share a bit, so nothing carries)
__device__ __forceinline__ uint32_t spread4(uint32_t b) { return ((b & 0xFu) * 0x00204081u) & 0x01010101u; }

// LDS table fillers shared by the grid formats
__device__ __forceinline__ void fill_sign_masks(uint2* sgn, int count) {  // 128: 7 bits + parity bit; 256: plain byte
  for (int t = threadIdx.x; t < count; t += blockDim.x) {
    const uint32_t sg = count == 128 ? (uint32_t)t | ((__builtin_popcount(t) & 1) << 7) : (uint32_t)t;
    uint32_t m[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j) m[j >> 2] |= ((sg >> j) & 1 ? 0xFFu : 0u) << (8 * (j & 3));
    sgn[t] = make_uint2(m[0], m[1]);
  }
}
__device__ __forceinline__ void fill_grid2(uint2* grid, const uint16_t* codes, int count) {  // 8 magnitudes {8,25,43}
  for (int t = threadIdx.x; t < count; t += blockDim.x) {
    const uint32_t code = codes[t];
    uint32_t w[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t c = (code >> (2 * j)) & 3;
      w[j >> 2] |= (8 + 17 * c + (c >> 1)) << (8 * (j & 3));
    }
    grid[t] = make_uint2(w[0], w[1]);
  }
}
__device__ __forceinline__ void fill_grid3(uint32_t* grid, const uint16_t* codes, int count, bool xxs) {  // 4 magnitudes
  for (int t = threadIdx.x; t < count; t += blockDim.x) {
    const uint32_t code = codes[t];
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t c = (code >> (3 * j)) & 7;
      w |= (4 + 8 * c + (xxs ? 2 * ((c + 1) >> 3) : 0)) << (8 * j);
    }
    grid[t] = w;
  }
}
__device__ __forceinline__ void fill_grid1(uint32_t* grid) {  // eight values {0,1,2}, value j in nibble j
  for (int t = threadIdx.x; t < 2048; t += blockDim.x) {
    const uint32_t code = k_iq1s_grid_gpu_codes[t];
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) w |= ((code >> (2 * j)) & 3) << (4 * j);
    grid[t] = w;
  }
}

// activations of a unit that is one whole q8_1 block: 32 quants, the block scale and one extra per-block value
struct ActBlock32 { int2 a[4]; float d, s; const char* tab; };
__device__ __forceinline__ ActBlock32 load_act_block32(const Act& x, int u, bool with_aux) {
  ActBlock32 a;
#pragma unroll
  for (int l = 0; l < 4; ++l) a.a[l] = *(const int2*)(x.q + 32 * u + 8 * l);
  a.d = x.d[u];
  a.s = with_aux ? x.a[u] : 0.0f;
  a.tab = x.tab;
  return a;
}

// ------------------------------------------------------------------ Q4_1 (vecdotq.cuh:71-93,573-589)
struct FmtQ4_1 {
  static constexpr int QK = 32, BS = 20, AUX = AUX_S8, TABLE_BYTES = 0;
  struct Regs { uint32_t dm; uint4 q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const uint8_t* b = row + (int64_t)(u0 + u) * BS;
    Regs r; r.dm = ld<uint32_t>(b); r.q = ld<uint4>(b + 4); return r;
  }
  static constexpr int SPAN = 64 * BS;
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    const uint32_t* w = (const uint32_t*)(span + lane * BS);
    Regs r; r.dm = w[0]; r.q = make_uint4(w[1], w[2], w[3], w[4]); return r;
  }
  typedef FmtQ4_0::ActRegs ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return FmtQ4_0::load_act(x, u); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = dot4((int)(q[i] & 0x0F0F0F0Fu), al[i], s);
      s = dot4((int)((q[i] >> 4) & 0x0F0F0F0Fu), ah[i], s);
    }
    // both scale products are rounded to half, as __hmul2(dm4, ds8) does; x.d and x.a hold fp16 values exactly
    const _Float16 d4d8 = __builtin_bit_cast(_Float16, (uint16_t)(r.dm & 0xFFFF)) * (_Float16)x.d;
    const _Float16 m4s8 = __builtin_bit_cast(_Float16, (uint16_t)(r.dm >> 16)) * (_Float16)x.a;
    return (float)s * (float)d4d8 + (float)m4s8;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ Q5_0 / Q5_1 (vecdotq.cuh:98-160,648-769)
template <bool HAS_M>
struct FmtQ5 {
  static constexpr int QK = 32, BS = HAS_M ? 24 : 22, AUX = AUX_S8, TABLE_BYTES = 0;
  struct Regs { uint32_t dm, qh; uint4 q; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const uint8_t* b = row + (int64_t)(u0 + u) * BS;
    Regs r;
    if (HAS_M) { r.dm = ld<uint32_t>(b); r.qh = ld<uint32_t>(b + 4); r.q = ld<uint4>(b + 8); }
    else {
      uint32_t w[6];
      const uint32_t sh = ld_block_dwords(b, w);
      r = cut(w, sh);
    }
    return r;
  }
  static __device__ __forceinline__ Regs cut(const uint32_t (&w)[6], uint32_t sh) {
    const uint32_t shq = sh + 16;
    Regs r;
    r.dm = (w[0] >> sh) & 0xFFFFu;
    r.qh = funnel(w[0], w[1], shq);
    r.q = make_uint4(funnel(w[1], w[2], shq), funnel(w[2], w[3], shq), funnel(w[3], w[4], shq), funnel(w[4], w[5], shq));
    return r;
  }
  static constexpr int SPAN = 64 * BS, SPAN_SLACK = 16;
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    Regs r;
    if (HAS_M) {
      const uint32_t* w = (const uint32_t*)(span + lane * BS);
      r.dm = w[0]; r.qh = w[1]; r.q = make_uint4(w[2], w[3], w[4], w[5]);
    } else {
      uint32_t w[6];
      const uint32_t sh = lds_block_dwords(span, lane * BS, w);
      r = cut(w, sh);
    }
    return r;
  }
  typedef FmtQ4_0::ActRegs ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return FmtQ4_0::load_act(x, u); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {  // bit j of qh is the fifth bit of element j
      s = dot4((int)((q[i] & 0x0F0F0F0Fu) | (spread4(r.qh >> (4 * i)) << 4)), al[i], s);
      s = dot4((int)(((q[i] >> 4) & 0x0F0F0F0Fu) | (spread4(r.qh >> (16 + 4 * i)) << 4)), ah[i], s);
    }
    if (HAS_M) {
      const _Float16 d5d8 = __builtin_bit_cast(_Float16, (uint16_t)(r.dm & 0xFFFF)) * (_Float16)x.d;
      const _Float16 m5s8 = __builtin_bit_cast(_Float16, (uint16_t)(r.dm >> 16)) * (_Float16)x.a;
      return (float)s * (float)d5d8 + (float)m5s8;
    }
    return h2f(r.dm) * ((float)s * x.d - 16.0f * x.a);
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};
typedef FmtQ5<false> FmtQ5_0;
typedef FmtQ5<true> FmtQ5_1;

// ------------------------------------------------------------------ IQ4_NL (vecdotq.cuh:1766-1788)
struct FmtIQ4_NL {
  static constexpr int QK = 32, BS = 18, AUX = AUX_NONE, TABLE_BYTES = 0;
  typedef FmtQ4_0::Regs Regs;
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char* t) { return FmtQ4_0::load(row, u0, u, t); }
  static constexpr int SPAN = FmtQ4_0::SPAN, SPAN_SLACK = FmtQ4_0::SPAN_SLACK;
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) { return FmtQ4_0::from_span(span, lane); }
  typedef FmtIQ4_XS::ActRegs ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return FmtIQ4_XS::load_act(x, u); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    constexpr uint32_t T0 = 0xBFAD9881u, T1 = 0xF6EADDCFu, T2 = 0x26190D01u, T3 = 0x71594535u;
    const uint32_t qq[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s = dot4(lut16<0>(qq[i], T0, T1, T2, T3), al[i], s);
      s = dot4(lut16<4>(qq[i], T0, T1, T2, T3), ah[i], s);
    }
    return h2f(r.d) * x.d * (float)s;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ Q2_K (vecdotq.cuh:204-263,923-944)
// unit c of a super-block: half n = c>>2, columns l in [8*(c&3), +8): the eight bytes qs[32n + l] hold elements
// 128n + 32t + l for t = 0..3, i.e. eight values in each of four q8_1 blocks (the Q6_K arrangement).
struct FmtQ2_K {
  static constexpr int QK = 256, BS = 84, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { uint2 q, sc; uint32_t dm; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7, n = c >> 2, cc = c & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.q = ld<uint2>(b + 16 + 32 * n + 8 * cc); r.sc = ld<uint2>(b + 8 * n); r.dm = ld<uint32_t>(b + 80); return r;
  }
  static constexpr int SPAN = 8 * BS;   // 8 blocks, 672 bytes, every field of the LDS copy at a dword boundary
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    const int c = lane & 7, n = c >> 2, cc = c & 3;
    const uint32_t* w = (const uint32_t*)(span + (lane >> 3) * BS);
    Regs r;
    r.q = make_uint2(w[4 + 8 * n + 2 * cc], w[5 + 8 * n + 2 * cc]); r.sc = make_uint2(w[2 * n], w[2 * n + 1]); r.dm = w[20];
    return r;
  }
  // `du8`: d8 times the sum of the lane's eight quants of block t, what the group's min multiplies
  struct ActRegs { int2 a[4]; float d8[4]; float du8[4]; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    const FmtQ6_K::ActRegs b = FmtQ6_K::load_act_off<1>(x, u);
    ActRegs a;
#pragma unroll
    for (int t = 0; t < 4; ++t) { a.a[t] = b.a[t]; a.d8[t] = b.d8[t]; a.du8[t] = b.d8[t] * (float)b.off[t]; }
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    // scale (low nibble) and min (high nibble) of the lane's four 16-value groups, gathered into one register
    const uint32_t scm = __builtin_amdgcn_perm(r.sc.y, r.sc.x, k8_group_bytes(u));
    const uint32_t sc4 = scm & 0x0F0F0F0Fu, mn4 = (scm >> 4) & 0x0F0F0F0Fu;
    float pos = 0.0f, neg = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int vx = (int)((r.q.x >> (2 * t)) & 0x03030303u), vy = (int)((r.q.y >> (2 * t)) & 0x03030303u);
      const int s = dot4(vx, x.a[t].x, dot4(vy, x.a[t].y, 0));
      // (the integer products s * scale and min * sum are exact as products of the converted factors)
      pos += x.d8[t] * ((float)s * (float)((sc4 >> (8 * t)) & 0xFF));
      neg += x.du8[t] * (float)((mn4 >> (8 * t)) & 0xFF);
    }
    return h2f(r.dm & 0xFFFF) * pos - h2f(r.dm >> 16) * neg;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ Q3_K (vecdotq.cuh:269-322,1024-1049)
// same unit arrangement as Q2_K; the high bit of element (n, t, l) is bit 4n + t of hmask[l], and a clear bit means -4
struct FmtQ3_K {
  static constexpr int QK = 256, BS = 110, AUX = AUX_NONE, TABLE_BYTES = 0;
  struct Regs { uint2 q, hm, sc01; uint32_t sc2; uint16_t d; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7, n = c >> 2, cc = c & 3;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r;
    r.q = ld<uint2>(b + 32 + 32 * n + 8 * cc); r.hm = ld<uint2>(b + 8 * cc);
    r.sc01 = ld<uint2>(b + 96); r.sc2 = ld<uint32_t>(b + 104); r.d = ld<uint16_t>(b + 108);
    return r;
  }
  static constexpr int SPAN = 8 * BS, SPAN_SLACK = 16;   // 8 blocks, 880 bytes, at 2-byte alignment in the LDS copy
  static constexpr bool SPAN_ANY = true;
  static __device__ __forceinline__ Regs from_span(const char* span, int lane, int at = 0) {
    const int c = lane & 7, n = c >> 2, cc = c & 3, b = at + (lane >> 3) * BS;
    Regs r;
    r.q = lds_cut8(span, b + 32 + 32 * n + 8 * cc); r.hm = lds_cut8(span, b + 8 * cc);
    uint32_t w[5];    // bytes 96 .. 109: twelve of scales and d
    const uint32_t sh = lds_block_dwords(span, b + 96, w);
    r.sc01 = make_uint2(funnel(w[0], w[1], sh), funnel(w[1], w[2], sh)); r.sc2 = funnel(w[2], w[3], sh);
    r.d = (uint16_t)(funnel(w[3], w[4], sh));
    return r;
  }
  typedef FmtQ6_K::ActRegs ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return FmtQ6_K::load_act_off<4>(x, u); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const int n4 = (u & 4);   // 4 n: the super-block's second half takes the high nibbles and the upper bit pairs
    // The 6-bit scale of group is = 8 n + g, g = 2 t + h: low nibble from nibble n of byte g of the first eight scale
    // bytes, two high bits from bits 4 n + 2 (t / 2) of byte g mod 4 of the last four.  Byte permutes gather the four
    // bytes of either kind, so that the four scales are formed together in one register.
    const uint32_t h = (u >> 1) & 1;
    const uint32_t lo4 = (__builtin_amdgcn_perm(r.sc01.y, r.sc01.x, k8_group_bytes(u)) >> n4) & 0x0F0F0F0Fu;
    const uint32_t p2 = __builtin_amdgcn_perm(r.sc2, r.sc2, h ? 0x03010301u : 0x02000200u) >> n4;
    const uint32_t us4 = lo4 | (((p2 & 0x00000303u) | ((p2 >> 2) & 0x03030000u)) << 4);
    const uint32_t hmx = r.hm.x >> n4, hmy = r.hm.y >> n4;
    float acc = 0.0f;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const uint32_t hx = (hmx >> t) & 0x01010101u, hy = (hmy >> t) & 0x01010101u;
      const int vx = (int)(((r.q.x >> (2 * t)) & 0x03030303u) | (hx << 2)), vy = (int)(((r.q.y >> (2 * t)) & 0x03030303u) | (hy << 2));
      const int s = dot4(vx, x.a[t].x, dot4(vy, x.a[t].y, 0)) - x.off[t];
      // ((scale - 32) * s is exact as a product of the converted factors: |.| < 2^19)
      acc += x.d8[t] * (((float)((us4 >> (8 * t)) & 0xFF) - 32.0f) * (float)s);
    }
    return h2f(r.d) * acc;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ Q5_K (vecdotq.cuh:384-441,1279-1323)
// the Q4_K unit with a fifth bit: bit 2g of qh[l] for the low-nibble sub-block, bit 2g+1 for the high-nibble one
struct FmtQ5_K {
  static constexpr int QK = 256, BS = 176, AUX = AUX_DU, TABLE_BYTES = 0;
  struct Regs { uint4 hdr, q, qh; };
  static __device__ __forceinline__ void init_tables(char*) {}
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, c = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.hdr = ld<uint4>(b); r.q = ld<uint4>(b + 48 + 16 * c); r.qh = ld<uint4>(b + 16 + 16 * (c & 1)); return r;
  }
  static constexpr int SPAN = 8 * BS;   // 8 blocks, 1408 bytes
  static __device__ __forceinline__ Regs from_span(const char* span, int lane) {
    const char* b = span + (lane >> 3) * BS;
    const int c = lane & 7;
    Regs r; r.hdr = *(const uint4*)b; r.q = *(const uint4*)(b + 48 + 16 * c); r.qh = *(const uint4*)(b + 16 + 16 * (c & 1)); return r;
  }
  typedef FmtQ4_K::ActRegs ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return FmtQ4_K::load_act(x, u); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const int g = (u & 7) >> 1;
    const int sh = 16 * (g & 1);
    const uint32_t A = (r.hdr.y >> sh) & 0xFFFF, B = (r.hdr.z >> sh) & 0xFFFF, C = (r.hdr.w >> sh) & 0xFFFF;
    uint32_t a0, a1;
    if (g < 2) {
      a0 = A & 0x3F3F; a1 = B & 0x3F3F;
    } else {
      a0 = (C & 0x0F0F) | ((A & 0xC0C0) >> 2);
      a1 = ((C >> 4) & 0x0F0F) | ((B & 0xC0C0) >> 2);
    }
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w}, h[4] = {r.qh.x, r.qh.y, r.qh.z, r.qh.w};
    const int al[4] = {x.lo.x, x.lo.y, x.lo.z, x.lo.w}, ah[4] = {x.hi.x, x.hi.y, x.hi.z, x.hi.w};
    int s0 = 0, s1 = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      s0 = dot4((int)((q[i] & 0x0F0F0F0Fu) | (((h[i] >> (2 * g)) & 0x01010101u) << 4)), al[i], s0);
      s1 = dot4((int)(((q[i] >> 4) & 0x0F0F0F0Fu) | (((h[i] >> (2 * g + 1)) & 0x01010101u) << 4)), ah[i], s1);
    }
    const float pos = x.d8.x * (float)(s0 * (int)(a0 & 0xFF)) + x.d8.y * (float)(s1 * (int)(a0 >> 8));
    const float neg = x.du.x * (float)(a1 & 0xFF) + x.du.y * (float)(a1 >> 8);
    return h2f(r.hdr.x & 0xFFFF) * pos - h2f(r.hdr.x >> 16) * neg;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ IQ2_XS (vecdotq.cuh:1554-1583)
struct FmtIQ2_XS {
  static constexpr int QK = 256, BS = 74, AUX = AUX_NONE, TABLE_BYTES = 512 * 8 + 128 * 8;
  struct Regs { uint2 q; uint16_t d; uint8_t sc; };
  static __device__ __forceinline__ void init_tables(char* tab) {
    fill_grid2((uint2*)tab, k_iq2xs_grid_codes, 512);
    fill_sign_masks((uint2*)tab + 512, 128);
  }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.d = ld<uint16_t>(b); r.q = ld<uint2>(b + 2 + 8 * ib); r.sc = b[66 + ib]; return r;
  }
  typedef ActBlock32 ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return load_act_block32(x, u, false); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint2* grid = (const uint2*)x.tab;
    const uint2* sgn = grid + 512;
    int sumi[2] = {0, 0};
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t q2 = ((l < 2 ? r.q.x : r.q.y) >> (16 * (l & 1))) & 0xFFFF;
      const uint2 mag = grid[q2 & 511], m = sgn[q2 >> 9];
      sumi[l >> 1] = dot4((int)neg_bytes(mag.x, m.x), x.a[l].x, dot4((int)neg_bytes(mag.y, m.y), x.a[l].y, sumi[l >> 1]));
    }
    const float d = h2f(r.d) * x.d * 0.25f;
    return d * ((0.5f + (float)(r.sc & 0xF)) * (float)sumi[0] + (0.5f + (float)(r.sc >> 4)) * (float)sumi[1]);
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ IQ2_S (vecdotq.cuh:1585-1620)
struct FmtIQ2_S {
  static constexpr int QK = 256, BS = 82, AUX = AUX_NONE, TABLE_BYTES = 1024 * 8 + 256 * 8;
  struct Regs { uint32_t q, sg; uint16_t d; uint8_t qh, sc; };
  static __device__ __forceinline__ void init_tables(char* tab) {
    fill_grid2((uint2*)tab, k_iq2s_grid_codes, 1024);
    fill_sign_masks((uint2*)tab + 1024, 256);
  }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r;
    r.d = ld<uint16_t>(b); r.q = ld<uint32_t>(b + 2 + 4 * ib); r.sg = ld<uint32_t>(b + 34 + 4 * ib); r.qh = b[66 + ib]; r.sc = b[74 + ib];
    return r;
  }
  typedef ActBlock32 ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return load_act_block32(x, u, false); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint2* grid = (const uint2*)x.tab;
    const uint2* sgn = grid + 1024;
    int sumi[2] = {0, 0};
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t idx = ((r.q >> (8 * l)) & 0xFF) | (((uint32_t)r.qh << (8 - 2 * l)) & 0x300);
      const uint2 mag = grid[idx], m = sgn[(r.sg >> (8 * l)) & 0xFF];
      sumi[l >> 1] = dot4((int)neg_bytes(mag.x, m.x), x.a[l].x, dot4((int)neg_bytes(mag.y, m.y), x.a[l].y, sumi[l >> 1]));
    }
    const float d = h2f(r.d) * x.d * 0.25f;
    return d * ((0.5f + (float)(r.sc & 0xF)) * (float)sumi[0] + (0.5f + (float)(r.sc >> 4)) * (float)sumi[1]);
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ IQ3_XXS (vecdotq.cuh:1622-1647)
struct FmtIQ3_XXS {
  static constexpr int QK = 256, BS = 98, AUX = AUX_NONE, TABLE_BYTES = 256 * 4 + 128 * 8;
  struct Regs { uint2 q; uint32_t aux; uint16_t d; };
  static __device__ __forceinline__ void init_tables(char* tab) {
    fill_grid3((uint32_t*)tab, k_iq3xxs_grid_codes, 256, true);
    fill_sign_masks((uint2*)(tab + 256 * 4), 128);
  }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.d = ld<uint16_t>(b); r.q = ld<uint2>(b + 2 + 8 * ib); r.aux = ld<uint32_t>(b + 66 + 4 * ib); return r;
  }
  typedef ActBlock32 ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return load_act_block32(x, u, false); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint32_t* grid = (const uint32_t*)x.tab;
    const uint2* sgn = (const uint2*)(x.tab + 256 * 4);
    int s = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t qw = (l < 2 ? r.q.x : r.q.y) >> (16 * (l & 1));
      const uint2 m = sgn[(r.aux >> (7 * l)) & 127];
      s = dot4((int)neg_bytes(grid[qw & 0xFF], m.x), x.a[l].x, dot4((int)neg_bytes(grid[(qw >> 8) & 0xFF], m.y), x.a[l].y, s));
    }
    return h2f(r.d) * (0.5f + (float)(r.aux >> 28)) * x.d * 0.5f * (float)s;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ IQ3_S (vecdotq.cuh:1649-1672)
struct FmtIQ3_S {
  static constexpr int QK = 256, BS = 110, AUX = AUX_NONE, TABLE_BYTES = 512 * 4 + 256 * 8;
  struct Regs { uint2 q; uint32_t sg; uint16_t d; uint8_t qh, sc; };
  static __device__ __forceinline__ void init_tables(char* tab) {
    fill_grid3((uint32_t*)tab, k_iq3xs_grid_codes, 512, false);
    fill_sign_masks((uint2*)(tab + 512 * 4), 256);
  }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r;
    r.d = ld<uint16_t>(b); r.q = ld<uint2>(b + 2 + 8 * ib); r.qh = b[66 + ib]; r.sg = ld<uint32_t>(b + 74 + 4 * ib); r.sc = b[106 + (ib >> 1)];
    return r;
  }
  typedef ActBlock32 ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return load_act_block32(x, u, false); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const int ib = u & 7;
    const uint32_t* grid = (const uint32_t*)x.tab;
    const uint2* sgn = (const uint2*)(x.tab + 512 * 4);
    int s = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t qw = (l < 2 ? r.q.x : r.q.y) >> (16 * (l & 1));
      const uint32_t i1 = (qw & 0xFF) | (((uint32_t)r.qh << (8 - 2 * l)) & 256), i2 = ((qw >> 8) & 0xFF) | (((uint32_t)r.qh << (7 - 2 * l)) & 256);
      const uint2 m = sgn[(r.sg >> (8 * l)) & 0xFF];
      s = dot4((int)neg_bytes(grid[i1], m.x), x.a[l].x, dot4((int)neg_bytes(grid[i2], m.y), x.a[l].y, s));
    }
    return h2f(r.d) * (0.5f + (float)((r.sc >> (4 * (ib & 1))) & 0xF)) * x.d * 0.5f * (float)s;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ IQ1_S (vecdotq.cuh:1674-1704)
// the delta term uses the activation block's stored sum, the grid term its quants
struct FmtIQ1_S {
  static constexpr int QK = 256, BS = 50, AUX = AUX_S8, TABLE_BYTES = 2048 * 4;
  struct Regs { uint32_t q; uint16_t d, qh; };
  static __device__ __forceinline__ void init_tables(char* tab) { fill_grid1((uint32_t*)tab); }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.d = ld<uint16_t>(b); r.q = ld<uint32_t>(b + 2 + 4 * ib); r.qh = ld<uint16_t>(b + 34 + 2 * ib); return r;
  }
  typedef ActBlock32 ActRegs;
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) { return load_act_block32(x, u, true); }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const uint32_t* grid = (const uint32_t*)x.tab;
    const uint32_t qh = r.qh;
    int s = 0;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t g = grid[((r.q >> (8 * l)) & 0xFF) | (((qh >> (3 * l)) & 7) << 8)];
      s = dot4((int)(g & 0x0F0F0F0Fu), x.a[l].x, dot4((int)((g >> 4) & 0x0F0F0F0Fu), x.a[l].y, s));
    }
    const float d1q = h2f(r.d) * (float)(2 * ((qh >> 12) & 7) + 1);
    const float delta = qh & 0x8000 ? -1.0f - 0.125f : -1.0f + 0.125f;
    return d1q * (x.d * (float)s + x.s * delta);
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

// ------------------------------------------------------------------ IQ1_M (vecdotq.cuh:1706-1750)
// delta applies per eight elements to the sum of their activation quants; two 3-bit scales per 32-element unit
struct FmtIQ1_M {
  static constexpr int QK = 256, BS = 56, AUX = AUX_NONE, TABLE_BYTES = 2048 * 4;
  struct Regs { uint32_t q; uint2 sc; uint16_t qh; };
  static __device__ __forceinline__ void init_tables(char* tab) { fill_grid1((uint32_t*)tab); }
  static __device__ __forceinline__ Regs load(const uint8_t* row, int u0, int u, const char*) {
    const int uu = u0 + u, sb = uu >> 3, ib = uu & 7;
    const uint8_t* b = row + (int64_t)sb * BS;
    Regs r; r.q = ld<uint32_t>(b + 4 * ib); r.qh = ld<uint16_t>(b + 32 + 2 * ib); r.sc = ld<uint2>(b + 48); return r;
  }
  struct ActRegs { int2 a[4]; int ones[4]; float d; const char* tab; };
  static __device__ __forceinline__ ActRegs load_act(const Act& x, int u) {
    ActRegs a;
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      a.a[l] = *(const int2*)(x.q + 32 * u + 8 * l);
      a.ones[l] = dot4(0x01010101, a.a[l].x, dot4(0x01010101, a.a[l].y, 0));
    }
    a.d = x.d[u]; a.tab = x.tab;
    return a;
  }
  static __device__ __forceinline__ float dot(const Regs& r, const ActRegs& x, int u) {
    const int ib = u & 7;
    const uint32_t* grid = (const uint32_t*)x.tab;
    int sumi[2] = {0, 0};
    float sumf[2] = {0.0f, 0.0f};
#pragma unroll
    for (int l = 0; l < 4; ++l) {
      const uint32_t qhl = ((uint32_t)r.qh >> (4 * l)) & 0xF;
      const uint32_t g = grid[((r.q >> (8 * l)) & 0xFF) | ((qhl & 7) << 8)];
      sumi[l >> 1] = dot4((int)(g & 0x0F0F0F0Fu), x.a[l].x, dot4((int)((g >> 4) & 0x0F0F0F0Fu), x.a[l].y, sumi[l >> 1]));
      sumf[l >> 1] += (qhl & 8 ? -1.0f - 0.125f : -1.0f + 0.125f) * (float)x.ones[l];
    }
    const uint32_t w0 = r.sc.x & 0xFFFF, w1 = r.sc.x >> 16, w2 = r.sc.y & 0xFFFF, w3 = r.sc.y >> 16;
    const uint32_t sbits = (w0 >> 12) | ((w1 >> 8) & 0x00F0) | ((w2 >> 4) & 0x0F00) | (w3 & 0xF000);
    const uint32_t wsel = (ib >> 1) == 0 ? w0 : (ib >> 1) == 1 ? w1 : (ib >> 1) == 2 ? w2 : w3;
    const uint32_t tmp = wsel >> (6 * (ib & 1));
    const float sc0 = (float)(2 * (tmp & 7) + 1), sc1 = (float)(2 * ((tmp >> 3) & 7) + 1);
    return h2f(sbits) * x.d * (((float)sumi[0] + sumf[0]) * sc0 + ((float)sumi[1] + sumf[1]) * sc1);
  }
  static __device__ __forceinline__ float dot(const Regs& r, const Act& x, int u, int lane) { return dot(r, load_act(x, u), u); }
};

}  // namespace gguf
