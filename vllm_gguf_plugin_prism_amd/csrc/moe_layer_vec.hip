// A whole MoE layer for a few tokens in two launches (reference, as five steps: ggml_moe_a8_vec, act(), ggml_moe_a8_vec,
// out.mul_(topk_weights), ops.moe_sum -- quantization/fused_moe.py:98-111, csrc/gguf/moe_vec.cuh:3-53).
//
// With fewer than about two pairs per expert nothing is shared between pairs, and what the separate steps cost beyond
// the two weight streams is their seams: the second GEMV's workgroups each apply the activation to their pair's row
// and quantize it (once per row band, 32 times per row for a 2048-feature layer), and the sum over the top-k axis
// crosses workgroups, so it is a kernel of its own (3-4 us of a 15 us layer at one token).
//   1. moe_up_act_kernel: the per-pair GEMV of the first expert matrix, whose workgroups own the same R features in
//      the gate half and in the up half of [gate | up].  The workgroup that has both finishes them: y = T(sum),
//      h = T(T(act(gate)) up), and the q8_1 blocks of h go to the workspace -- the values the second GEMV would have
//      quantized, produced once, and no [pairs][2 I] tensor in between.
//   2. moe_down_sum_kernel: a workgroup owns a band of output features of ONE token and walks it in the matrices of all
//      its top_k experts: (half-)wave -> (pair, row slot), the pair's quantized activations read from the workspace
//      into registers (no staging, no barrier before the first row).  The partial sums of every (pair, row) meet in
//      LDS, where the adder forms y = T(sum), T(y w_k) and their fp32 sum in the order k = 0 .. top_k-1: the roundings
//      of the separate steps.
// Results are those of gguf_moe_vec, gguf_moe_vec_act and gguf_moe_weighted_sum in sequence up to the last bit of a dot
// product (the compiler contracts multiply-adds per kernel): the same per-lane arithmetic, the same order of the partial
// sums (ascending in K), the same quantizer and activation routines, every intermediate rounded where those steps store it.
//
// Where experts are shared by a few pairs each (the per-pair operator's tile route on blocks of 16 slots) the same entry
// point runs the layer in four launches on the tile kernels instead (mmq.hip, moe_tiles_layer).
#include "mmvq_core.h"

namespace gguf {

// mmq.hip
int moe_tiles_layer_block(int type13, int type2, int64_t pairs, int64_t num_experts, int64_t I, bool vec_sums);
int64_t moe_tiles_layer_workspace(int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out, int64_t num_experts, int elt, int block);
int moe_tiles_layer(const void* X, int xdtype, void* workspace, const void* W13, int type13, const void* W2, int type2, const int32_t* topk_ids,
                    const float* topk_w, void* out, int H, int I, int N_out, int top_k, int tokens, int act, int num_experts, bool vec_sums,
                    int block, hipStream_t s);
int64_t moe_sorted_layer_workspace(int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out, int64_t num_experts, int elt, int block);
int moe_sorted_layer(const void* X, int xdtype, void* workspace, const void* W13, int type13, const void* W2, int type2, const int32_t* topk_ids,
                     const float* topk_w, void* out, int H, int I, int N_out, int top_k, int tokens, int act, int num_experts, int block,
                     hipStream_t s);

struct MoeUpArgs {
  const int32_t* topk_ids;
  int64_t expert_bytes;    // between the matrices of two experts
  char* ws;                // q8_1 rows of h, one per pair
  int64_t ws_row_bytes;
  int top_k, num_experts, act;
  int I, R, kp_i;          // inner features; features per band (a multiple of 32); q8_kp(I)
};

template <class F, int NW, typename T, bool HALF>
__global__ __launch_bounds__(64 * NW) void moe_up_act_kernel(const uint8_t* __restrict__ W, const T* __restrict__ X, MoeUpArgs moe, StreamGeom geom) {
  extern __shared__ __align__(16) char smem[];
  constexpr int NT = 64 * NW, D = 2;
  const int z = blockIdx.y;
  const int e = moe.topk_ids[z];
  if (moe.num_experts > 0 && (e < 0 || e >= moe.num_experts)) return;   // names no weights: its row is never read
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = geom.K, nb = K >> 5, g8 = K >> 3, S = geom.S(), slots = geom.slots();
  const int I = moe.I, R = moe.R, vrows = 2 * R;      // virtual rows of the band: R of the gate half, then R of the up half
  X += (int64_t)(z / moe.top_k) * K;
  W += (int64_t)e * moe.expert_bytes;
  int8_t* lq = (int8_t*)smem;                          // [K]
  float* ldv = (float*)(smem + (size_t)K);             // [nb]
  float* lav = ldv + nb;                               // [nb]
  char* tab = (char*)(lav + (F::AUX != AUX_NONE ? nb : 0));
  float* part = (float*)(tab + F::TABLE_BYTES);        // [2 R][G]
  constexpr int GW = HALF ? 2 : 4;
  const int G = GW * S;
  float* hb = part + (size_t)vrows * G;                // [R]

  const int g0 = blockIdx.x * R, ng = min(R, I - g0);  // this band's features (ng > 0 and a multiple of 32: host)
  const int wh = HALF ? 2 * wave + (lane >> 5) : wave;
  const int slot = geom.slot_of(wh), step = wh - slot * S;
  const bool on = slot < slots;
  const int u_raw = HALF ? step * 32 + (lane & 31) : step * 64 + lane;
  const int u = min(u_raw, nb - 1);
  const bool lane_on = on && u_raw < nb;

  if (F::TABLE_BYTES > 0) {
    F::init_tables(tab);
    __syncthreads();
  }
  // virtual row -> row of [gate | up] (rows past the band's features are clamped, computed and not used)
  const auto load_row = [&](int i) {
    const int v = min((on ? slot : 0) + slots * i, vrows - 1);
    const int row = v < R ? g0 + min(v, ng - 1) : I + g0 + min(v - R, ng - 1);
    return F::load(W + (int64_t)row * geom.w_pitch, 0, u, tab);
  };
  // ---- the token's row -> q8_1 in LDS (four lanes per 32-value block), its first requests ahead of the weights'
  const auto quantize_group = [&](const raw8<T>& raw, int q) {
    float xv[8];
    raw.cvt(xv);
    const Q8Quad qq = q8_1_quantize8(xv);
    if (q < g8) {
      *(uint2*)(lq + 8 * q) = qq.q;
      if ((q & 3) == 0) {
        ldv[q >> 2] = qq.d;
        if (F::AUX == AUX_S8) lav[q >> 2] = qq.s;
        if (F::AUX == AUX_DU) lav[q >> 2] = qq.du;
      }
    }
  };
  raw8<T> x0;
  x0.load(X + 8 * min(tid, g8 - 1));
  __builtin_amdgcn_sched_barrier(0);
  typename F::Regs pre[D];
#pragma unroll
  for (int d = 0; d < D; ++d) pre[d] = load_row(d);
  __builtin_amdgcn_sched_barrier(0);
  if (wave * 64 < g8) quantize_group(x0, tid);         // (wave-uniform: whole quads take part)
  for (int q = tid + NT; q - tid < g8; q += NT) {      // uniform trip count; only for K > 8 NT
    raw8<T> r;
    r.load(X + 8 * min(q, g8 - 1));
    quantize_group(r, q);
  }
  __syncthreads();

  Act x;
  x.q = lq;
  x.d = ldv;
  x.a = lav;
  x.tab = tab;
  const typename F::ActRegs act = F::load_act(x, u);
  const int my_rows = on && vrows > slot ? (vrows - slot + slots - 1) / slots : 0;
  const int max_rows = (vrows + slots - 1) / slots;    // trip count, the same for every wave
  for (int i0 = 0; i0 < max_rows; i0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int i = i0 + d;
      const typename F::Regs cur = pre[d];
      const float v = F::dot(cur, act, u);
      pre[d] = load_row(i + D);
      const float acc[1] = {lane_on ? v : 0.0f};
      const float sum = rows16_sums<1>(acc, lane);
      if ((lane & 15) == 0 && i < my_rows) part[(size_t)(slot + slots * i) * G + step * GW + ((lane >> 4) & (GW - 1))] = sum;
    }
  }
  __syncthreads();
  // ---- feature t of the band: both halves' sums rounded as the GEMV stores them, then the gated activation
  for (int t = tid; t < R; t += NT) {
    float g = 0.0f, up = 0.0f;
    for (int st = 0; st < G; ++st) g += part[(size_t)t * G + st];
    for (int st = 0; st < G; ++st) up += part[(size_t)(R + t) * G + st];
    hb[t] = gate1<T>(to_f32<T>(from_f32<T>(g)), to_f32<T>(from_f32<T>(up)), moe.act);
  }
  __syncthreads();
  // ---- and its q8_1 blocks into the pair's workspace row (R / 8 threads: whole quads, ng is a multiple of 32)
  if (tid < R / 8) {
    float xv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) xv[i] = hb[8 * tid + i];
    const Q8Quad qq = q8_1_quantize8(xv);
    if (8 * tid < ng) {
      char* row = moe.ws + (int64_t)z * moe.ws_row_bytes;
      *(uint2*)(row + g0 + 8 * tid) = qq.q;
      if ((tid & 3) == 0) {
        float* fd = (float*)(row + moe.kp_i);
        const int b = (g0 >> 5) + (tid >> 2), nbp = moe.kp_i >> 5;
        fd[b] = qq.d;
        fd[nbp + b] = qq.s;
        fd[2 * nbp + b] = qq.du;
      }
    }
  }
}

struct MoeSumArgs {
  const int32_t* topk_ids;
  const float* topk_w;
  int64_t expert_bytes;    // between the matrices of two experts
  const char* ws;          // q8_1 rows of the pairs
  int64_t ws_row_bytes;
  int top_k, num_experts, slots, kp;   // slots: rows of the band that one pair's waves walk side by side; kp = q8_kp(K)
  uint32_t tk_inv;         // 65536 / top_k + 1: n / top_k for n < 4096 as (n * tk_inv) >> 16
};

template <class F, int NW, typename T, bool HALF>
__global__ __launch_bounds__(64 * NW) void moe_down_sum_kernel(const uint8_t* __restrict__ W, T* __restrict__ out, MoeSumArgs moe, StreamGeom geom) {
  extern __shared__ __align__(16) char smem[];
  constexpr int NT = 64 * NW, D = 2;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int token = blockIdx.y, top_k = moe.top_k;
  const int N = geom.N, K = geom.K, rows_per_wg = geom.rows_per_wg;
  const int nb = K >> 5, S = geom.S();
  char* tab = smem;
  float* part = (float*)(tab + ((F::TABLE_BYTES + 15) & ~15));   // [top_k][rows_per_wg][G]
  constexpr int GW = HALF ? 2 : 4;
  const int G = GW * S;

  const int r_begin = blockIdx.x * rows_per_wg, nrows = min(N, r_begin + rows_per_wg) - r_begin;   // > 0 (host)
  // this (half-)wave: which pair, which of the pair's side-by-side rows, which stretch of the row
  const int wh = HALF ? 2 * wave + (lane >> 5) : wave;
  const int rs = geom.slot_of(wh), step = wh - rs * S;
  const int slots = moe.slots;
  const bool on = rs < slots * top_k;
  const int slot = on ? (int)(((uint32_t)rs * moe.tk_inv) >> 16) : 0;   // rs / top_k
  const int pair = on ? rs - slot * top_k : 0;                          // rs % top_k
  const int u_raw = HALF ? step * 32 + (lane & 31) : step * 64 + lane;
  const int u = min(u_raw, nb - 1);
  const int z = token * top_k + pair;
  int e = moe.topk_ids[z];
  const bool known = moe.num_experts <= 0 || (e >= 0 && e < moe.num_experts);   // a pair that names no expert adds nothing
  if (!known) e = 0;
  const bool lane_on = on && known && u_raw < nb;

  if (F::TABLE_BYTES > 0) {
    F::init_tables(tab);
    __syncthreads();
  }
  const uint8_t* wbase = W + (int64_t)e * moe.expert_bytes + (int64_t)r_begin * geom.w_pitch;
  const auto load_row = [&](int i) { return F::load(wbase + (int64_t)min(slot + slots * i, nrows - 1) * geom.w_pitch, 0, u, tab); };
  typename F::Regs pre[D];
#pragma unroll
  for (int d = 0; d < D; ++d) pre[d] = load_row(d);
  // the pair's quantized activations, this lane's unit of them, straight from the workspace (a row the first kernel
  // left unwritten -- an unknown expert -- is not read)
  const char* xrow = moe.ws + (int64_t)(known ? z : token * top_k) * moe.ws_row_bytes;
  Act x;
  x.q = (const int8_t*)xrow;
  x.d = (const float*)(xrow + moe.kp);
  x.a = x.d + (F::AUX == AUX_DU ? 2 : 1) * (moe.kp >> 5);
  x.tab = tab;
  const typename F::ActRegs act = F::load_act(x, u);

  const int my_rows = on && nrows > slot ? (nrows - slot + slots - 1) / slots : 0;
  const int max_rows = (nrows + slots - 1) / slots;    // trip count, the same for every wave
  for (int i0 = 0; i0 < max_rows; i0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int i = i0 + d;
      const typename F::Regs cur = pre[d];
      const float v = F::dot(cur, act, u);
      pre[d] = load_row(i + D);
      const float acc[1] = {lane_on ? v : 0.0f};
      const float sum = rows16_sums<1>(acc, lane);
      if ((lane & 15) == 0 && i < my_rows)
        part[((size_t)pair * rows_per_wg + slot + slots * i) * G + step * GW + ((lane >> 4) & (GW - 1))] = sum;
    }
  }
  __syncthreads();
  for (int i = tid; i < nrows; i += NT) {
    float total = 0.0f;
    for (int p = 0; p < top_k; ++p) {
      float y = 0.0f;
      for (int st = 0; st < G; ++st) y += part[((size_t)p * rows_per_wg + i) * G + st];
      const int ep = moe.topk_ids[token * top_k + p];
      if (moe.num_experts > 0 && (ep < 0 || ep >= moe.num_experts)) continue;
      const T scaled = from_f32<T>(to_f32<T>(from_f32<T>(y)) * moe.topk_w[token * top_k + p]);
      total += to_f32<T>(scaled);
    }
    out[(int64_t)token * N + r_begin + i] = from_f32<T>(total);
  }
}

// (half-)waves per row and rows side by side for rows of K values: half-waves where those leave fewer lanes idle
struct RowSplit {
  bool ok, half;
  int S, slots;
};
static RowSplit row_split(int K) {
  constexpr int NW = MMVQ_NW;
  RowSplit r = {};
  const int nb = K / 32;
  if (nb <= 0) return r;
  const int s_full = (nb + 63) / 64, s_half = (nb + 31) / 32;
  r.half = 64 * s_full > 32 * s_half;
  r.S = r.half ? s_half : s_full;
  const int units = r.half ? 2 * NW : NW;
  r.slots = units / r.S;
  r.ok = r.slots >= 1;
  return r;
}

// How the first kernel is laid out: bands of R features (in both halves) such that the workgroups, one per CU at a
// time, make whole rounds; a workgroup's time is its turns of the row loop plus about sixteen turns' worth of start-up.
struct MoeUpPlan {
  bool ok;
  RowSplit rows;
  int R, bands;
  size_t lds;
};
template <class F>
static MoeUpPlan moe_up_plan(int H, int I, int pairs) {
  MoeUpPlan p = {};
  p.rows = row_split(H);
  if (!p.rows.ok || I <= 0 || I % 32 != 0 || pairs <= 0 || pairs > 65535) return p;
  if ((int64_t)(H / F::QK) * F::BS > (int64_t)UINT32_MAX) return p;
  const int64_t cus = num_cus();
  int64_t best = INT64_MAX;
  for (int R = 32; R <= I && R <= 4096; R += 32) {
    const int bands = (I + R - 1) / R;
    const int64_t rounds = ((int64_t)bands * pairs + cus - 1) / cus;
    const int64_t cost = rounds * ((2 * R + p.rows.slots - 1) / p.rows.slots + 16);
    if (cost < best) { best = cost; p.R = R; p.bands = bands; }
  }
  const int G = (p.rows.half ? 2 : 4) * p.rows.S;
  p.lds = (size_t)H + (size_t)(H / 32) * 4 * (F::AUX != AUX_NONE ? 2 : 1) + F::TABLE_BYTES + (size_t)2 * p.R * G * 4 + (size_t)p.R * 4;
  p.ok = p.lds <= 160 * 1024;
  return p;
}

// The second kernel: bands of output features per token, the same cost rule.
struct MoeSumPlan {
  bool ok;
  RowSplit rows;
  int slots, rows_per_wg, grid;
  size_t lds;
};
template <class F>
static MoeSumPlan moe_sum_plan(int N, int K, int top_k, int tokens) {
  MoeSumPlan p = {};
  p.rows = row_split(K);
  if (!p.rows.ok || N <= 0 || top_k <= 0 || tokens <= 0 || tokens > 65535) return p;
  p.slots = p.rows.slots / top_k;
  if (p.slots < 1) return p;
  if ((int64_t)(K / F::QK) * F::BS > (int64_t)UINT32_MAX) return p;
  const int64_t cus = num_cus();
  const int max_bands = (int)std::max<int64_t>(64, (cus + tokens - 1) / tokens);
  int64_t best = INT64_MAX;
  p.rows_per_wg = N;
  for (int b = 1; b <= max_bands; ++b) {
    const int rows = (N + b - 1) / b;
    if (rows < p.slots && b > 1) break;
    const int64_t wgs = (int64_t)((N + rows - 1) / rows) * tokens, rounds = (wgs + cus - 1) / cus;
    const int64_t cost = rounds * ((rows + p.slots - 1) / p.slots + 16);
    if (cost < best) { best = cost; p.rows_per_wg = rows; }
  }
  p.grid = (N + p.rows_per_wg - 1) / p.rows_per_wg;
  p.lds = ((F::TABLE_BYTES + 15) & ~(size_t)15) + (size_t)top_k * p.rows_per_wg * (p.rows.half ? 2 : 4) * p.rows.S * 4;
  p.ok = p.lds <= 160 * 1024;
  return p;
}

template <class F, typename T>
static int moe_up_typed(const void* W, const void* X, const int32_t* ids, void* ws, int H, int I, int top_k, int tokens, int act, int num_experts,
                        hipStream_t stream) {
  constexpr int NW = MMVQ_NW;
  const int pairs = tokens * top_k;
  const MoeUpPlan p = moe_up_plan<F>(H, I, pairs);
  if (!p.ok) return GGUF_ERR_SHAPE;
  const int64_t pitch = (int64_t)(H / F::QK) * F::BS;
  const MoeUpArgs moe = {ids, (int64_t)2 * I * pitch, (char*)ws, q8_row_bytes(I), top_k, num_experts, act, I, p.R, (int)q8_kp(I)};
  const StreamGeom geom = stream_geom(2 * I, H, 2 * p.R, pitch, 1, NW, p.rows.half);
  const auto go = [&](auto kern) {
    if (p.lds > 64 * 1024) {
      static std::atomic<uint64_t> done{0};
      allow_large_lds(kern, 160 * 1024, done);
    }
    hipLaunchKernelGGL(kern, dim3(p.bands, pairs), dim3(64 * NW), p.lds, stream, (const uint8_t*)W, (const T*)X, moe, geom);
  };
  if (p.rows.half) go(moe_up_act_kernel<F, NW, T, true>);
  else go(moe_up_act_kernel<F, NW, T, false>);
  return launch_status();
}

template <class F, typename T>
static int moe_sum_typed(const void* W, const void* ws, const int32_t* ids, const float* wts, void* out, int N, int K, int top_k, int tokens,
                         int num_experts, hipStream_t stream) {
  constexpr int NW = MMVQ_NW;
  const MoeSumPlan p = moe_sum_plan<F>(N, K, top_k, tokens);
  if (!p.ok) return GGUF_ERR_SHAPE;
  const int64_t pitch = (int64_t)(K / F::QK) * F::BS;
  const MoeSumArgs moe = {ids, wts, (int64_t)N * pitch, (const char*)ws, q8_row_bytes(K), top_k, num_experts, p.slots, (int)q8_kp(K),
                          65536u / (uint32_t)top_k + 1u};
  const StreamGeom geom = stream_geom(N, K, p.rows_per_wg, pitch, 1, NW, p.rows.half);
  const auto go = [&](auto kern) {
    if (p.lds > 64 * 1024) {
      static std::atomic<uint64_t> done{0};
      allow_large_lds(kern, 160 * 1024, done);
    }
    hipLaunchKernelGGL(kern, dim3(p.grid, tokens), dim3(64 * NW), p.lds, stream, (const uint8_t*)W, (T*)out, moe, geom);
  };
  if (p.rows.half) go(moe_down_sum_kernel<F, NW, T, true>);
  else go(moe_down_sum_kernel<F, NW, T, false>);
  return launch_status();
}

template <class F>
static int moe_up_fmt(int dtype, const void* W, const void* X, const int32_t* ids, void* ws, int H, int I, int top_k, int tokens, int act,
                      int num_experts, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_up_typed<F, scalar_t>(W, X, ids, ws, H, I, top_k, tokens, act, num_experts, s)));
  return GGUF_ERR_DTYPE;
}
template <class F>
static int moe_sum_fmt(int dtype, const void* W, const void* ws, const int32_t* ids, const float* wts, void* out, int N, int K, int top_k,
                       int tokens, int num_experts, hipStream_t s) {
  GGUF_DISPATCH_DTYPE(dtype, return (moe_sum_typed<F, scalar_t>(W, ws, ids, wts, out, N, K, top_k, tokens, num_experts, s)));
  return GGUF_ERR_DTYPE;
}

#define GGUF_MOE_LAYER_FORMATS(CASE) \
  CASE(T_Q4_0, FmtQ4_0) CASE(T_Q4_1, FmtQ4_1) CASE(T_Q5_0, FmtQ5_0) CASE(T_Q5_1, FmtQ5_1) CASE(T_Q8_0, FmtQ8_0) CASE(T_Q2_K, FmtQ2_K) CASE(T_Q3_K, FmtQ3_K) \
  CASE(T_Q4_K, FmtQ4_K) CASE(T_Q5_K, FmtQ5_K) CASE(T_Q6_K, FmtQ6_K) CASE(T_IQ4_NL, FmtIQ4_NL) CASE(T_IQ4_XS, FmtIQ4_XS) \
  CASE(T_IQ2_XXS, FmtIQ2_XXS) CASE(T_IQ2_XS, FmtIQ2_XS) CASE(T_IQ2_S, FmtIQ2_S) CASE(T_IQ3_XXS, FmtIQ3_XXS) CASE(T_IQ3_S, FmtIQ3_S) \
  CASE(T_IQ1_S, FmtIQ1_S) CASE(T_IQ1_M, FmtIQ1_M)

// 0: not served; 1: the two launches above; 2 / 3: four launches on the tile kernels with blocks of 16 / 32 slots (experts
// shared by a few pairs each)
static int moe_layer_takes(int type13, int type2, int H, int I, int N_out, int top_k, int tokens, int num_experts) {
  const int qk13 = block_elems(type13), qk2 = block_elems(type2);
  if (qk13 == 0 || qk2 == 0 || H % qk13 != 0 || I % qk2 != 0 || I % 32 != 0) return 0;
  // where experts are shared by enough pairs the per-pair operator reads each once per group of pairs instead
  const int64_t pairs = (int64_t)tokens * top_k;
  const bool shared13 = num_experts > 0 && moe_share_pays(pairs, num_experts, (int64_t)2 * I * (H / qk13) * block_bytes(type13));
  const bool shared2 = num_experts > 0 && moe_share_pays(pairs, num_experts, (int64_t)N_out * (I / qk2) * block_bytes(type2));
  if (shared13 || shared2) {
    // (where only one of the two says so -- the thresholds differ by half a pair per expert between experts that fit the
    //  last-level cache together and experts that do not -- the other is near its own break-even: both go to the tiles)
    const int block = moe_tiles_layer_block(type13, type2, pairs, num_experts, I, true);
    return block == 16 ? 2 : block == 32 ? 3 : 0;
  }
  bool up = false, down = false;
  switch (type13) {
#define MOE_LAYER_CASE(ID, FMT) case ID: up = moe_up_plan<FMT>(H, I, (int)pairs).ok; break;
    GGUF_MOE_LAYER_FORMATS(MOE_LAYER_CASE)
#undef MOE_LAYER_CASE
  }
  switch (type2) {
#define MOE_LAYER_CASE(ID, FMT) case ID: down = moe_sum_plan<FMT>(N_out, I, top_k, tokens).ok; break;
    GGUF_MOE_LAYER_FORMATS(MOE_LAYER_CASE)
#undef MOE_LAYER_CASE
  }
  return up && down ? 1 : 0;
}

}  // namespace gguf

static bool moe_layer_sizes_ok(int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens) {
  return H > 0 && I > 0 && N_out > 0 && top_k > 0 && tokens > 0 && H <= 0x7FFFFFF0LL && 2 * I <= 0x7FFFFFF0LL && N_out <= 0x7FFFFFF0LL &&
         tokens * top_k <= 65535;
}

extern "C" int gguf_moe_vec_layer_takes(int type13, int type2, int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens,
                                        int64_t num_experts) {
  if (!moe_layer_sizes_ok(H, I, N_out, top_k, tokens)) return 0;
  return gguf::moe_layer_takes(type13, type2, (int)H, (int)I, (int)N_out, (int)top_k, (int)tokens,
                               num_experts > 0 && num_experts <= 1024 ? (int)num_experts : 0);
}

extern "C" int64_t gguf_moe_vec_layer_workspace_bytes(int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out, int64_t num_experts,
                                                      int xdtype) {
  if (tokens <= 0 || top_k <= 0 || H <= 0 || I <= 0 || N_out <= 0 || num_experts < 0) return 0;
  const int64_t pair_rows = tokens * top_k * gguf::q8_row_bytes(I);
  const int elt = xdtype == GGUF_DTYPE_F32 ? 4 : 2;
  const int64_t t16 = gguf::moe_tiles_layer_workspace(tokens, top_k, H, I, N_out, num_experts, elt, 16);
  const int64_t t32 = gguf::moe_tiles_layer_workspace(tokens, top_k, H, I, N_out, num_experts, elt, 32);
  const int64_t tiles = t16 > t32 ? t16 : t32;
  return pair_rows > tiles ? pair_rows : tiles;
}

extern "C" int gguf_moe_vec_layer(const void* X, int xdtype, const void* W13, int type13, const void* W2, int type2, const int32_t* topk_ids,
                                  const float* topk_weights, void* workspace, int64_t workspace_bytes, void* out, int64_t H, int64_t I,
                                  int64_t N_out, int64_t top_k, int64_t tokens, int act, int64_t num_experts, gguf_stream_t stream) {
  using namespace gguf;
  if (act != ACT_SILU && act != ACT_GELU) return GGUF_ERR_SHAPE;
  if (block_elems(type13) == 0 || block_elems(type2) == 0) return GGUF_ERR_TYPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (tokens == 0) return GGUF_OK;
  if (!moe_layer_sizes_ok(H, I, N_out, top_k, tokens)) return GGUF_ERR_SHAPE;
  if (!X || !W13 || !W2 || !topk_ids || !topk_weights || !workspace || !out) return GGUF_ERR_NULL;
  if (((uintptr_t)W13 | (uintptr_t)W2) & 1) return GGUF_ERR_SHAPE;   // packed blocks sit at even addresses
  const int ne = num_experts > 0 && num_experts <= 1024 ? (int)num_experts : 0;
  const int route = moe_layer_takes(type13, type2, (int)H, (int)I, (int)N_out, (int)top_k, (int)tokens, ne);
  if (route == 0) return GGUF_ERR_SHAPE;
  hipStream_t s = (hipStream_t)stream;
  if (route >= 2) {
    const int block = route == 2 ? 16 : 32;
    if (workspace_bytes < moe_tiles_layer_workspace(tokens, top_k, H, I, N_out, ne, xdtype == GGUF_DTYPE_F32 ? 4 : 2, block)) return GGUF_ERR_WORKSPACE;
    return moe_tiles_layer(X, xdtype, workspace, W13, type13, W2, type2, topk_ids, topk_weights, out, (int)H, (int)I, (int)N_out, (int)top_k,
                           (int)tokens, act, ne, true, block, s);
  }
  if (workspace_bytes < tokens * top_k * q8_row_bytes(I)) return GGUF_ERR_WORKSPACE;
  int rc = GGUF_ERR_TYPE;
  switch (type13) {
#define MOE_LAYER_CASE(ID, FMT) \
  case ID: rc = moe_up_fmt<FMT>(xdtype, W13, X, topk_ids, workspace, (int)H, (int)I, (int)top_k, (int)tokens, act, ne, s); break;
    GGUF_MOE_LAYER_FORMATS(MOE_LAYER_CASE)
#undef MOE_LAYER_CASE
  }
  if (rc != GGUF_OK) return rc;
  switch (type2) {
#define MOE_LAYER_CASE(ID, FMT) \
  case ID: return moe_sum_fmt<FMT>(xdtype, W2, workspace, topk_ids, topk_weights, out, (int)N_out, (int)I, (int)top_k, (int)tokens, ne, s);
    GGUF_MOE_LAYER_FORMATS(MOE_LAYER_CASE)
#undef MOE_LAYER_CASE
  }
  return GGUF_ERR_TYPE;
}

// The same four launches with the grouped operator's arithmetic (gguf_moe_mmq_block twice and the weighted sum): what a
// layer with more than 64 tokens takes -- on blocks of 16 slots while its experts see at most 16 pairs each on average and
// both formats have such tiles (returns 1), else on the reference's blocks of 32 (returns 2); from MOE_SORTED_MIN_PAIRS
// pairs per expert on, where one of the formats changes its scale every 16 values (Q2_K, Q3_K, Q6_K: the 32-slot kernel
// multiplies those at half rate), the layer in slot order on the pipelined integer engine with blocks of 64 slots
// (returns 3).  Measured with Q4_K gate / up and a Q6_K down projection, against the 32-slot blocks at 64 pairs per
// expert: 8 experts [4096,14336] 12 % faster, 64 experts [2048,1024] 7 %, 128 experts [2048,768] 2 % slower; at 32 pairs
// per expert 4 - 6 % slower, at 128 pairs the 8-expert layer 26 % faster.  Blocks of 128 slots (128 x 64 tiles) were
// 1 - 13 % slower than blocks of 64 from 128 to 512 pairs per expert: half a block of padding per expert costs more than
// decoding each weight for 64 rows instead of 128.  Q4_0 layers gain nothing on either (64 experts: 0 - 22 % slower),
// hence the condition on the format.
static constexpr int64_t MOE_SORTED_MIN_PAIRS = 64, MOE_SORTED_BLOCK = 64;
// whether the layer runs in slot order
static bool moe_sorted_pays(int type13, int type2, int64_t pairs, int64_t num_experts) {
  using namespace gguf;
  const auto deep16 = [](int t) { return t == T_Q2_K || t == T_Q3_K || t == T_Q6_K; };
  return (deep16(type13) || deep16(type2)) && pairs >= MOE_SORTED_MIN_PAIRS * num_experts &&
         pairs + (MOE_SORTED_BLOCK - 1) * num_experts <= 65535;   // (a grid row per slot)
}
extern "C" int gguf_moe_mmq_layer_takes(int type13, int type2, int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens,
                                        int64_t num_experts) {
  using namespace gguf;
  if (!(H > 0 && I > 0 && N_out > 0 && top_k > 0 && tokens > 0 && H <= 0x7FFFFFF0LL && 2 * I <= 0x7FFFFFF0LL && N_out <= 0x7FFFFFF0LL)) return 0;
  if (num_experts <= 0 || num_experts > 256 || tokens > 0x7FFFFFF0LL / top_k || tokens * top_k + 31 * num_experts > 65535 * 32) return 0;   // (a grid row per block)
  const int qk13 = block_elems(type13), qk2 = block_elems(type2);
  if (qk13 == 0 || qk2 == 0 || H % qk13 != 0 || I % qk2 != 0) return 0;
  const int block = moe_tiles_layer_block(type13, type2, tokens * top_k, num_experts, I, false);
  if (block != 0 && moe_sorted_pays(type13, type2, tokens * top_k, num_experts)) return 3;
  return block == 16 ? 1 : block == 32 ? 2 : 0;
}

extern "C" int64_t gguf_moe_mmq_layer_workspace_bytes(int type13, int type2, int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out,
                                                      int64_t num_experts, int xdtype) {
  using namespace gguf;
  const int route = gguf_moe_mmq_layer_takes(type13, type2, H, I, N_out, top_k, tokens, num_experts);
  const int elt = xdtype == GGUF_DTYPE_F32 ? 4 : 2;
  if (route == 3) return moe_sorted_layer_workspace(tokens, top_k, H, I, N_out, num_experts, elt, (int)MOE_SORTED_BLOCK);
  return route ? moe_tiles_layer_workspace(tokens, top_k, H, I, N_out, num_experts, elt, route == 1 ? 16 : 32) : 0;
}

extern "C" int gguf_moe_mmq_layer(const void* X, int xdtype, const void* W13, int type13, const void* W2, int type2, const int32_t* topk_ids,
                                  const float* topk_weights, void* workspace, int64_t workspace_bytes, void* out, int64_t H, int64_t I,
                                  int64_t N_out, int64_t top_k, int64_t tokens, int act, int64_t num_experts, gguf_stream_t stream) {
  using namespace gguf;
  if (act != ACT_SILU && act != ACT_GELU) return GGUF_ERR_SHAPE;
  if (block_elems(type13) == 0 || block_elems(type2) == 0) return GGUF_ERR_TYPE;
  if (xdtype < 0 || xdtype > 2) return GGUF_ERR_DTYPE;
  if (tokens == 0) return GGUF_OK;
  const int route = gguf_moe_mmq_layer_takes(type13, type2, H, I, N_out, top_k, tokens, num_experts);
  if (!route) return GGUF_ERR_SHAPE;
  if (!X || !W13 || !W2 || !topk_ids || !topk_weights || !workspace || !out) return GGUF_ERR_NULL;
  if (((uintptr_t)W13 | (uintptr_t)W2) & 1) return GGUF_ERR_SHAPE;   // packed blocks sit at even addresses
  if (route == 3) {
    const int sorted_block = (int)MOE_SORTED_BLOCK;
    if (workspace_bytes < moe_sorted_layer_workspace(tokens, top_k, H, I, N_out, num_experts, xdtype == GGUF_DTYPE_F32 ? 4 : 2, sorted_block))
      return GGUF_ERR_WORKSPACE;
    return moe_sorted_layer(X, xdtype, workspace, W13, type13, W2, type2, topk_ids, topk_weights, out, (int)H, (int)I, (int)N_out, (int)top_k,
                            (int)tokens, act, (int)num_experts, sorted_block, (hipStream_t)stream);
  }
  const int block = route == 1 ? 16 : 32;
  if (workspace_bytes < moe_tiles_layer_workspace(tokens, top_k, H, I, N_out, num_experts, xdtype == GGUF_DTYPE_F32 ? 4 : 2, block))
    return GGUF_ERR_WORKSPACE;
  return moe_tiles_layer(X, xdtype, workspace, W13, type13, W2, type2, topk_ids, topk_weights, out, (int)H, (int)I, (int)N_out, (int)top_k,
                         (int)tokens, act, (int)num_experts, false, block, (hipStream_t)stream);
}
