/*
 * C ABI of the MI355X (gfx950) GGUF quantized-matmul library, libgguf_hip.so.
 *
 * Every entry point is the native half of one operator of the reference plugin's
 * extension module `_C_gguf` (vllm_gguf_plugin/csrc/torch_bindings.cpp:22-53); the
 * reference file:line each one replaces is cited next to it.  The ABI carries
 * plain pointers and sizes only: no torch types, no exceptions, no host
 * synchronisation and no allocation.  The caller owns every buffer, including the
 * activation-quantisation workspace, and passes the HIP stream to launch on.
 *
 * Conventions
 *   - all pointers are device pointers valid on the current HIP device;
 *   - W is the packed GGUF tensor, row-major, `K / block_elems * block_bytes`
 *     bytes per row, rows contiguous (what the reference receives as a uint8
 *     tensor);
 *   - X and Y are row-major and share one dtype, given as a GGUF_DTYPE_* code;
 *   - `type` is the ggml type id (2,3,6,7,8,10-14,16-23,29);
 *   - return value: 0 on success, a negative GGUF_ERR_* code otherwise.  On error
 *     nothing has been launched.  The reference's native ops do no validation at
 *     all (an unknown type returns zeros or calls a null pointer,
 *     gguf_kernel.cu:97-98,119-217); this library rejects such calls instead.
 */
#ifndef GGUF_HIP_H
#define GGUF_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GGUF_DTYPE_F32 0
#define GGUF_DTYPE_F16 1
#define GGUF_DTYPE_BF16 2

#define GGUF_OK 0
#define GGUF_ERR_TYPE (-1)   /* ggml type id not supported by this entry point */
#define GGUF_ERR_DTYPE (-2)  /* dtype code not one of GGUF_DTYPE_* */
#define GGUF_ERR_SHAPE (-3)  /* K not a multiple of the block size, negative size, ... */
#define GGUF_ERR_NULL (-4)   /* required pointer is null */
#define GGUF_ERR_LAUNCH (-5) /* hipLaunchKernel reported an error */
#define GGUF_ERR_WORKSPACE (-6) /* the call needs more workspace than the entry point has */

typedef void* gguf_stream_t; /* a hipStream_t */

/* Library version and the code-object architecture it was built for ("gfx950"). */
const char* gguf_hip_version(void);

/* Elements and bytes of one block of a ggml type; 0 if the type is unknown.
 * Replaces gguf.GGML_QUANT_SIZES as used at quantization/linear.py:51. */
int gguf_block_elems(int type);
int gguf_block_bytes(int type);

/* Bytes of activation workspace per row of X for inner dimension K.
 * The reference sizes its workspace as int32[M, roundup(K,512)/32*9]
 * (gguf_kernel.cu:114-115); this library's private layout needs 44 bytes per 32
 * values instead of 36 (int8 quants, then fp32 planes of the scale, the stored sum and
 * scale x quant sum), so callers must size the workspace with this function.  The
 * half-MFMA engine of gguf_mmq keeps a half-precision copy of the rows as well: its
 * callers size the workspace with gguf_mmq_workspace_bytes_engine(..., GGUF_MMQ_HALF). */
int64_t gguf_q8_1_row_bytes(int64_t K);

/* q8_1 activation quantizer: M rows of K values -> workspace.
 * Replaces quantize_q8_1 / quantize_row_q8_1_cuda (gguf_kernel.cu:32-85). */
int gguf_quantize_q8_1(const void* x, int xdtype, void* q8_workspace, int64_t M, int64_t K, gguf_stream_t stream);

/* Read back the reference-visible content of a workspace row set (test hook):
 * int8 quants [M, Kp] and (d, sum) as float pairs [M, Kp/32, 2], Kp = roundup(K,512). */
int gguf_q8_1_unpack(const void* q8_workspace, int8_t* q, float* ds, int64_t M, int64_t K, gguf_stream_t stream);

/* Dense values of `nelem` packed weights in element order.
 * Replaces ggml_dequantize (gguf_kernel.cu:87-102, dequantize.cuh:527-571). */
int gguf_dequantize(const void* W, int type, void* Y, int ydtype, int64_t nelem, gguf_stream_t stream);

/* Row gather fused with dequantisation: Y[i,:] = dense values of row row_ids[i] of the packed table W[n_rows, K].
 * Replaces torch.index_select followed by ggml_dequantize in the embedding path
 * (quantization/vocal_embeds.py:90-96).  A row id outside [0, n_rows) yields a row of zeros. */
int gguf_dequantize_rows(const void* W, int type, const int64_t* row_ids, int64_t n_ids, int64_t n_rows, int64_t K, void* Y,
                         int ydtype, gguf_stream_t stream);

/* Y[M,N] = q8_1(X[M,K]) . W[N,K]^T, decode GEMV path.
 * Replaces ggml_mul_mat_vec_a8 (gguf_kernel.cu:104-218, mmvq.cuh:2-212). */
int gguf_mmvq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N, int64_t K,
              int64_t M, gguf_stream_t stream);

/* Same contraction, prefill path on int8 MFMA.
 * Replaces ggml_mul_mat_a8 (gguf_kernel.cu:220-290, mmq.cuh:2-610). */
int gguf_mmq(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N, int64_t K,
             int64_t M, gguf_stream_t stream);

/* gguf_mmq with the arithmetic engine chosen by the caller.  The reference has one engine (dp4a, mmq.cuh:2-104);
 * this library has two:
 *   GGUF_MMQ_INT8  int8 MFMA on the block codes, block scales applied in fp32: the reference's arithmetic, differing
 *                  only in the order of the fp32 additions.  This is what gguf_mmq runs.
 *   GGUF_MMQ_HALF  half-precision MFMA on operands that carry their scales (activation d8*q and weight d*q, each
 *                  rounded to half): about 1.8 times faster, relative deviation about 2e-4 in the l2 norm, below
 *                  the rounding of a half or bfloat16 result -- but not the reference's arithmetic, so only for
 *                  callers that ask.  Not for fp32 results; not for Q4_1 / Q5_1.
 *   GGUF_MMQ_AUTO  INT8; with M <= 8 the streaming GEMV kernel instead, switched to this operator's offset sums
 *                  (Q4_K, Q5_K, Q5_0 are the formats where the reference's GEMV and its tile GEMM form them
 *                  differently), which is exact in int8 and reads W once at the GEMV's rate.
 * workspace_bytes is the size of q8_workspace; 0 stands for the minimum, M * gguf_q8_1_row_bytes(K).  Given
 * gguf_mmq_workspace_bytes(M, N, K) bytes, either engine splits K over several workgroups per output tile where the
 * output tiles alone would leave much of the chip idle (few tokens, a narrow N with a long K, a sparse last round of
 * tiles), keeping fp32 partial tiles behind the rows and adding them in a second launch in fixed order.  The result
 * does not depend on the run, only on the shape and on whether the room was given. */
#define GGUF_MMQ_AUTO 0
#define GGUF_MMQ_INT8 1
#define GGUF_MMQ_HALF 2
int64_t gguf_mmq_workspace_bytes(int64_t M, int64_t N, int64_t K);   /* room for either engine */
/* The same for one engine (GGUF_MMQ_AUTO counts as GGUF_MMQ_INT8): only the half engine pays for the half-precision
 * copy of the rows (64 bytes per 32 values on top of the 44).  GGUF_MMQ_HALF needs at least its row region,
 * M * (gguf_q8_1_row_bytes(K) + 2 * (roundup(K, 512) + 128)) bytes, and returns GGUF_ERR_WORKSPACE below that; for it
 * workspace_bytes = 0 is not accepted. */
int64_t gguf_mmq_workspace_bytes_engine(int64_t M, int64_t N, int64_t K, int engine);
int gguf_mmq_engine(const void* W, const void* x, int xdtype, void* q8_workspace, void* Y, int type, int64_t N, int64_t K,
                    int64_t M, int engine, int64_t workspace_bytes, gguf_stream_t stream);

/* gguf_mmq without a workspace argument, for callers that cannot allocate device memory: code running under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference (whose
 * operator allocates its result and workspace through torch on every call, gguf_kernel.cu:228-231).  The quantized rows and, for
 * shapes whose K is split, the fp32 partial tiles live in a fixed 32 MiB array of device memory that the library
 * holds on every GPU it runs on until the process ends; the call allocates and frees nothing.  Arithmetic, engine
 * choice and results are those of gguf_mmq_engine(..., GGUF_MMQ_AUTO, workspace_bytes) given the same room for
 * partial tiles.  GGUF_ERR_WORKSPACE if the quantized rows alone, M * roundup(K, 512) / 32 * 44 bytes rounded up to
 * 256, exceed the array.  Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 * streams, two threads) race; calls on one stream are ordered and need no clearing between them.
 * gguf_mmq_static_capacity returns the array's size (0 if the current device cannot be queried) and, as its side
 * effect, looks up the array's address for the current device; callers that are about to capture call it once
 * before they begin, so that the first gguf_mmq_static inside the capture does no set-up. */
int64_t gguf_mmq_static_capacity(void);
int gguf_mmq_static(const void* W, const void* x, int xdtype, void* Y, int type, int64_t N, int64_t K, int64_t M,
                    gguf_stream_t stream);

/* The two a8 operators for one shard of a merged linear layer.  quantization/linear.py:229-262 keeps the shards of a
 * fused layer (q/k/v, gate/up) in one uint8 tensor padded to the widest row; when their ggml types differ it copies
 * every shard out with .contiguous() on each forward pass, multiplies, concatenates the results and adds the bias.
 * These entry points read the shard where it lies and write where the result belongs:
 *   W                  first row of the shard; rows are w_row_pitch_bytes apart (>= K / block * block_bytes);
 *   Y                  first result column of the shard in the merged output; rows are y_row_pitch elements apart;
 *   bias               null, or N values of Y's dtype (the shard's slice of the layer bias), added to every row after
 *                      the product is rounded to Y's dtype, as out.add_(bias) does.
 * gguf_mmvq / gguf_mmq / gguf_mmq_engine are these with dense rows, y_row_pitch = N and no bias. */
int gguf_mmvq_linear(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                     int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M, gguf_stream_t stream);
int gguf_mmq_linear(const void* W, int64_t w_row_pitch_bytes, const void* x, int xdtype, void* q8_workspace, void* Y,
                    int64_t y_row_pitch, const void* bias, int type, int64_t N, int64_t K, int64_t M, int engine,
                    int64_t workspace_bytes, gguf_stream_t stream);

/* Y[M,N] = X[M,K] . dequant(W[N,K])^T with the activations as they are (no q8_1 quantisation): one GEMM on
 * half-precision MFMA that decodes the packed blocks on the fly instead of the reference's fallback for formats and
 * batch sizes without an a8 kernel, ggml_dequantize followed by x @ weight.T (quantization/linear.py:50-58,
 * diffusion_config.py:21-30), which writes and re-reads the dense weights.  The weights take the half-precision
 * values the reference's dequantize kernels produce; X is converted to half.  X / Y dtype: fp16 or bf16.  Types: the
 * twelve standard and K formats plus IQ4_XS and IQ2_XXS.  Workspace: gguf_mmq_workspace_bytes_engine(M, N, K,
 * GGUF_MMQ_HALF); GGUF_ERR_WORKSPACE below the half engine's row region. */
int gguf_dequant_gemm(const void* W, const void* x, int xdtype, void* workspace, void* Y, int type, int64_t N, int64_t K,
                      int64_t M, int64_t workspace_bytes, gguf_stream_t stream);

/* Grouped (MoE) variant: for every sorted slot s with p = sorted_token_ids[s] < tokens*top_k,
 * Y[p,:] = q8_1(X[p / top_k,:]) . W[expert_ids[s / block],:,:]^T.  Rows of Y that no slot names are zero.
 * Replaces ggml_moe_a8 (gguf_kernel.cu:292-393, moe.cuh:5-739).  `block` must equal
 * gguf_moe_block_size(type). */
int gguf_moe_mmq(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                 const int32_t* sorted_token_ids, const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                 int64_t num_sorted, void* Y, int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens,
                 gguf_stream_t stream);

/* Per-pair MoE GEMV: Y[z,:] = q8_1(X[z / top_k,:]) . W[topk_ids[z],:,:]^T for z < tokens*top_k.
 * Replaces ggml_moe_a8_vec (gguf_kernel.cu:395-530, moe_vec.cuh:3-338).  Experts are densely packed. */
int gguf_moe_vec(const void* X, int xdtype, void* q8_workspace, const void* W, const int32_t* topk_ids, void* Y, int type,
                 int64_t N, int64_t K, int64_t top_k, int64_t tokens, gguf_stream_t stream);

/* The two MoE entry points with the layer's gated activation folded into their activation quantisation: X has
 * 2*K columns per row, [gate | up], and the kernels see act(gate) * up rounded to X's dtype exactly as a separate
 * activation kernel would have stored it (quantization/fused_moe.py:44-51,80,92: act() between the two GEMMs).
 * act: 0 = none (X has K columns, same as the plain entry points), 1 = SiLU, 2 = GELU (erf).
 * gguf_moe_vec_act also takes the number of experts in W (0 = unknown) and the size of the workspace (0 = the
 * minimum, tokens * gguf_q8_1_row_bytes(K)).  When experts are shared -- tokens*top_k >= 2*num_experts, or >= 2.5 *
 * num_experts while all experts together are at most 192 MiB and so stay in the last-level cache, where the per-pair
 * kernel reads them from -- and the workspace has room for the routing sort as well, gguf_moe_vec_workspace_bytes(),
 * the pairs are sorted by expert, the activations quantized once, and the pairs of an expert share each pass over its
 * weights, so a shared expert is read about once per call rather than once per pair (the reference's grid re-reads it
 * per pair, moe_vec.cuh:3-53): on the grouped int8-MFMA kernels for the formats that have tiles (up to 256 experts;
 * Q5_0 excepted) -- blocks of 16 slots while tokens*top_k <= 16*num_experts (Q4_0, Q8_0, Q3_K, Q4_K, Q5_K, Q6_K,
 * IQ4_XS, IQ2_XXS), blocks of 32 above -- and four pairs per pass on the vector kernel for the others.  The operator's arithmetic is the GEMV's on every route (Q4_K / Q5_K offsets from the
 * quant sums); results agree to fp32 summation order. */
int64_t gguf_moe_vec_workspace_bytes(int64_t tokens, int64_t top_k, int64_t K, int64_t num_experts);
int gguf_moe_mmq_act(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                     const int32_t* sorted_token_ids, const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                     int64_t num_sorted, void* Y, int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens, int act,
                     gguf_stream_t stream);
int gguf_moe_vec_act(const void* X, int xdtype, void* q8_workspace, const void* W, const int32_t* topk_ids, void* Y, int type,
                     int64_t N, int64_t K, int64_t top_k, int64_t tokens, int act, int64_t num_experts, int64_t workspace_bytes,
                     gguf_stream_t stream);

/* Token-tile size that moe_align_block_size must pad expert groups to; 0 for unknown types.
 * Replaces ggml_moe_get_block_size (gguf_kernel.cu:532-566). */
int gguf_moe_block_size(int type);

/* The grouped operator with the block size of the routing sort stated by the caller, 32 or 16, and the number of
 * experts in W (0 = not stated).  The reference tiles 4 or 8 tokens (moe.cuh:131-139, gguf_kernel.cu:532-566); here
 * blocks of 32 slots suit experts with many pairs and blocks of 16 (int8 MFMA 16x16 tiles; Q4_0, Q8_0, Q3_K, Q4_K,
 * Q5_K, Q6_K, IQ4_XS, IQ2_XXS, GGUF_ERR_TYPE otherwise) suit a layer whose experts see 12 pairs or fewer on average, where most
 * of a 32-slot block would be padding: gguf_moe_block_size_for(type, tokens * top_k, num_experts) returns the one to
 * sort with.  Arithmetic is the tile operator's either way (offset terms on the stored block sums).  num_experts above
 * 256 is GGUF_ERR_SHAPE: the kernels keep the reference's guard that skips blocks of experts above 255 (moe.cuh:33),
 * and a caller who states the count is told instead of receiving rows of zeros.  act as for gguf_moe_mmq_act. */
int gguf_moe_block_size_for(int type, int64_t pairs, int64_t num_experts);
int gguf_moe_mmq_block(const void* X, int xdtype, void* q8_workspace, const void* W, int64_t expert_stride_bytes,
                       const int32_t* sorted_token_ids, const int32_t* expert_ids, const int32_t* num_tokens_post_padded,
                       int64_t num_sorted, void* Y, int type, int64_t N, int64_t K, int64_t top_k, int64_t tokens, int act,
                       int64_t block, int64_t num_experts, gguf_stream_t stream);

/* Routing sort for the grouped kernel: pairs (flat index token*top_k + choice) grouped by expert in ascending index
 * order, every expert's run padded to a multiple of `block` with the value `numel`; one expert id per block (-1 past
 * the padded total); the padded total.  Capacities: sorted >= numel + num_experts*(block-1), experts >= that / block
 * rounded up.  The reference takes this from vLLM (quantization/fused_moe.py:53-66, moe_align_block_size); the
 * meaning of the three outputs is the one moe.cuh:20-45 consumes.  num_experts <= 1024. */
int gguf_moe_align_block_size(const int32_t* topk_ids, int64_t numel, int64_t num_experts, int64_t block,
                              int32_t* sorted_token_ids, int64_t sorted_capacity, int32_t* expert_ids,
                              int64_t expert_capacity, int32_t* num_tokens_post_padded, gguf_stream_t stream);

/* out[t,:] = sum over k of round(Y[t*top_k + k,:] * topk_weights[t,k]) with fp32 accumulation, one launch for
 * out.mul_(topk_weights) followed by ops.moe_sum (quantization/fused_moe.py:87-95, ops.py:285-286). */
int gguf_moe_weighted_sum(const void* Y, const float* topk_weights, void* out, int dtype, int64_t tokens, int64_t top_k,
                          int64_t N, gguf_stream_t stream);

/* A whole MoE layer on the per-pair operators' arithmetic in one call: X[tokens][H] -> out[tokens][N_out] through
 * W13[E][2 I][H packed] ([gate | up] rows) and W2[E][N_out][I packed], with topk_ids[tokens][top_k] and fp32
 * topk_weights[tokens][top_k] (ggml_moe_a8_vec, act(), ggml_moe_a8_vec, out.mul_(topk_weights), ops.moe_sum:
 * quantization/fused_moe.py:98-111; here gguf_moe_vec, gguf_moe_vec_act and gguf_moe_weighted_sum in sequence, whose
 * result it reproduces up to the last bit of the fp32 dot products -- every intermediate is rounded to the dtype where
 * those steps store it).  No counterpart as one call in the reference.  gguf_moe_vec_layer_takes says how a layer is
 * served:
 *   1  a few tokens, experts not shared (fewer than 2 - 2.5 pairs per expert): two launches.  The first GEMV's workgroups
 *      own the same features in the gate and the up half, apply the activation and write h as q8_1 rows into the
 *      workspace; the second's own a band of output features of one token, walk it in all top_k experts and form the
 *      weighted sum, so neither [tokens*top_k][2 I] nor [tokens*top_k][N_out] exists in memory.
 *   2  experts shared by a few pairs each (at most 16 per expert on average, formats with 16-slot tiles, E <= 256): four
 *      launches on the tile kernels -- one that quantizes X and sorts the routing for both GEMMs, first GEMM with the
 *      activation and the quantisation of its result in the epilogue, second GEMM from those rows, weighted sum -- where
 *      the separate operators take seven.
 *   3  the same four launches on blocks of 32 slots: shared experts in the other tile formats (Q4_1, Q5_1, Q2_K) or with
 *      more than 16 pairs each.
 *   0  not served (I no multiple of 32 or of type2's block, top_k times the waves a row of W2 takes beyond a workgroup,
 *      more than 65535 pairs, shared experts in a format without tiles or in Q5_0, whose tile arithmetic is not its
 *      GEMV's, or more than 256 of them): gguf_moe_vec_layer returns GGUF_ERR_SHAPE.
 * workspace: gguf_moe_vec_layer_workspace_bytes(...) bytes, layout private; GGUF_ERR_WORKSPACE if workspace_bytes is less
 * than the route needs.  act: 1 = SiLU, 2 = GELU.  A pair whose expert id is outside [0, num_experts) (num_experts > 0)
 * adds nothing on route 1. */
int gguf_moe_vec_layer_takes(int type13, int type2, int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens,
                             int64_t num_experts);
int64_t gguf_moe_vec_layer_workspace_bytes(int64_t tokens, int64_t top_k, int64_t H, int64_t I, int64_t N_out,
                                           int64_t num_experts, int xdtype);
int gguf_moe_vec_layer(const void* X, int xdtype, const void* W13, int type13, const void* W2, int type2,
                       const int32_t* topk_ids, const float* topk_weights, void* workspace, int64_t workspace_bytes,
                       void* out, int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens, int act,
                       int64_t num_experts, gguf_stream_t stream);

/* The same layer on the grouped operator's arithmetic (moe_align_block_size, ggml_moe_a8, act(), ggml_moe_a8,
 * out.mul_(topk_weights), ops.moe_sum: quantization/fused_moe.py:62-95; here gguf_moe_align_block_size with blocks of
 * 16 or 32 slots, gguf_moe_mmq_block, gguf_moe_mmq_block with act and gguf_moe_weighted_sum in sequence, whose result it
 * reproduces up to the last bit of the fp32 dot products), for layers with more than 64 tokens: the four launches of
 * route 2 above where the separate operators take nine (sort; zero-fill, quantize and GEMM twice; weighted sum).  No
 * counterpart as one call in the reference.  gguf_moe_mmq_layer_takes:
 *   1  blocks of 16 slots: both formats have such tiles and tokens * top_k <= 16 num_experts;
 *   2  the reference's blocks of 32 slots: every other layer of two tile formats (the twelve of ggml_moe_a8);
 *   0  not served (num_experts outside 1..256, I no multiple of 32 or of type2's block, a format without tiles, more
 *      than about two million pairs): gguf_moe_mmq_layer returns GGUF_ERR_SHAPE.
 *   3  experts that see 64 pairs or more each on average, one of the formats being Q2_K, Q3_K or Q6_K: six launches on
 *      the pipelined integer engine of gguf_mmq with blocks of 64 slots -- the routing sort with its inverse, the rows of X quantized into slot order, the
 *      first GEMM as a dense product over runs of rows (only the weight matrix changes from block to block), its
 *      result quantized with the activation, the second GEMM, and the weighted sum gathering its rows through the
 *      inverse of the sort.
 * A pair whose expert id is outside [0, num_experts) adds nothing, like the rows the grouped operator leaves at zero.
 * Workspace: gguf_moe_mmq_layer_workspace_bytes(...) bytes for the route the same arguments take (0 where none does). */
int gguf_moe_mmq_layer_takes(int type13, int type2, int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens,
                             int64_t num_experts);
int64_t gguf_moe_mmq_layer_workspace_bytes(int type13, int type2, int64_t tokens, int64_t top_k, int64_t H, int64_t I,
                                           int64_t N_out, int64_t num_experts, int xdtype);
int gguf_moe_mmq_layer(const void* X, int xdtype, const void* W13, int type13, const void* W2, int type2,
                       const int32_t* topk_ids, const float* topk_weights, void* workspace, int64_t workspace_bytes,
                       void* out, int64_t H, int64_t I, int64_t N_out, int64_t top_k, int64_t tokens, int act,
                       int64_t num_experts, gguf_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* GGUF_HIP_H */
