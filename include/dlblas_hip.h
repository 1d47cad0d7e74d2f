/*
 * dlblas_hip.h -- C ABI of libdlblas_hip.so: hand-written gfx950 (MI355X) kernels for the
 * dlBLAS LLM-inference operator set.
 *
 * The reference library (DLCompiler's dlBLAS) has no FFI boundary: its Python host wrappers
 * launch Triton kernels.  Each entry point below replaces one such "host wrapper -> Triton
 * launch" pair; the reference location is cited per function as
 * python/dlBLAS/dlblas/kernels/<file>:<lines>.
 *
 * Conventions (all entry points):
 *   - plain pointers to DEVICE memory, sizes and strides in ELEMENTS unless stated otherwise;
 *   - the library never allocates or frees: outputs and workspaces are caller-owned;
 *   - `stream` is a hipStream_t passed as void*; every call is asynchronous on it, re-entrant,
 *     and holds no mutable global state;
 *   - return value: DLB_OK (0) or a negative DLB_ERR_* code; nothing is launched on error.
 */
#ifndef DLBLAS_HIP_H_
#define DLBLAS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DLB_OK 0
#define DLB_ERR_BAD_ARG (-1)     /* null pointer, negative size, inconsistent shapes        */
#define DLB_ERR_UNSUPPORTED (-2) /* legal request the kernels do not cover (shape/dtype)    */
#define DLB_ERR_LAUNCH (-3)      /* hipGetLastError() != hipSuccess after the launch        */
#define DLB_ERR_WORKSPACE (-4)   /* workspace pointer null or too small                     */

/* element types of activations */
#define DLB_DTYPE_BF16 0
#define DLB_DTYPE_F16 1
#define DLB_DTYPE_F32 2

/* ABI version: bumped whenever a signature below changes; dlb_version() returns the value the
 * library was built with, and a binding should refuse a library whose version differs. */
#define DLB_ABI_VERSION 5
int dlb_version(void);

/* Index arrays (block tables, sequence lengths, start offsets) are read in the integer width the
 * caller's framework holds them in: every entry point that takes such arrays has an
 * `index64_mask` argument whose bit i is set when the i-th index array of its signature (in
 * argument order) holds int64 instead of int32.  Values must lie in [0, 2^31). */
/* static string for a status code (never NULL). */
const char* dlb_status_string(int status);

/* ------------------------------------------------------------------------------------------
 * silu_and_mul: out[m, j] = silu(x[m, j]) * x[m, N + j], math in fp32, one rounding to dtype.
 * Replaces silu_and_mul + _silu_and_mul[_no_align]_kernel, kernels/activation.py:17-130.
 *   x   [M, 2N] row stride ld_x (elements), unit column stride
 *   out [M, N]  row stride ld_out
 * Any M >= 0, N >= 0; a 128-bit vector path is taken when N % 8 == 0 (bf16/f16) or N % 4 == 0
 * (f32) and pointers/strides are 16-byte aligned, otherwise an element-wise path.
 * ---------------------------------------------------------------------------------------- */
int dlb_silu_and_mul(const void* x, void* out, int64_t M, int64_t N, int64_t ld_x,
                     int64_t ld_out, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * moe_topk_softmax: router softmax over experts + top-k (+ renormalise).
 * Replaces the router the reference leaves to the caller in torch
 * (tests/kernels/test_fused_moe.py:213-216: softmax(fp32) then torch.topk; renormalise
 * kernels/fused_moe.py:322-323) and the fused softmax+argmax of
 * kernels/topk_gating_fwd_part1.py:24-60.
 *   logits  [T, E] of type logits_dtype (DLB_DTYPE_F32, or BF16 / F16 converted to fp32 on the
 *           way in, as the reference's gate kernel does, topk_gating_fwd_part1.py:44-46),
 *           row stride ld_logits (elements)
 *   weights fp32 [T, K] (contiguous) ; ids int32 [T, K] (contiguous)
 * Selection is on the logits, descending, ties to the LOWEST expert index; weights are
 * p = exp(l - max) / sum(exp(l - max)) of the selected experts, divided by their sum when
 * renormalize != 0.  1 <= K <= 16, K <= E <= 256.
 * Two optional outputs (NULL to skip) are those of the reference's fused gate kernel
 * _topk_gating_kernel_part1 / call, kernels/topk_gating_fwd_part1.py:24-81:
 *   probs fp32 [T, E] (contiguous): the full softmax row ("gates");
 *   masks int64 [K, T, E] (contiguous): masks[r, t, :] is the one-hot row of the r-th selected
 *         expert of token t (the reference's K rounds of argmax / overwrite, :52-60).
 * ---------------------------------------------------------------------------------------- */
int dlb_moe_topk_softmax_f32(const void* logits, float* weights, int32_t* ids, float* probs,
                             int64_t* masks, int64_t T, int E, int K, int64_t ld_logits,
                             int logits_dtype, int renormalize, void* stream);

/* ------------------------------------------------------------------------------------------
 * moe_align_block_size: per-expert counts, expert-sorted flat slot ids padded per expert to a
 * multiple of `block`, and the expert of every block.
 * Replaces the routing bookkeeping of fused_moe: argsort + get_start_end/_start_end_kernel,
 * kernels/fused_moe.py:238-293,314-320 (the pad-to-block layout itself has no reference
 * counterpart).
 *   topk_ids    int32 [numel], or int64 with ids_int64 != 0 (what torch.topk returns and the
 *               reference's callers hand over, kernels/fused_moe.py:296-320); flat index
 *               i = token * K + j; ids outside [0, E) are dropped
 *   sorted_ids  int32 [sorted_cap], sorted_cap >= numel + E * (block - 1):
 *               expert segments in expert order, each a multiple of `block` long, holding the
 *               flat indices of that expert ASCENDING, then pad slots; every slot that is not
 *               a real entry (pads and the tail up to sorted_cap) holds the sentinel `numel`
 *   expert_ids  int32 [expert_ids_cap], expert_ids_cap >= ceil(sorted_cap / block):
 *               expert of block b for b < num_post_pad / block, -1 after
 *   counts      int32 [E] tokens per expert (may be NULL)
 *   num_post_pad int32 [1] total padded length
 *   ws          device scratch of dlb_moe_align_ws_bytes(numel, E) bytes
 * 1 <= E <= 256, block >= 1, numel < 2^31 - E * block.
 * ---------------------------------------------------------------------------------------- */
size_t dlb_moe_align_ws_bytes(int64_t numel, int E);
int dlb_moe_align_block_size(const void* topk_ids, int ids_int64, int64_t numel, int E, int block,
                             int32_t* sorted_ids, int64_t sorted_cap, int32_t* expert_ids,
                             int64_t expert_ids_cap, int32_t* counts, int32_t* num_post_pad,
                             void* ws, size_t ws_bytes, void* stream);

/* dlb_moe_align_block_size and dlb_per_token_group_quant_fp8 (declared further down) as one
 * pipeline of two launches instead of three: the activation quantiser runs in the launch of the
 * alignment's placement pass (the two jobs are independent).  Arguments and results are those of
 * the two functions, bit for bit; it is what fused_moe_fp8 runs in front of its GEMMs (the
 * reference sorts inside fused_moe as well, kernels/fused_moe.py:314-320).  Inputs beyond 524288
 * routing slots fall back to the separate launches. */
int dlb_moe_align_quant_fp8(const void* topk_ids, int ids_int64, int64_t numel, int E, int block,
                            int32_t* sorted_ids, int64_t sorted_cap, int32_t* expert_ids,
                            int64_t expert_ids_cap, int32_t* counts, int32_t* num_post_pad,
                            void* ws, size_t ws_bytes, const void* x, void* xq, float* xs,
                            int64_t M, int K, int64_t ld_x, int64_t ld_q, int64_t ld_s, int dtype,
                            void* stream);

/* ------------------------------------------------------------------------------------------
 * dlb_moe_align_block_size without a workspace argument and without any allocation: same
 * arguments, same results bit for bit.  It has no counterpart in the reference; it exists for
 * callers that cannot allocate device memory around the call (code under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  The scratch (the per-chunk count
 * table) is a 256 KB array in the library's device image, one copy per GPU, held until the
 * process ends.  Limit: numel <= dlb_moe_align_block_size_static_max_numel() (524288 routing
 * slots); more returns DLB_ERR_WORKSPACE.  All calls on one GPU share that GPU's array: calls
 * that overlap on one GPU (different streams) race; calls on one stream are ordered.  Nothing
 * in the array has to be cleared between calls.  The first call on a device looks up the array's
 * address there (hipGetSymbolAddress, which may load the library's device code): make one call on
 * every device outside stream capture before the entry point is used in a captured region.
 * ---------------------------------------------------------------------------------------- */
int64_t dlb_moe_align_block_size_static_max_numel(void);
int dlb_moe_align_block_size_static(const void* topk_ids, int ids_int64, int64_t numel, int E, int block,
                                    int32_t* sorted_ids, int64_t sorted_cap,
                                    int32_t* expert_ids, int64_t expert_ids_cap, int32_t* counts,
                                    int32_t* num_post_pad, void* stream);

/* ------------------------------------------------------------------------------------------
 * Router and alignment in one call (two launches instead of three): the outputs of
 * dlb_moe_topk_softmax_f32 followed by dlb_moe_align_block_size on its ids, bit for bit.
 * The same reference lines as the two calls above: the router of
 * tests/kernels/test_fused_moe.py:213-216 + kernels/fused_moe.py:322-323 and the routing
 * bookkeeping of kernels/fused_moe.py:238-293,314-320.
 * Arguments as in those two functions (numel = T * K); ws of
 * dlb_moe_topk_softmax_align_ws_bytes(T, E) bytes.  Returns DLB_ERR_UNSUPPORTED for more than
 * 32768 tokens: make the two calls then.
 * ---------------------------------------------------------------------------------------- */
size_t dlb_moe_topk_softmax_align_ws_bytes(int64_t T, int E);
int dlb_moe_topk_softmax_align_f32(const void* logits, float* weights, int32_t* ids, int64_t T,
                                   int E, int K, int64_t ld_logits, int logits_dtype,
                                   int renormalize, int block,
                                   int32_t* sorted_ids, int64_t sorted_cap, int32_t* expert_ids,
                                   int64_t expert_ids_cap, int32_t* counts, int32_t* num_post_pad,
                                   void* ws, size_t ws_bytes, void* stream);

/* ------------------------------------------------------------------------------------------
 * Paged decode attention: one query token per sequence against a paged KV cache, GQA.
 * Replaces the decode branch of paged_attention_fwd, kernels/paged_attention.py:604-671
 * (_fwd_grouped_split_kernel :45-234 and _reduce_split_kernel :238-285).
 *   q            [B, Hq, D]            strides q_stride_b, q_stride_h, unit last stride
 *   k cache      [pages, page, Hkv, D] strides k_stride_page, k_stride_tok, k_stride_head
 *   v cache      [pages, page, Hkv, Dv] strides v_stride_page, v_stride_tok, v_stride_head
 *   o            [B, Hq, Dv]           strides o_stride_b, o_stride_h
 *   block_table  int32/int64 [B, max_blocks] row stride bt_stride (elements): physical page of
 *                logical page j (index64_mask bit 0)
 *   kv_len       int32/int64 [B]       context length; rows with kv_len <= 0 produce zeros
 *                (index64_mask bit 1); the reference reads both in whatever integer type arrives,
 *                kernels/paged_attention.py:492-559
 * out[b, h] = softmax(q[b, h] . K[b, h / (Hq/Hkv)]^T * sm_scale) V, softmax in fp32 and P
 * rounded to `dtype` before P.V, as in the reference.
 * window_size > 0 masks keys older than kv_len - 1 - window_size (sliding window,
 * paged_attention.py:163-167,191-199); logit_softcapping > 0 replaces the scaled logits by
 * cap * tanh(logits / cap) (:186-189); pass <= 0 to disable either.
 * Supported: dtype bf16/f16, key head size D and value head size Dv any multiples of 8 up to
 * 256 (64 and 128 run the unmasked kernels; other sizes are computed in the next of 64, 128 and
 * 256 with the extra dims masked, as the reference splits them into power-of-two blocks,
 * kernels/paged_attention.py:531-539; sizes above 128 run one wavefront per SIMD), page % 16 == 0, all strides multiples of 8 and base
 * pointers 16-byte aligned.  ws: dlb_paged_decode_ws_bytes(B, Hq, Hkv, max(D, Dv), page,
 * max_blocks) bytes of device scratch (split-KV partials), caller-owned.
 * ---------------------------------------------------------------------------------------- */
size_t dlb_paged_decode_ws_bytes(int B, int Hq, int Hkv, int D, int page, int max_blocks);
int dlb_paged_decode_attn(const void* q, const void* k_cache, const void* v_cache, void* o,
                          const void* block_table, const void* kv_len, int index64_mask, int B,
                          int Hq, int Hkv, int D, int Dv, int page, int max_blocks, int64_t q_stride_b,
                          int64_t q_stride_h, int64_t k_stride_page, int64_t k_stride_tok,
                          int64_t k_stride_head, int64_t v_stride_page, int64_t v_stride_tok,
                          int64_t v_stride_head, int64_t o_stride_b, int64_t o_stride_h,
                          int64_t bt_stride, float sm_scale, int window_size,
                          float logit_softcapping, int dtype, void* ws, size_t ws_bytes,
                          void* stream);

/* ------------------------------------------------------------------------------------------
 * Varlen causal flash-attention prefill on packed sequences, GQA.
 * Replaces context_attention_fwd + _fwd_kernel, kernels/prefill_attention.py:39-181.
 *   q [tokens, Hq, D], k/v [tokens, Hkv, D], o [tokens, Hq, D]; token and head strides given,
 *   unit stride in D.  Sequence s owns tokens start_loc[s] .. start_loc[s] + seq_len[s] - 1
 *   (int32 or int64 [B] each: index64_mask bit 0 = start_loc, bit 1 = seq_len; with cu_seqlens:
 *   start_loc = cu[:-1], seq_len = cu[1:] - cu[:-1]).
 *   max_len >= max(seq_len) sizes the grid (the reference's max_input_len).
 * o[t, h] = sum_{t' <= t, same sequence} softmax_t'(q[t, h] . k[t', h / (Hq/Hkv)] * sm_scale)
 *           v[t', h / (Hq/Hkv)], softmax in fp32, P rounded to `dtype` before P.V.
 * (The reference fixes sm_scale = 1/sqrt(D); pass that for drop-in behaviour.)
 * Supported: dtype bf16/f16, D any multiple of 8 up to 256 (the reference asserts
 * D in {16, 32, 64, 128}, prefill_attention.py:160; sizes above 128 run one wavefront per SIMD), q/k/v strides multiples of 8 and bases
 * 16-byte aligned, o strides multiples of 4 and base 8-byte aligned.  Tokens outside every
 * sequence are not written.
 * ---------------------------------------------------------------------------------------- */
int dlb_prefill_attn_varlen(const void* q, const void* k, const void* v, void* o,
                            const void* start_loc, const void* seq_len, int index64_mask, int B,
                            int Hq, int Hkv, int D, int max_len, int64_t q_stride_tok,
                            int64_t q_stride_head, int64_t k_stride_tok, int64_t k_stride_head,
                            int64_t v_stride_tok, int64_t v_stride_head, int64_t o_stride_tok,
                            int64_t o_stride_head, float sm_scale, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Causal attention of new query tokens over a paged KV cache that already holds them and
 * their history (chunked prefill / prefix-cache hit), GQA.
 * Replaces the non-decoding branch of paged_attention_fwd + _fwd_kernel,
 * kernels/paged_attention.py:319-489, 559-607.
 *   q [tokens, Hq, D], o [tokens, Hq, Dv]: sequence s owns query tokens q_start_loc[s] ..
 *   q_start_loc[s] + q_len[s] - 1; k_cache [pages, page, Hkv, D], v_cache [pages, page, Hkv, Dv];
 *   block_table [B, max_blocks]; kv_len [B] = history + q_len[s] (sequences with kv_len < q_len
 *   are skipped); the four index arrays are int32 or int64 (index64_mask bit 0 = block_table,
 *   1 = q_start_loc, 2 = q_len, 3 = kv_len).  Query i of sequence s sits at context position kv_len[s] - q_len[s] + i and
 *   sees keys 0 .. that position (paged_attention.py:455), or, with window_size > 0, only the
 *   keys >= position - window_size (:429-431,457-458); logit_softcapping > 0 replaces the
 *   scaled logits by cap * tanh(logits / cap) (:450-453).  Pass <= 0 to disable either.
 *   max_q_len >= max(q_len) sizes the grid.
 * Supported: dtype bf16/f16, D and Dv any multiples of 8 up to 256 (as for the decode entry
 * point), any page size >= 1, sm_scale > 0, q/k/v strides multiples of 8 and bases 16-byte
 * aligned, o strides multiples of 4 and base 8-byte aligned.
 * ---------------------------------------------------------------------------------------- */
int dlb_paged_prefill_attn(const void* q, const void* k_cache, const void* v_cache, void* o,
                           const void* block_table, const void* q_start_loc, const void* q_len,
                           const void* kv_len, int index64_mask, int B, int Hq, int Hkv,
                           int D, int Dv, int page, int max_blocks, int max_q_len,
                           int64_t q_stride_tok,
                           int64_t q_stride_head, int64_t k_stride_page, int64_t k_stride_tok,
                           int64_t k_stride_head, int64_t v_stride_page, int64_t v_stride_tok,
                           int64_t v_stride_head, int64_t o_stride_tok, int64_t o_stride_head,
                           int64_t bt_stride, float sm_scale, int window_size,
                           float logit_softcapping, int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * fp8 fused-MoE building blocks (OCP e4m3fn, fp32 scales per 128 along K; weights carry one
 * scale per 128 x 128 block).  Pipeline shape follows fused_moe, kernels/fused_moe.py:296-376
 * (grouped GEMM kernel :82-175); the fp8 scheme has no reference counterpart -- nearest
 * precedent: per-token int8 quant and scale-in-epilogue GEMM, kernels/w8a8.py:102-106,275-335.
 *
 * Quantisation rule (activations and the intermediate): for each group of 128 consecutive
 * elements of a row, scale = max(absmax, 1e-10) / 448 and q = rne_e4m3(clamp(x / scale, +-448)).
 * ---------------------------------------------------------------------------------------- */

/* x [M, K] bf16/f16 (row stride ld_x) -> xq [M, K] fp8 (row stride ld_q, bytes),
 * xs [M, K/128] fp32 (row stride ld_s).  K % 128 == 0. */
int dlb_per_token_group_quant_fp8(const void* x, void* xq, float* xs, int64_t M, int K,
                                  int64_t ld_x, int64_t ld_q, int64_t ld_s, int dtype,
                                  void* stream);

/* gate_up grouped GEMM + SiLU-and-mul + re-quantisation.
 *   xq [num_tokens, H] fp8, xs [num_tokens, H/128]
 *   w1q [num_local_experts, 2I, H] fp8 (gate rows first), w1s [num_local_experts, 2I/128, H/128]
 *   sorted_ids [num_mblocks * block_m] and expert_counts [num_experts]: the sorted slot list and
 *     the per-expert counts written by dlb_moe_align_block_size with block = block_m over all
 *     num_experts (global) experts; block_m in {64, 128} = rows per workgroup tile; flat slot =
 *     token * topk + j, sentinel num_tokens * topk.  num_mblocks = whole blocks sorted_ids
 *     holds (it has at least num_mblocks * block_m entries; floor(sorted_cap / block_m) of the
 *     alignment call is always >= sum over experts of ceil(count / block_m), the blocks in use;
 *     a workgroup whose block index is not below num_mblocks touches nothing).  Expert e's
 *     blocks start at block
 *     sum_{e' < e} ceil(count[e'] / block_m); blocks of experts outside
 *     [expert_offset, expert_offset + num_local_experts) are skipped.  num_experts <= 256.
 *   hq [num_mblocks * block_m, I] fp8 and hs [num_mblocks * block_m, I/128]: row r holds
 *     quant(silu(x_t W_gate^T) * (x_t W_up^T)) for the slot at sorted position r (rows of
 *     32-row groups that hold padding only are not written)
 * H % 128 == 0, I % 128 == 0, and the reduction length (H here, I in the down GEMM) at most
 * 16384.  Scales must be positive: activation scales below 1e-13 count as 1e-13 (the quantisation
 * rule above never produces less than 1e-10 / 448) and weight block scales below 1e-12 count as
 * 1e-12 (an all-zero block may carry the scale 0).
 * One kernel serves both tile heights and both weight layouts: four-wave tiles of block_m rows
 * x 256 columns, weights streamed straight into operand registers, activations staged in LDS.
 * Outputs are stored 16 bytes at a time: hq, out and the 16-bit act must be 16-byte aligned;
 * other alignments return DLB_ERR_UNSUPPORTED.
 * w_layout selects how the fp8 weight bytes of both GEMMs are stored:
 *   0  row-major [E, N, K] (the reference's w1/w2 layout);
 *   1  MFMA-operand order, a one-time re-arrangement done when the weights are loaded: for
 *      expert e, 16-row tile nb and 128-byte K chunk kc, a 2 KB block at
 *      ((e * N/16 + nb) * K/128 + kc) * 2048 holding [half h][lane l][16 bytes] =
 *      W[e][16 nb + l % 16][128 kc + 64 h + 16 (l / 16) .. + 16].  Same bytes, same scales;
 *      every operand load becomes one contiguous 1 KB access. */
int dlb_moe_gemm_fp8_gate_up(const void* xq, const float* xs, const void* w1q, const float* w1s,
                             const int32_t* sorted_ids, const int32_t* expert_counts,
                             int num_experts, int num_mblocks, int block_m, int num_tokens,
                             int topk, int H, int I, int expert_offset, int num_local_experts,
                             int w_layout, void* hq, float* hs, void* stream);

/* down grouped GEMM: out[slot, :] = (h_r W_down^T) * topk_weights[slot] for every real slot
 * (pad rows are skipped), out [num_tokens * topk, H] bf16/f16;
 * w2q [num_local_experts, H, I] fp8, w2s [num_local_experts, H/128, I/128].  H is the output
 * width of this GEMM (the reference takes it from w2.shape[1], kernels/fused_moe.py:354-357): it
 * need not equal the H of the gate_up call. */
int dlb_moe_gemm_fp8_down(const void* hq, const float* hs, const void* w2q, const float* w2s,
                          const int32_t* sorted_ids, const int32_t* expert_counts,
                          int num_experts, const float* topk_weights, int num_mblocks,
                          int block_m, int num_tokens, int topk, int H, int I, int expert_offset,
                          int num_local_experts, int w_layout, void* out, int out_dtype,
                          void* stream);

/* out[t, :] = sum_j in[t * topk + j, :] (fp32 accumulation in slot order, one rounding);
 * replaces intermediate_cache2.sum(dim=1), kernels/fused_moe.py:375.  N % 8 == 0. */
int dlb_moe_topk_sum(const void* in, void* out, int64_t num_tokens, int topk, int64_t N,
                     int dtype, void* stream);

/* ------------------------------------------------------------------------------------------
 * Unquantised (bf16/f16) fused MoE: the reference's own fused_moe pipeline,
 * kernels/fused_moe.py:82-235 (grouped GEMM kernel + launcher) and :334-373 (the two calls).
 * Same routing inputs (sorted_ids, expert_counts), tile height and weight layouts as the fp8 GEMMs above (w_layout 1 is
 * the same byte re-arrangement applied to the 2-byte elements: 128-byte chunks = 64 elements).
 *   gate_up: act[r, :] = round(silu(round(x_t W_gate^T)) * round(x_t W_up^T)) for the slot at
 *            sorted position r -- the rounding points of the reference (GEMM result stored in
 *            the activation dtype, then F.silu(...) * up, :351-352); act [num_mblocks*block_m, I]
 *   down:    out[slot, :] = round((act_r W_down^T) * topk_weights[slot]), out [T * topk, H]
 * x [T, H], w1 [E_local, 2I, H], w2 [E_local, H, I], all of `dtype`; the hidden size of the
 * gate_up call and I multiples of 64 (whole 128-byte chunks; the reference masks any size,
 * kernels/fused_moe.py:119-160), the output width of the down call a multiple of 8.
 * Follow with dlb_moe_topk_sum.
 * ---------------------------------------------------------------------------------------- */
int dlb_moe_gemm_16bit_gate_up(const void* x, const void* w1, const int32_t* sorted_ids,
                               const int32_t* expert_counts, int num_experts, int num_mblocks,
                               int block_m, int num_tokens, int topk, int H, int I,
                               int expert_offset, int num_local_experts, int w_layout, void* act,
                               int dtype, void* stream);
int dlb_moe_gemm_16bit_down(const void* act, const void* w2, const int32_t* sorted_ids,
                            const int32_t* expert_counts, int num_experts,
                            const float* topk_weights, int num_mblocks, int block_m,
                            int num_tokens, int topk, int H, int I, int expert_offset,
                            int num_local_experts, int w_layout, void* out, int dtype,
                            void* stream);

/* The reference's grouped-GEMM launcher in its own argument form: replaces fused_moe_kernel +
 * fused_moe_kernel_launcher, kernels/fused_moe.py:82-235 (16-bit operands, fp32 accumulation).
 *   a [a_rows, K], b [num_local_experts, N, K] (row-major), c [rows, N], all of `dtype`
 *   sorted_idx [num_slots]: the flat routing slots (token * topk + j) sorted by expert, NOT padded
 *   exp_start / exp_end [num_experts]: expert e owns sorted positions exp_start[e] .. exp_end[e] - 1
 *     (:267-293); local expert i is global expert expert_offset + i (:113-114)
 *   the three index arrays are int32 or int64 (index64_mask bit 0 = sorted_idx, 1 = exp_start,
 *   2 = exp_end; the reference passes the int64 result of argsort)
 *   for sorted position p with slot s = sorted_idx[p] of expert e:
 *     c[reindex_c ? s : p, :] = (a[reindex_a ? s / topk : p, :] . b[e]^T) * (weights ? weights[s] : 1)
 *   rounded once to `dtype` (:119-175); rows of c that no slot maps to are not written.
 * K % 64 == 0 (whole 128-byte chunks), N % 8 == 0, 16-byte aligned pointers, num_experts <= 256. */
int dlb_moe_gemm_16bit_launcher(const void* a, const void* b, void* c, const void* sorted_idx,
                                const void* exp_start, const void* exp_end, int index64_mask,
                                const float* weights, int num_experts, int expert_offset,
                                int num_local_experts, int64_t num_slots, int64_t a_rows, int topk,
                                int N, int K, int reindex_a, int reindex_c, int dtype,
                                void* stream);

/* ------------------------------------------------------------------------------------------
 * Decoder-layer helpers around the attention / MoE kernels (memory-bound).
 * ---------------------------------------------------------------------------------------- */

/* fill_kv_cache: scatter the new K/V tokens of each sequence into the paged cache.
 * Replaces fill_kv_cache + _fill_kv_cache_kernel, kernels/fill_kv_cache.py:23-185.
 *   k_states/v_states [num_tokens, heads, head_dim(_v)]  (token / head strides, unit last)
 *   k_cache/v_cache   [pages, page, heads, head_dim(_v)] (page / slot / head strides)
 *   sequence b owns tokens q_start_loc[b] .. + q_seq_len[b]; its i-th new token lands at
 *   context position kv_seq_len[b] - q_seq_len[b] + i, i.e. page
 *   block_table[b][pos / page], slot pos % page.  Tokens outside every sequence are ignored.
 *   The four index arrays are int32 or int64 (index64_mask bit 0 = q_start_loc, 1 = q_seq_len,
 *   2 = kv_seq_len, 3 = block_table).
 * elem_size = bytes per element (the copy is type-agnostic); strides in elements. */
int dlb_fill_kv_cache(const void* k_states, const void* v_states, void* k_cache, void* v_cache,
                      const void* q_start_loc, const void* q_seq_len, const void* kv_seq_len,
                      const void* block_table, int index64_mask, int64_t num_tokens, int batch, int heads, int head_dim, int head_dim_v, int page, int max_blocks,
                      int elem_size, int64_t ks_stride_tok, int64_t ks_stride_head,
                      int64_t vs_stride_tok, int64_t vs_stride_head, int64_t kc_stride_page,
                      int64_t kc_stride_slot, int64_t kc_stride_head, int64_t vc_stride_page,
                      int64_t vc_stride_slot, int64_t vc_stride_head, int64_t bt_stride,
                      void* stream);

/* rms_norm: out = weight * round(x * rsqrt(mean(x^2) + eps)); with `residual` != NULL the
 * input is first replaced by round(x + residual), which is also written to out_residual.
 * Replaces rms_norm / add_rms_norm, kernels/rms_norm.py:8-133 and kernels/add_rms_norm.py:9-80.
 * x/out/residual/out_residual [M, N] with row strides, weight [N]; bf16/f16 or f32 (nothing is
 * rounded on the way).  Any N >= 1: rows of whole 16-byte vectors (N % 8 == 0, f32 N % 4 == 0) up
 * to 16384 elements with 16-byte aligned pointers and strides stay in registers between the sum of
 * squares and the scaling; every other row length or alignment runs an element-wise kernel that
 * reads the row twice (the reference masks the tail, kernels/rms_norm.py:8-75). */
int dlb_rms_norm(const void* x, const void* weight, const void* residual, void* out,
                 void* out_residual, int64_t M, int N, int64_t ld_x, int64_t ld_res,
                 int64_t ld_out, int64_t ld_out_res, float eps, int dtype, void* stream);

/* apply_rotary_pos_emb: out = x * cos + rotate_half(x) * sin on q [T, Hq, D] and k [T, Hk, D],
 * cos/sin [T, D] (row stride cs_stride_tok); outputs may alias the inputs.
 * Replaces apply_rotary_pos_emb, kernels/apply_rotary_pos_emb.py:8-164.  bf16/f16/f32, any even
 * D; 16-byte vectors are moved when D % 16 == 0 (f32: D % 8 == 0) and pointers and strides are
 * multiples of a 16-byte vector, single elements otherwise. */
int dlb_apply_rotary_pos_emb(const void* q, const void* k, const void* cos, const void* sin,
                             void* q_out, void* k_out, int64_t num_tokens, int Hq, int Hk, int D,
                             int64_t q_stride_tok, int64_t q_stride_head, int64_t k_stride_tok,
                             int64_t k_stride_head, int64_t qo_stride_tok, int64_t qo_stride_head,
                             int64_t ko_stride_tok, int64_t ko_stride_head, int64_t cs_stride_tok,
                             int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DLBLAS_HIP_H_ */
