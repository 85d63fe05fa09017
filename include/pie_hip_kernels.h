/*
 * pie_hip_kernels.h — C ABI of the gfx950 (MI355X) kernel library behind the
 * Pie driver forward pass.
 *
 * Every entry point takes plain device pointers, shapes and a HIP stream
 * (passed as `void*`, i.e. a `hipStream_t`; NULL = the default stream), does no
 * allocation, keeps no global state, never throws, and returns a status code.
 * The functions replace, one for one, the `launch_*` C++ launchers of the
 * reference CUDA driver (the .hpp files under driver/cuda/src/kernels and driver/cuda/src/ops);
 * each declaration cites the launcher whose contract it follows.
 *
 * Conventions
 *   - bf16 tensors are raw 16-bit words (`uint16_t`), row-major.
 *   - "act x W" products follow the reference: act[M,K] · W[N,K]^T -> y[M,N]
 *     (driver/cuda/src/ops/gemm.hpp:152-160).
 *   - `beta` is 0 (overwrite y) or 1 (y += result, the residual fuse of
 *     driver/cuda/src/model/llama_like.cpp:626-628).
 */
#ifndef PIE_HIP_KERNELS_H
#define PIE_HIP_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* RoPE pairings of the rotation kernels and fused epilogues */
#define PIE_HIP_ROPE_HALF 0
#define PIE_HIP_ROPE_ADJACENT 1
#define PIE_HIP_ROPE_HALF_PAIRED_ROWS 2

#define PIE_HIP_OK 0
#define PIE_HIP_ERR_INVALID 1     /* null pointer, non-positive size, bad enum   */
#define PIE_HIP_ERR_UNSUPPORTED 2 /* shape the kernels do not cover              */
#define PIE_HIP_ERR_LAUNCH 3      /* HIP reported an error at launch             */

/* Library/ABI version: bumped on any change of a signature or of a memory layout an entry point
 * reads or writes.  A caller compares the macro it was built against with what the loaded
 * library returns and refuses to run on a mismatch (an old caller would link and compute
 * garbage).  History:
 *   1  first layout
 *   2  `pairing` argument of pie_hip_qkv_rope_fused / pie_hip_qkv_rope_skinny_tiled; `page_size`
 *      argument of pie_hip_kv_write_quant / pie_hip_qkv_rope_kvwrite_quant; KV scale pools
 *      [pages, hk, page_size] (were [pages, page_size, hk]); int4 tile-major weights in decode
 *      order (pie_hip_repack_mfma_tiles_int4); pie_hip_gemv_time_next removed
 *   3  current */
#define PIE_HIP_ABI_VERSION 3
int pie_hip_abi_version(void);

/* ---- W4A16 ("int4b8", symmetric, group-quantised) ------------------------- */

/*
 * Integer unpack test hook: q[n, k] = ((packed[n, k/8] >> (4*(k%8))) & 0xF) - 8
 * as int8.  Bit-exact statement of the nibble order used everywhere else.
 * Reference: driver/cuda/src/kernels/dequant_wna16.cu:31-36.
 */
int pie_hip_unpack_w4(const uint32_t* packed, int8_t* q, int out_dim, int in_dim,
                      void* stream);

/*
 * w[n, k] = bf16( float(nibble - 8) * float(scale[n, k / group_size]) ).
 * packed: [out_dim, in_dim/8] u32, scale: [out_dim, in_dim/group_size] bf16,
 * out: [out_dim, in_dim] bf16.
 * Reference: launch_dequant_wna16_int4b8_to_bf16,
 * driver/cuda/src/kernels/dequant_wna16.hpp:16-23, dequant_wna16.cu:11-38.
 */
int pie_hip_dequant_w4a16(const uint32_t* packed, const uint16_t* scale_bf16,
                          uint16_t* out_bf16, int out_dim, int in_dim, int group_size,
                          void* stream);

/*
 * Weight-only int4 GEMV/skinny GEMM for decode:
 *   y[m, n] = bf16( beta*y[m, n] + sum_k act[m, k] * (nibble(n, k) - 8) * scale[n, k/G] )
 * with fp32 accumulation; the group scale is applied to each group's partial
 * sum (same value as the reference's per-element `x * (q * s)` up to fp32
 * rounding, driver/cuda/src/kernels/dequant_wna16.cu:96-110).
 * Requires K % 32 == 0, G % 32 == 0, K % G == 0.  Tuned for decode (small M): up to four
 * activation rows share one pass over the weights, larger M re-streams them per group of four.
 * Replaces the Marlin call `marlin_w4a16_gemm` for small M
 * (driver/cuda/third_party/marlin/marlin_wrapper.hpp:39-51) and the
 * dequant-then-GEMM fallback of gemm_act_x_w (driver/cuda/src/ops/gemm.cpp:1414-1583).
 */
int pie_hip_gemv_w4a16(const uint16_t* act_bf16, const uint32_t* packed,
                       const uint16_t* scale_bf16, uint16_t* y_bf16, int M, int N, int K,
                       int group_size, int beta, void* stream);
/* Same contract with explicit tiling (rows walked per wave step, resident waves per SIMD;
 * 0 = library default).  For tuning sweeps; no reference counterpart. */
int pie_hip_gemv_w4a16_tuned(const uint16_t* act_bf16, const uint32_t* packed,
                             const uint16_t* scale_bf16, uint16_t* y_bf16, int M, int N, int K,
                             int group_size, int beta, int rows_per_wave, int waves_per_simd,
                             void* stream);

/*
 * The decoder layer's fused projection: y = epilogue( rmsnorm?(act) · W^T ) in one kernel.
 *   norm_weight_bf16 != NULL: act is replaced, while it is staged, by
 *     bf16(act * rsqrt(mean(act^2) + eps) * norm_weight) — value and rounding of the separate
 *     RMSNorm kernel (driver/cuda/src/kernels/rmsnorm.cu:14-54), so results do not change;
 *   swiglu != 0: W's rows are interleaved (gate_0, up_0, gate_1, up_1, ...) and
 *     y[m, i] = bf16( silu(bf16(g_i)) * bf16(u_i) ), y is [M, N/2] — the values of the unfused
 *     projection followed by swiglu_bf16_kernel (driver/cuda/src/kernels/swiglu.cu:9-22);
 *     not combinable with beta.
 * format: PIE_HIP_FMT_*; scale: int4b8 bf16 [N, K/G]; int8/fp8 row scale [N] (f32, or bf16
 * when scale_is_bf16); bf16: NULL.  Other arguments as the per-format GEMV entry points.
 * Replaces the rmsnorm -> gemm_act_x_w (-> swiglu) sequences of
 * driver/cuda/src/model/llama_like.cpp:370-705.
 */
#define PIE_HIP_FMT_INT4B8 0
#define PIE_HIP_FMT_INT8 1
#define PIE_HIP_FMT_FP8 2
#define PIE_HIP_FMT_BF16 3
int pie_hip_linear_fused(int format, const uint16_t* act_bf16, const uint16_t* norm_weight_bf16,
                         float eps, const void* weight, const void* scale, int scale_is_bf16,
                         int group_size, uint16_t* y_bf16, int M, int N, int K, int beta,
                         int swiglu, void* stream);

/*
 * The attention output projection of a decode step with the attention's split merge in its
 * prologue: y[m, :] = bf16( (beta ? y[m, :] : 0) + o[m, :] . W^T ), where o[m, :] (K = num_q_heads *
 * head_dim values) is the merged, normalised, bf16-rounded attention output of row m — computed
 * from the partial results pie_hip_attn_rows_paged_partials left in attn_workspace with the
 * operations of the separate merge launch in the same order, so y is bit-identical to
 * pie_hip_attn_rows_paged followed by pie_hip_linear_fused.  One launch less per layer: the merge
 * hides behind the projection's first weight requests.  num_splits / units_per_split: the plan
 * pie_hip_attn_decode_plan gave for the same (num_rows = M, num_kv_heads, max_kv_len).  Takes one
 * row with up to eight splits or two rows with up to four, K <= 4096, head_dim a power of two;
 * otherwise PIE_HIP_ERR_UNSUPPORTED (then run pie_hip_attn_rows_paged and pie_hip_linear_fused).
 * Reference: the split-KV merge of the decode attention (attention_flashinfer.hpp:17-24 plans it,
 * the library merges) followed by the o_proj gemm of driver/cuda/src/model/llama_like.cpp:370-705.
 */
int pie_hip_linear_attn_merge_supported(int format, int M, int num_splits, int num_q_heads, int head_dim,
                                        int group_size);   /* 1: taken, 0: PIE_HIP_ERR_UNSUPPORTED */
int pie_hip_linear_attn_merge(int format, const void* attn_workspace, int num_splits, int units_per_split,
                              const int32_t* row_kv_len, int num_q_heads, int head_dim, const void* weight,
                              const void* scale, int scale_is_bf16, int group_size, uint16_t* y_bf16, int M,
                              int N, int beta, void* stream);

/*
 * The fused q|k|v projection of a decode step with RoPE and the KV-cache write in its epilogue:
 * rows of W are the q, k and v heads ([(hq + 2 hk) * d, K]); adjacent output pairs (2i, 2i+1)
 * of every q and k head are rotated by rope_table[m] (interleaved pairing,
 * driver/cuda/src/kernels/rope.cu:14-33), q goes to q_out [M, hq*d], k and v to slot
 * kv_slots[m] of the paged pools (NHD addressing, driver/cuda/src/kernels/split_packed.cu:116-138).
 * Values are those of pie_hip_linear_fused followed by pie_hip_qkv_rope_kvwrite with
 * interleaved = pairing and no q/k norm (every intermediate rounded to bf16 at the same points).
 * pairing = PIE_HIP_ROPE_ADJACENT: as described.  pairing = PIE_HIP_ROPE_HALF_PAIRED_ROWS: the
 * half-split pairing of Llama / Qwen checkpoints (i, i + d/2; driver/cuda/src/kernels/rope.cu:10-21)
 * over weights whose q / k rows were re-ordered at load so that rows (2i, 2i+1) of a head are
 * that pair; the rotated values are written to positions i and i + d/2, so q_out and the pools
 * hold what the unpermuted projection followed by half-split RoPE gives, bit for bit.
 * Replaces the qkv gemm + qkv_decode_qk_norm_rope_write_kv_kernel pair of
 * driver/cuda/src/model/llama_like.cpp:370-470 for llama-type decode.  head_dim a power of two,
 * M <= 4 per weight pass like the GEMV.
 */
int pie_hip_qkv_rope_fused(int format, const uint16_t* act_bf16, const uint16_t* norm_weight_bf16,
                           float eps, const void* weight, const void* scale, int scale_is_bf16,
                           int group_size, int M, int K, const float* rope_table,
                           const int64_t* kv_slots, uint16_t* q_out, uint16_t* k_pages,
                           uint16_t* v_pages, int num_q_heads, int num_kv_heads, int head_dim,
                           int pairing, void* stream);

/*
 * lm_head for greedy decode rows: logits[m, v] = bf16( rmsnorm?(act[m]) . W[v] ) for the bf16
 * matrix W [V, H], and out_tokens[m] = argmax_v logits[m, v] over the bf16 values (the lowest
 * index among equals, NaN never wins, an all -inf row gives 0) — pie_hip_linear_fused followed by
 * pie_hip_argmax, bit for bit, in two launches that read the logits row only once: the GEMV
 * keeps per-lane (largest value, row) pairs while it stores, a one-block-per-row kernel reduces
 * them.  M <= 4 (one pass over the weights); workspace of
 * pie_hip_lm_head_argmax_workspace_bytes(M, V) bytes, need not be cleared.
 * Reference: lm_head_gemv_argmax_bf16 / _int8 (partial (value, index) pairs per block, then a
 * reduce), driver/cuda/src/kernels/argmax.cu:795-935.
 */
size_t pie_hip_lm_head_argmax_workspace_bytes(int M, int V);
int pie_hip_lm_head_argmax(const uint16_t* act_bf16, const uint16_t* norm_weight_bf16, float eps,
                           const uint16_t* w_bf16, uint16_t* logits_bf16, uint32_t* out_tokens, int M,
                           int V, int H, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Weight-only GEMM for a handful to a few dozen activation rows on the matrix cores:
 *   y[m, n] = epilogue( sum_k act[m,k] * w(n,k) ), same formats, scales, beta and swiglu
 * contracts as pie_hip_linear_fused (no fused norm); the weights are streamed once per 16
 * activation rows instead of once per 4.  bf16 products, fp32 accumulation; int4/int8 weights
 * enter the MFMA offset-binary (128+nibble / 128+byte, exact in bf16) and the offset is removed
 * per group / per row in fp32, so the result differs from the GEMV only by fp32 summation order.
 * Requirements (else PIE_HIP_ERR_UNSUPPORTED): K % 512 == 0 and group_size = 128 * 2^i dividing
 * K (int4b8); K % 256 == 0 (int8, fp8); K % 128 == 0 (bf16).
 * Replaces Marlin W4A16 for small/medium M (driver/cuda/third_party/marlin/marlin_wrapper.hpp:39-51)
 * and the cuBLASLt small-M path of gemm_act_x_w (driver/cuda/src/ops/gemm.cpp:1414-1583).
 */
int pie_hip_gemm_skinny(int format, const uint16_t* act_bf16, const void* weight,
                        const void* scale, int scale_is_bf16, int group_size, uint16_t* y_bf16,
                        int M, int N, int K, int beta, int swiglu, void* stream);

/*
 * Tiled weight-only GEMM on the matrix cores for prefill and large batches (compute-bound M):
 *   y[M, N] = epilogue( act[M, K] · W[N, K]^T ), formats / scales / beta / swiglu as above.
 * Evaluation order of the reference's large-M paths: the weights become bf16 first — int4b8 as
 * bf16((nibble-8) * group_scale), the value of launch_dequant_wna16_int4b8_to_bf16
 * (driver/cuda/src/kernels/dequant_wna16.cu:11-38) followed by a bf16 GEMM
 * (driver/cuda/src/ops/gemm.cpp:1213-1236); int8 / fp8 values are exact in bf16 and their row
 * scale multiplies the fp32 sum — then bf16 x bf16 products, fp32 accumulation, one rounding.
 * 128 x 128 x 64 tiles (64 x 128 for M <= 64, 256 x 128 for bf16 weights at large M),
 * v_mfma_f32_16x16x32_bf16.  Requirements: K % 64 == 0; int4b8
 * group_size a power of two >= 32 dividing K.
 */
int pie_hip_gemm_mfma(int format, const uint16_t* act_bf16, const void* weight, const void* scale,
                      int scale_is_bf16, int group_size, uint16_t* y_bf16, int M, int N, int K,
                      int beta, int swiglu, void* stream);

/*
 * The same GEMM for a decode batch (M <= 128 rows), where the output has too few 128-column
 * tiles to fill the machine: K is split into shares, one block per (tile, share), fp32 partial
 * sums go to `workspace` and a second kernel adds them and applies beta / swiglu.  Same
 * evaluation order per share; the shares are added in fp32 in ascending K.
 * pie_hip_gemm_mfma_workspace_bytes(M, N, K) is the workspace this shape needs (0: the shape is
 * not split and the call is pie_hip_gemm_mfma).  Role in the reference: cuBLASLt's split-K
 * heuristics inside gemm_act_x_w for small M (driver/cuda/src/ops/gemm.cpp:1414-1583).
 */
size_t pie_hip_gemm_mfma_workspace_bytes(int M, int N, int K);
int pie_hip_gemm_mfma_splitk(int format, const uint16_t* act_bf16, const void* weight,
                             const void* scale, int scale_is_bf16, int group_size,
                             uint16_t* y_bf16, int M, int N, int K, int beta, int swiglu,
                             void* workspace, size_t workspace_bytes, void* stream);

/*
 * MoE grouped weight-only GEMM: one skinny problem per expert in a single launch.
 *   rows [expert_offsets[e], expert_offsets[e+1]) of y (routes sorted by expert) are
 *   act[route_act_rows[r]] (or act[r] when route_act_rows is NULL) times expert e's [N,K]
 *   weights at weights + e*weight_stride_bytes (scales at scales + e*scale_stride_bytes).
 * Experts without routes cost nothing and their weights are never read; an expert's weights
 * are read once per 16 routes that hit it.  max_rows_per_expert is a hint (> 0) of the largest
 * per-expert row count.  With swiglu the weight rows are interleaved (gate_0, up_0, ...) and y
 * is [routes, N/2].  Same K requirements as pie_hip_gemm_skinny.
 * Replaces the per-route MoE decode GEMVs (driver/cuda/src/kernels/dequant_wna16.cu:59-169)
 * and the grouped GEMM of driver/cuda/src/ops/gemm.hpp:189-198.
 */
int pie_hip_moe_grouped_gemm(int format, const uint16_t* act_bf16, const int32_t* route_act_rows,
                             const int32_t* expert_offsets, int num_experts,
                             int max_rows_per_expert, const void* weights,
                             size_t weight_stride_bytes, const void* scales,
                             size_t scale_stride_bytes, int scale_is_bf16, int group_size,
                             uint16_t* y_bf16, int N, int K, int swiglu, void* stream);

/*
 * Tile-major weight layout for the skinny and grouped GEMMs.  The 16 bytes that lane (j, q) of a
 * wave loads for the 16-row tile t and K block b — byte 64 b + 16 q of row 16 t + j in the
 * row-major [N, K] matrix — are stored at byte ((t * nb + b) * 64 + 16 q + j) * 16, nb =
 * row_bytes / 64, so every wave load is 1 KiB contiguous instead of 16 rows x 64 bytes (rows past
 * N are zero; dst holds ceil(N/16) * 16 * row_bytes bytes).  int4 group scales [N, groups] become
 * [tile][group][16 rows].  Built once at load; the values are those of the row-major entry
 * points.  int4b8 weights take pie_hip_repack_mfma_tiles_int4, which also re-orders the eight
 * codes of every 32-bit word (codes 2i and 2i + 1 to nibbles i and i + 4) so that the kernels'
 * decode yields them in k order; the other formats take pie_hip_repack_mfma_tiles.  Role in the
 * reference: Marlin's offline weight repack (driver/cuda/third_party/marlin/marlin_wrapper.hpp:39-51).
 */
int pie_hip_repack_mfma_tiles(const void* src, void* dst, int N, size_t row_bytes, void* stream);
int pie_hip_repack_mfma_tiles_int4(const void* src, void* dst, int N, size_t row_bytes, void* stream);
int pie_hip_repack_scale_tiles(const uint16_t* src, uint16_t* dst, int N, int groups, void* stream);
/* pie_hip_gemm_skinny / pie_hip_moe_grouped_gemm over weights (and int4 group scales) in that
 * layout; every other argument as there (expert strides in bytes of the tiled buffers). */
int pie_hip_gemm_skinny_tiled(int format, const uint16_t* act_bf16, const void* weight,
                        const void* scale, int scale_is_bf16, int group_size, uint16_t* y_bf16,
                        int M, int N, int K, int beta, int swiglu, void* stream);
/* pie_hip_qkv_rope_fused for more rows than the GEMV takes (a decode batch): the q|k|v projection
 * over tile-major weights with interleaved RoPE and the KV-cache write in its epilogue.  act_bf16
 * is the normalised activation [M, K]; values are those of pie_hip_gemm_skinny_tiled followed by
 * pie_hip_qkv_rope_kvwrite (interleaved = pairing, 1 or 2; no q/k norm), every intermediate rounded to bf16 at
 * the same points.  Same reference role: the qkv gemm + qkv_decode_qk_norm_rope_write_kv_kernel
 * pair of driver/cuda/src/model/llama_like.cpp:370-470.  head_dim a power of two, K % 256 == 0. */
int pie_hip_qkv_rope_skinny_tiled(int format, const uint16_t* act_bf16, const void* weight,
                                  const void* scale, int scale_is_bf16, int group_size, int M, int K,
                                  const float* rope_table, const int64_t* kv_slots, uint16_t* q_out,
                                  uint16_t* k_pages, uint16_t* v_pages, int num_q_heads,
                                  int num_kv_heads, int head_dim, int pairing, void* stream);
int pie_hip_moe_grouped_gemm_tiled(int format, const uint16_t* act_bf16, const int32_t* route_act_rows,
                             const int32_t* expert_offsets, int num_experts,
                             int max_rows_per_expert, const void* weights,
                             size_t weight_stride_bytes, const void* scales,
                             size_t scale_stride_bytes, int scale_is_bf16, int group_size,
                             uint16_t* y_bf16, int N, int K, int swiglu, void* stream);

/*
 * MoE routing: per token softmax over router_logits[t, 0..E) (bf16 in, fp32 inside), top_k by
 * repeated argmax with exclusion (ties to the lowest expert index), weights renormalised to
 * sum 1 — topk_softmax_bf16_kernel, driver/cuda/src/kernels/topk_softmax.cu:19-86 (graph form:
 * driver/portable/src/graph_common.cpp:262-283).  A second small kernel builds the grouped layout of
 * pie_hip_moe_grouped_gemm: routes (t, k) counting-sorted by expert.
 *   topk_idx [T, top_k] int32, topk_weight [T, top_k] f32 (bit-exact integer outputs given the
 *   probabilities; the order of routes inside one expert is unspecified),
 *   expert_offsets [E+1], route_token [T*top_k] (token of each sorted route),
 *   route_pos [T*top_k] (sorted position of route (t, k)).
 * num_experts <= 512, top_k <= 16 (the reference's bounds).
 * pie_hip_moe_route_opt: renormalize = 0 leaves the chosen experts' softmax probabilities undivided
 * (norm_topk = false: the graph form divides only under it, graph_common.cpp:279-283);
 * pie_hip_moe_route is renormalize = 1.
 */
int pie_hip_moe_route(const uint16_t* router_logits_bf16, int32_t* topk_idx, float* topk_weight,
                      int32_t* expert_offsets, int32_t* route_token, int32_t* route_pos,
                      int num_tokens, int num_experts, int top_k, void* stream);
int pie_hip_moe_route_opt(const uint16_t* router_logits_bf16, int32_t* topk_idx, float* topk_weight,
                      int32_t* expert_offsets, int32_t* route_token, int32_t* route_pos,
                      int num_tokens, int num_experts, int top_k, int renormalize, void* stream);

/*
 * A decode batch's way into the MoE block in two launches instead of four: per token the RMSNorm
 * of its hidden row (norm_out = what pie_hip_rmsnorm stores, bit for bit), the router logits
 * bf16(sum_k norm_out[t, k] * router[e, k]) over the bf16 router matrix [E, hidden] (fp32 sums in
 * this kernel's own order: they may differ from a GEMM's in the last bf16 bit), pie_hip_moe_route_opt's
 * softmax / top-k on them, then the expert-sorted layout.  router_logits may be NULL (not stored).
 * Each token's block reads the whole router matrix through the L2: meant for batches of up to a
 * few hundred rows.  hidden <= 8192, a multiple of 8; expert and top-k bounds as pie_hip_moe_route.
 * Replaces rmsnorm + router gemm + topk_softmax_bf16_kernel of the reference's MoE block
 * (driver/cuda/src/model/kimi_forward.cpp:640-700; graph form driver/portable/src/graph_common.cpp:237-283).
 */
int pie_hip_moe_norm_route(const uint16_t* x_bf16, const uint16_t* norm_weight_bf16, float eps,
                           const uint16_t* router_bf16, uint16_t* norm_out_bf16,
                           uint16_t* router_logits_bf16, int32_t* topk_idx, float* topk_weight,
                           int32_t* expert_offsets, int32_t* route_token, int32_t* route_pos,
                           int num_tokens, int hidden, int num_experts, int top_k, int renormalize,
                           void* stream);

/*
 * pie_hip_moe_combine with add = 1 followed by pie_hip_rmsnorm of the updated rows with the next
 * layer's norm weight, in one launch and with both results bit-identical to the two:
 * out[t, :] = bf16(out[t, :] + sum_k w[t, k] * y_routes[route_pos[t, k], :]),
 * norm_out[t, :] = rmsnorm(out[t, :]) * norm_weight.  hidden <= 8192, a multiple of 8.
 * Reference: token_batched_weighted_sum_add_bf16_kernel (driver/cuda/src/kernels/moe_dispatch.cu:152-196)
 * + rmsnorm_bf16_kernel (driver/cuda/src/kernels/rmsnorm.cu:14-54).
 */
int pie_hip_moe_combine_norm(const uint16_t* y_routes_bf16, const int32_t* route_pos,
                             const float* topk_weight, uint16_t* out_bf16,
                             const uint16_t* norm_weight_bf16, float eps, uint16_t* norm_out_bf16,
                             int num_tokens, int top_k, int hidden, void* stream);

/*
 * MoE combine: out[t, :] = bf16( (add ? out[t, :] : 0) + sum_k topk_weight[t, k] *
 * y_routes[route_pos[t, k], :] ), fp32 sum in top-k order, one rounding —
 * token_batched_weighted_sum[_add]_bf16_kernel, driver/cuda/src/kernels/moe_dispatch.cu:152-196.
 * hidden % 8 == 0.
 */
int pie_hip_moe_combine(const uint16_t* y_routes_bf16, const int32_t* route_pos,
                        const float* topk_weight, uint16_t* out_bf16, int num_tokens, int top_k,
                        int hidden, int add, void* stream);

/*
 * Prefill attention on the matrix cores: the result contract of pie_hip_attn_rows_paged for
 * query rows grouped into tiles.  Tile i covers rows tile_row_start[i] .. + tile_num_rows[i]
 * (consecutive rows that share one page list, i.e. row_page_begin is equal across the tile;
 * at most rows_per_tile rows, which is pie_hip_attn_prefill_tile_rows(hq, hk) = 128 / (hq/hk)
 * or half of it — the smaller tile doubles the number of blocks for small batches); each row
 * still sees its own first row_kv_len[row] keys.  Tiles may come in any order; blocks start in tile
 * order (the kv heads of a tile side by side), so listing the tiles with the longest key extents
 * first lets the short ones fill the slots that free up — on a causal prompt of more tiles than the
 * device holds at once that is worth 15-30 % (4096 tokens: 355 -> 278 us).  Probabilities are rounded to bf16 before they multiply V
 * (fp32 softmax sums and accumulators), so results agree with the per-row kernel to about one
 * bf16 step rather than bit for bit.  d in {64,128}, hq/hk in {1,2,4,8}, page_size % 16 == 0.
 * Reference: the causal prefill branch of launch_attention_naive_paged_prefill,
 * driver/cuda/src/ops/attention_naive_paged.cu:148-317; per-request flash attention of the
 * portable driver, driver/portable/src/graph_common.cpp:347-396.
 */
int pie_hip_attn_prefill_tile_rows(int num_q_heads, int num_kv_heads);
int pie_hip_attn_prefill_tiles(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                               uint16_t* o, const uint32_t* kv_page_indices,
                               const uint32_t* row_page_begin, const int32_t* row_kv_len,
                               const int32_t* tile_row_start, const int32_t* tile_num_rows,
                               int num_tiles, int rows_per_tile, int num_q_heads, int num_kv_heads,
                               int head_dim, int page_size, float sm_scale, void* stream);
/* The same over one-byte KV pools (kv_format / k_scales / v_scales as for
 * pie_hip_attn_rows_paged_kvq; PIE_HIP_KV_BF16 with null scales is pie_hip_attn_prefill_tiles):
 * codes are decoded exactly into the bf16 tiles, the K scale multiplies the score and the V
 * scale the rounded probability. */
int pie_hip_attn_prefill_tiles_kvq(int kv_format, const uint16_t* q, const void* k_pages,
                                   const void* v_pages, const float* k_scales, const float* v_scales,
                                   uint16_t* o, const uint32_t* kv_page_indices,
                                   const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                   const int32_t* tile_row_start, const int32_t* tile_num_rows,
                                   int num_tiles, int rows_per_tile, int num_q_heads, int num_kv_heads,
                                   int head_dim, int page_size, float sm_scale, void* stream);

/*
 * Custom attention masks for the per-row form.  pie_hip_attn_mask_bitmap turns per-row BRLE
 * runs into one u16 per 16-token unit (bit t = key 16*unit + t visible): run_bounds holds each
 * row's cumulative run ends, [run_bounds_indptr[r], run_bounds_indptr[r+1]); runs alternate
 * hidden / visible from key 0, keys past the last run are hidden, a row without runs sees its
 * whole window; no key at or past row_kv_len[r] (= the row's position + 1) is ever visible, and
 * window > 0 also hides keys below row_kv_len[r] - window
 * (build_attn_mask_f16, driver/portable/src/plan.cpp:54-94).  bitmap: [num_rows, stride_units],
 * stride_units >= ceil(max_kv_len / 16).
 * pie_hip_attn_rows_paged_masked is pie_hip_attn_rows_paged restricted to the visible keys; a
 * row with no visible key gives o = 0, lse = -inf.
 */
int pie_hip_attn_mask_bitmap(const uint32_t* run_bounds, const int32_t* run_bounds_indptr,
                             const int32_t* row_kv_len, int window, uint16_t* bitmap, int num_rows,
                             int stride_units, void* stream);
int pie_hip_attn_rows_paged_masked(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                                   uint16_t* o, float* lse, const uint32_t* kv_page_indices,
                                   const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                   const uint16_t* mask_bitmap, int mask_stride_units, int num_rows,
                                   int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                   float sm_scale, int max_kv_len, void* workspace,
                                   size_t workspace_bytes, void* stream);

/*
 * Sampling beyond greedy argmax, one slot = one sampled logits row.
 *
 * pie_hip_sample_gather_logits: out[s, :] = f32(logits[rows[s], :]) (rows == NULL: row s), with
 * slot s's BRLE logit mask applied: mask_bounds[mask_bounds_indptr[s] .. [s+1]) are the
 * cumulative ends of the slot's runs; run j (0-based) allows its tokens when j is odd, tokens
 * past the last run are masked (-inf), a slot with no runs is unconstrained
 * (apply_brle_logit_mask, driver/portable/src/sampler.cpp:169-198).
 *
 * pie_hip_sample: per slot, by `kind` (the wire order of the Sampler variants,
 * driver/bridge/include/pie_bridge/view.hpp:346-358):
 *   MULTINOMIAL / TOP_K / TOP_P / MIN_P / TOP_K_TOP_P -> tokens[s]
 *       (sample_token, driver/portable/src/sampler.cpp:345-409; uniform[s] is the draw the
 *       reference takes from its per-slot PCG32, made by the caller)
 *   DIST      -> ids / values [out_indptr[s], out_indptr[s+1]): the most probable tokens of
 *                softmax(logits / T), descending (run_distribution, :224-251); the range length
 *                is the caller's k (the whole vocabulary for k = 0)
 *   LOGPROB / LOGPROBS -> values[i] = log_softmax(logits)[labels[i]] over the slot's range
 *                (run_logprob / run_logprobs_many, :262-292); labels must be < vocab
 *   ENTROPY   -> values[out_indptr[s]] (run_entropy, :294-306)
 *   RAW_LOGITS -> nothing: the f32 row of pie_hip_sample_gather_logits is the payload
 * Equal probabilities are ordered by ascending token id.  Running sums are taken in double and
 * compared after rounding to float.  workspace: pie_hip_sample_workspace_bytes(S, vocab).
 */
enum {
    PIE_HIP_SAMPLER_MULTINOMIAL = 0, PIE_HIP_SAMPLER_TOP_K = 1, PIE_HIP_SAMPLER_TOP_P = 2,
    PIE_HIP_SAMPLER_MIN_P = 3, PIE_HIP_SAMPLER_TOP_K_TOP_P = 4,
    PIE_HIP_SAMPLER_EMBEDDING = 5,   /* a slot without output (the reference's executor emits nothing for it) */
    PIE_HIP_SAMPLER_DIST = 6,
    PIE_HIP_SAMPLER_RAW_LOGITS = 7, PIE_HIP_SAMPLER_LOGPROB = 8, PIE_HIP_SAMPLER_LOGPROBS = 9,
    PIE_HIP_SAMPLER_ENTROPY = 10
};
size_t pie_hip_sample_workspace_bytes(int num_slots, int vocab);
int pie_hip_sample_gather_logits(const uint16_t* logits_bf16, const int32_t* rows, float* out_f32,
                                 const uint32_t* mask_bounds, const int32_t* mask_bounds_indptr,
                                 int num_slots, int vocab, void* stream);
int pie_hip_sample(const float* logits_f32, const int32_t* kind, const float* temperature,
                   const uint32_t* top_k, const float* top_p, const float* min_p,
                   const float* uniform, const int32_t* out_indptr, const uint32_t* labels,
                   uint32_t* tokens, float* values, uint32_t* ids, void* workspace,
                   size_t workspace_bytes, int num_slots, int vocab, void* stream);

/* Measurement form of pie_hip_gemv_w4a16 (M <= 4: one kernel): that kernel is bracketed by the
 * caller's two HIP events (hipEvent_t), so hipEventElapsedTime(start, stop) is its own duration.
 * The events belong to this call only; the library keeps nothing.  No reference counterpart. */
int pie_hip_gemv_w4a16_timed(const uint16_t* act_bf16, const uint32_t* packed,
                             const uint16_t* scale_bf16, uint16_t* y_bf16, int M, int N, int K,
                             int group_size, int beta, void* start_event, void* stop_event,
                             void* stream);

/*
 * Weight-only int8 GEMV (W8A16), per-output-channel scale:
 *   y[m, n] = bf16( beta*y[m, n] + (sum_k f32(act[m,k]) * f32(q[n,k])) * scale_inv[n] )
 * fp32 sum, scale applied once after it — the evaluation order of the reference's own
 * weight-only int8 GEMV (driver/cuda/src/kernels/argmax.cu:846-854).  q: int8 [N,K];
 * scale_inv (= absmax/127, driver/cuda/src/kernels/quant_bf16_to_fp8.cu:311-313) is given
 * as f32 [N] or as bf16 [N]: pass exactly one of the two pointers.  K % 16 == 0.
 */
int pie_hip_gemv_w8a16(const uint16_t* act_bf16, const int8_t* w_int8,
                       const float* scale_inv_f32, const uint16_t* scale_inv_bf16,
                       uint16_t* y_bf16, int M, int N, int K, int beta, void* stream);

/*
 * Weight-only fp8 (OCP e4m3fn bytes) GEMV with per-output-channel scale, same shape rules
 * and scale arguments as the int8 entry point.  Format:
 * driver/cuda/src/kernels/dequant_fp8.cu:25-39 (w = fp8 * scale_inv[row]).
 */
int pie_hip_gemv_fp8(const uint16_t* act_bf16, const uint8_t* w_e4m3,
                     const float* scale_inv_f32, const uint16_t* scale_inv_bf16,
                     uint16_t* y_bf16, int M, int N, int K, int beta, void* stream);

/*
 * bf16 GEMV: y[m, n] = bf16( beta*y + sum_k act[m,k]*W[n,k] ), fp32 accumulation
 * (gemm_act_x_w bf16 path, driver/cuda/src/ops/gemm.hpp:152-160; the lm_head and router
 * projections stay unquantised in the reference).  K % 8 == 0.
 */
int pie_hip_gemv_bf16(const uint16_t* act_bf16, const uint16_t* w_bf16, uint16_t* y_bf16, int M,
                      int N, int K, int beta, void* stream);

/* ---- paged-KV decode attention -------------------------------------------- */

/*
 * One query token per request over a paged KV pool:
 *   o[r, h, :] = softmax_j( q[r,h,:]·K[j, kvh, :] * sm_scale ) · V[j, kvh, :],  kvh = h / (hq/hk)
 * for j over the request's context, kv_len = (pages-1)*page_size + last_page_len
 * (0 when the request lists no page; then o = 0 and lse = -inf).
 *   q, o          [R, hq, d] bf16
 *   k_pages/v_pages [num_pages, page_size, hk, d] bf16 (driver/cuda/src/kv_cache.hpp:3-8)
 *   kv_page_indices / kv_page_indptr[R+1] / kv_last_page_lens[R]: the wire arrays of
 *     the forward request, as the runtime sends them; requests may list the same
 *     physical pages (forked prefixes) — they are read in place.
 *   lse           optional [R, hq] f32, natural-log sum-exp of the scaled scores
 *   sm_scale      <= 0 selects 1/sqrt(d)
 *   max_kv_len    host-side upper bound on any request's kv_len (sizes the split grid)
 *   workspace     device scratch of pie_hip_attn_decode_workspace_bytes(...) bytes
 * fp32 maths, one bf16 rounding at the output.  d in {64,128}, hq/hk in {1,2,4,8},
 * page_size % 16 == 0.
 * Reference: launch_attention_naive_paged_decode,
 * driver/cuda/src/ops/attention_naive_paged.hpp:57-69, kernel attention_naive_paged.cu:319-447;
 * split-KV planning role of driver/cuda/src/ops/attention_flashinfer.hpp:17-24.
 */
size_t pie_hip_attn_decode_workspace_bytes(int num_requests, int num_q_heads, int num_kv_heads,
                                           int head_dim, int max_kv_len);
int pie_hip_attn_decode_paged(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                              uint16_t* o, float* lse, const uint32_t* kv_page_indices,
                              const uint32_t* kv_page_indptr, const uint32_t* kv_last_page_lens,
                              int num_requests, int num_q_heads, int num_kv_heads, int head_dim,
                              int page_size, float sm_scale, int max_kv_len, void* workspace,
                              size_t workspace_bytes, void* stream);

/*
 * Same attention over explicit per-row extents: query row r reads the page-list entries
 * starting at kv_page_indices[row_page_begin[r]] and sees its first row_kv_len[r] keys.  A
 * planner derives the pairs from the page table and the token positions
 * (visible keys = min(seq_len, position + 1), driver/portable/src/plan.cpp:54-94), so a
 * prefill or mixed batch runs as one row per query token, causal by construction, and a
 * decode batch as one row per request.  Workspace: pie_hip_attn_decode_workspace_bytes with
 * num_requests = num_rows.
 */
/* How a decode attention launch over (num_rows, num_kv_heads, max_kv_len) splits its rows:
 * units_per_split 16-token units per split, num_splits splits per row (1: no workspace, no merge). */
int pie_hip_attn_decode_plan(int num_rows, int num_kv_heads, int max_kv_len, int* units_per_split,
                             int* num_splits);
/* Whether a decode attention launch without custom masks over pools of kv_format takes the chunked
 * form instead of that grid of splits: as many blocks as the device holds at once, each with the same
 * share of the batch's keys (one wave per kv head, the rows' keys in 16-token units cut into equal
 * chunks), for one-byte pools when the grid would queue blocks behind one another.  The workspace
 * query covers both forms; results agree to the rounding of the fp32 merge.  Informational (tests,
 * profiles): 1 or 0. */
int pie_hip_attn_decode_is_chunked(int kv_format, int num_rows, int num_kv_heads, int max_kv_len);
/* pie_hip_attn_rows_paged (kv_format PIE_HIP_KV_BF16) / pie_hip_attn_rows_paged_kvq without the merge
 * launch: the splits' partial results stay in the workspace — [rows, q heads, splits, head_dim] f32
 * unnormalised outputs, then [rows, q heads, splits, 2] f32 (max, sum) in units of scale * log2(e);
 * slots of splits past a row's own extent are left unwritten — for pie_hip_linear_attn_merge.
 * PIE_HIP_ERR_INVALID when the plan has a single split (nothing to merge). */
int pie_hip_attn_rows_paged_partials(int kv_format, const uint16_t* q, const void* k_pages, const void* v_pages,
                                     const float* k_scales, const float* v_scales,
                                     const uint32_t* kv_page_indices, const uint32_t* row_page_begin,
                                     const int32_t* row_kv_len, int num_rows, int num_q_heads,
                                     int num_kv_heads, int head_dim, int page_size, float sm_scale,
                                     int max_kv_len, void* workspace, size_t workspace_bytes, void* stream);
int pie_hip_attn_rows_paged(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                            uint16_t* o, float* lse, const uint32_t* kv_page_indices,
                            const uint32_t* row_page_begin, const int32_t* row_kv_len,
                            int num_rows, int num_q_heads, int num_kv_heads, int head_dim,
                            int page_size, float sm_scale, int max_kv_len, void* workspace,
                            size_t workspace_bytes, void* stream);

/*
 * pie_hip_attn_rows_paged without a workspace argument and without any allocation, for callers
 * that cannot allocate device memory: code running under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The split partials
 * go to a device array built into the library, PIE_HIP_ATTN_STATIC_SCRATCH_BYTES per GPU, held
 * until the process ends; a batch whose partials
 * (pie_hip_attn_decode_workspace_bytes(num_rows, ...)) exceed it is refused with
 * PIE_HIP_ERR_UNSUPPORTED and a message on stderr.  Same kernels and results as
 * pie_hip_attn_rows_paged, bit for bit.  All calls on one GPU share that GPU's array: calls
 * that overlap on one GPU (different streams, or threads) race; serialise them.  The first call
 * on a device looks up the array's address (no allocation, but make it outside graph capture).
 */
#define PIE_HIP_ATTN_STATIC_SCRATCH_BYTES (16u << 20)
int pie_hip_attn_rows_paged_static(const uint16_t* q, const uint16_t* k_pages,
                                   const uint16_t* v_pages, uint16_t* o, float* lse,
                                   const uint32_t* kv_page_indices, const uint32_t* row_page_begin,
                                   const int32_t* row_kv_len, int num_rows, int num_q_heads,
                                   int num_kv_heads, int head_dim, int page_size, float sm_scale,
                                   int max_kv_len, void* stream);

/*
 * KV-cache storage formats of the pool (the CUDA driver's kv_cache_dtype values,
 * driver/cuda/src/kv_cache_format.cpp:46-110).  One-byte formats keep the bf16 layout
 * [pages, page_size, hk, d] with one byte per element; the per-token-head formats add fp32 side
 * scales [pages, hk, page_size] for K and for V (see pie_hip_kv_write_quant).  The 4-bit block format
 * ("fp4_e2m1" / "nvfp4": the same scheme under two names) packs two e2m1 codes per byte,
 * [pages, page_size, hk, d/2] with the even element in the low nibble, and keeps one fp32 scale
 * per block of 16 elements, [pages, hk, page_size, d/16]; the attention entry points do not read
 * it directly (PIE_HIP_ERR_UNSUPPORTED): as in the reference, the pages a batch reads are first
 * expanded into a bf16 pool by pie_hip_kv_dequant_pages.
 */
enum {
    PIE_HIP_KV_BF16 = 0,
    PIE_HIP_KV_FP8_E4M3 = 1,             /* saturating cast of the value, no scales */
    PIE_HIP_KV_INT8_PER_TOKEN_HEAD = 2,  /* scale = absmax/127, code = rint(x / scale) */
    PIE_HIP_KV_FP8_PER_TOKEN_HEAD = 3,   /* scale = absmax/448, code = e4m3(x / scale) */
    PIE_HIP_KV_FP8_E5M2 = 4,             /* saturating e5m2 cast of the value, no scales */
    PIE_HIP_KV_FP4_BLOCK = 5             /* per 16 elements: scale = absmax/6, code = nearest e2m1 level */
};

/*
 * pie_hip_attn_rows_paged over a pool in a one-byte format: every K / V element is
 * float(code) * scale as load_kv_scalar reads it (driver/cuda/src/ops/attention_naive_paged.cu:56-112),
 * everything else as for bf16 pools.  k_scales / v_scales: required for the per-token-head
 * formats, NULL for PIE_HIP_KV_FP8_E4M3 and PIE_HIP_KV_FP8_E5M2.  Custom masks are not available with these formats.
 */
int pie_hip_attn_rows_paged_kvq(int kv_format, const uint16_t* q, const void* k_pages,
                                const void* v_pages, const float* k_scales, const float* v_scales,
                                uint16_t* o, float* lse, const uint32_t* kv_page_indices,
                                const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                int num_rows, int num_q_heads, int num_kv_heads, int head_dim,
                                int page_size, float sm_scale, int max_kv_len, void* workspace,
                                size_t workspace_bytes, void* stream);
/* The same call (any kv_format, PIE_HIP_KV_BF16 with NULL scales included) for a batch whose rows
 * the caller knows to be about equally long, e.g. a decode batch whose longest context is within an
 * eighth of the mean: the launch then takes one round of resident blocks — for 64 rows of 8 kv
 * heads one block per (row, kv head), nothing to merge — where rows of unknown lengths get several
 * splits so that a long one does not run on alone.  Same results contract and workspace query;
 * a wrong hint costs time, not correctness.  Reference: the decode branch of
 * launch_attention_naive_paged, driver/cuda/src/ops/attention_naive_paged.cu:319-447 (one launch
 * per batch; the split plan is this library's). */
int pie_hip_attn_rows_paged_kvq_uniform(int kv_format, const uint16_t* q, const void* k_pages,
                                        const void* v_pages, const float* k_scales, const float* v_scales,
                                        uint16_t* o, float* lse, const uint32_t* kv_page_indices,
                                        const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                        int num_rows, int num_q_heads, int num_kv_heads, int head_dim,
                                        int page_size, float sm_scale, int max_kv_len, void* workspace,
                                        size_t workspace_bytes, void* stream);
/* The same over rows with custom attention masks: mask_bitmap as for
 * pie_hip_attn_rows_paged_masked (one visibility word per row and 16-token unit). */
int pie_hip_attn_rows_paged_kvq_masked(int kv_format, const uint16_t* q, const void* k_pages,
                                       const void* v_pages, const float* k_scales,
                                       const float* v_scales, uint16_t* o, float* lse,
                                       const uint32_t* kv_page_indices,
                                       const uint32_t* row_page_begin, const int32_t* row_kv_len,
                                       const uint16_t* mask_bitmap, int mask_stride_units,
                                       int num_rows, int num_q_heads, int num_kv_heads, int head_dim,
                                       int page_size, float sm_scale, int max_kv_len,
                                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * Quantising KV write: this step's K and V rows [num_tokens, hk, d] bf16 (after RoPE) go to
 * slot kv_slots[t] of a one-byte pool (slot < 0: skipped).  Per-token-head formats:
 * scale = absmax / qmax (qmax 127 / 448; 1 for an all-zero row), code = x * (1/scale) rounded
 * to nearest even, clamped / saturated; PIE_HIP_KV_FP8_E4M3 / _E5M2: the saturating cast of x
 * (largest finite value 448 / 57344).  The fp32 scale pools are laid out
 * [pages, kv heads, page_size] (the 16 scales an attention block reads for one page and head are
 * contiguous; a page's scales are one run, so page copies move them like the codes): the scale of
 * slot s and head h sits at ((s / page_size) * hk + h) * page_size + s % page_size.
 * Reference: write_kv_per_token_head_kernel and write_kv_fp8_per_tensor_kernel,
 * driver/cuda/src/kernels/kv_paged.cu:155-297.
 */
int pie_hip_kv_write_quant(int kv_format, const uint16_t* k_rows, const uint16_t* v_rows,
                           const int64_t* kv_slots, void* k_pages, void* v_pages, float* k_scales,
                           float* v_scales, int num_tokens, int num_kv_heads, int head_dim,
                           int page_size, void* stream);
/* PIE_HIP_KV_FP4_BLOCK in pie_hip_kv_write_quant: per block of 16 elements scale = absmax / 6
 * (1 for an all-zero block), code = the nearest of +-{0, .5, 1, 1.5, 2, 3, 4, 6} to x * (1/scale),
 * the smaller magnitude on a tie, sign bit for x < 0 (write_kv_fp4_block_kernel,
 * driver/cuda/src/kernels/kv_paged.cu:292-417); head_dim a multiple of 16.
 *
 * Expansion of the pages a batch reads into bf16 pools of the same geometry
 * [pages, page_size, hk, d] (page ids unchanged; other pages are not touched): every element
 * becomes bf16(float(code) * scale), for any of the one-byte formats and the 4-bit block format.
 * page_ids may name a page more than once.
 * Reference: launch_dequant_kv_cache_layer_to_bf16_active and the dequant_*_pages_active kernels,
 * driver/cuda/src/kernels/kv_paged.cu:419-531, :698-770. */
int pie_hip_kv_dequant_pages(int kv_format, const void* k_pages, const void* v_pages,
                             const float* k_scales, const float* v_scales, uint16_t* k_out,
                             uint16_t* v_out, const uint32_t* page_ids, int num_pages,
                             int num_kv_heads, int head_dim, int page_size, void* stream);
/* pie_hip_qkv_rope_kvwrite and pie_hip_kv_write_quant in one launch for one-byte pools: every
 * (token, head) of the packed q|k|v rows is rotated (optional per-head q/k RMSNorm, either
 * pairing) and rounded to bf16 as by pie_hip_qkv_rope_kvwrite; q goes to q_out, the K and V
 * heads are quantised from those bf16 values into the token's slot with the arithmetic of
 * pie_hip_kv_write_quant (driver/cuda/src/kernels/kv_paged.cu:155-297) — the same bytes and
 * scales as the two calls in a row.  head_dim <= 256. */
int pie_hip_qkv_rope_kvwrite_quant(int kv_format, const uint16_t* packed_qkv, uint16_t* q_out,
                                   void* k_pages, void* v_pages, float* k_scales, float* v_scales,
                                   const uint16_t* q_norm_weight, const uint16_t* k_norm_weight,
                                   const float* rope_table, const int64_t* kv_slots, int num_tokens,
                                   int num_q_heads, int num_kv_heads, int head_dim, int page_size,
                                   int interleaved, float eps, void* stream);

/* ---- per-layer kernels of the llama-like decoder ---------------------------- */

/* y[n,:] = table[token_ids[n],:]; ids >= vocab read row 0.
 * Reference: launch_embed_bf16, driver/cuda/src/kernels/embed.cu:8-23. */
int pie_hip_embed(const uint32_t* token_ids, const uint16_t* table_bf16, uint16_t* y_bf16,
                  int num_tokens, int hidden, int vocab, void* stream);

/* y = bf16( x * rsqrt(mean(x^2) + eps) * w ), fp32 inside.  hidden % 8 == 0.
 * Reference: rmsnorm_bf16_kernel, driver/cuda/src/kernels/rmsnorm.cu:14-54. */
int pie_hip_rmsnorm(const uint16_t* x_bf16, const uint16_t* weight_bf16, uint16_t* y_bf16,
                    int rows, int hidden, float eps, void* stream);

/* hidden = bf16(hidden + residual) (stored), norm_out = rmsnorm(hidden) of the rounded sum.
 * Reference: residual_add_rmsnorm_bf16_kernel, driver/cuda/src/kernels/rmsnorm.cu:56-98. */
int pie_hip_residual_rmsnorm(uint16_t* hidden_bf16, const uint16_t* residual_bf16,
                             const uint16_t* weight_bf16, uint16_t* norm_out_bf16, int rows,
                             int hidden, float eps, void* stream);

/* table[n, i] = cos(positions[n] * inv_freq[i]); table[n, i + d/2] = sin(same), i < d/2,
 * angle and sincos in fp32.  inv_freq[d/2] is a host table (theta^(-2i/d), optionally with
 * llama3 band scaling, driver/portable/src/model.cpp:1414-1448).
 * Reference: rope_standard_table_kernel, driver/cuda/src/kernels/rope.cu:35-53. */
int pie_hip_rope_table(const int32_t* positions, const float* inv_freq, float* table,
                       int num_tokens, int head_dim, void* stream);
/* The same with cos and sin multiplied by mscale (> 0): YaRN's attention factor
 * (rope_yarn_original_bf16_kernel, driver/cuda/src/kernels/rope.cu:509-548; the frequencies of
 * that scheme are a host-side inv_freq table like any other). */
int pie_hip_rope_table_scaled(const int32_t* positions, const float* inv_freq, float* table,
                              int num_tokens, int head_dim, float mscale, void* stream);

/*
 * Split a packed QKV row [N, (hq + 2*hk)*d], apply optional per-head RMSNorm (both norm
 * weights or neither) and RoPE to q and k, write q to q_out[N, hq, d], and write k (rotated)
 * and v (copied) into the KV pool [pages, page_size, hk, d] at physical slot
 * kv_slots[n] = page*page_size + offset (negative = token has no slot).  One bf16 rounding at
 * the store.  interleaved: PIE_HIP_ROPE_HALF (0) pairs (i, i+d/2), PIE_HIP_ROPE_ADJACENT (1) pairs
 * (2i, 2i+1), PIE_HIP_ROPE_HALF_PAIRED_ROWS (2): the q / k rows of the projection were re-ordered
 * at load so that elements (2i, 2i+1) of packed_qkv hold the half-split pair (i, i+d/2); they are
 * rotated as that pair and written to positions i and i+d/2 (V rows are as stored) — the output
 * of mode 0 over the original row order, bit for bit.
 * Reference: launch_qkv_decode_qk_norm_rope_write_kv_bf16,
 * driver/cuda/src/kernels/split_packed.hpp:34-57, split_packed.cu:62-178; slot arithmetic of
 * driver/portable/src/plan.hpp:36-45 is done by the caller.
 */
int pie_hip_qkv_rope_kvwrite(const uint16_t* packed_qkv, uint16_t* q_out, uint16_t* k_pages,
                             uint16_t* v_pages, const uint16_t* q_norm_weight,
                             const uint16_t* k_norm_weight, const float* rope_table,
                             const int64_t* kv_slots, int num_tokens, int num_q_heads,
                             int num_kv_heads, int head_dim, int interleaved, float eps,
                             void* stream);

/* y[n, i] = bf16( g/(1+exp(-g)) * u ), g = gate_up[n, i], u = gate_up[n, I + i].
 * Reference: swiglu_bf16_kernel, driver/cuda/src/kernels/swiglu.cu:9-22 (fused-row form
 * swiglu.hpp:82). */
int pie_hip_swiglu(const uint16_t* gate_up_bf16, uint16_t* y_bf16, int num_tokens,
                   int intermediate, void* stream);

/* out_idx[r] = argmax_i logits[r, i]; ties -> lowest index; NaN never wins.  vocab % 8 == 0.
 * Reference: argmax_bf16_kernel, driver/cuda/src/kernels/argmax.cu:36-80. */
int pie_hip_argmax(const uint16_t* logits_bf16, uint32_t* out_idx, int rows, int vocab,
                   void* stream);

/* pool page dst_pages[i] <- page src_pages[i] (device arrays), page_bytes each, in one pool.
 * Reference: Copy D2D handling, driver/portable/src/service/inproc_service.cpp:149-172. */
int pie_hip_copy_kv_pages(void* pool, const uint32_t* src_pages, const uint32_t* dst_pages,
                          int num_copies, size_t page_bytes, void* stream);

/* ---- load-time quantisers (bf16 weights -> storage formats) ---------------------- */

/* Per-output-channel int8: scale_inv[r] = absmax/127 (1 for a zero row),
 * q = clamp(rintf(w * 127/absmax), -128, 127), round half to even.
 * Reference: quantize_bf16_to_int8_per_channel, driver/cuda/src/kernels/quant_bf16_to_fp8.cu:273-333. */
int pie_hip_quant_int8_per_channel(const uint16_t* w_bf16, int8_t* q, float* scale_inv, int rows,
                                   int cols, void* stream);
/* Per-output-channel fp8 e4m3fn: scale_inv[r] = absmax/448, q = e4m3_satfinite(w * 448/absmax).
 * Reference: quant_per_channel_kernel, driver/cuda/src/kernels/quant_bf16_to_fp8.cu:181-226. */
int pie_hip_quant_fp8_per_channel(const uint16_t* w_bf16, uint8_t* q_e4m3, float* scale_inv,
                                  int rows, int cols, void* stream);
/* Symmetric group-wise int4 into the int4b8 layout: scale = bf16(absmax/7) per (row, group)
 * (1 for a zero group), nibble = clamp(rintf(w/scale), -8, 7) + 8.  The reference defines the
 * layout (driver/cuda/src/kernels/dequant_wna16.cu:11-38) but ships no quantiser for it. */
int pie_hip_quant_int4b8_group(const uint16_t* w_bf16, uint32_t* packed, uint16_t* scale_bf16,
                               int rows, int cols, int group_size, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PIE_HIP_KERNELS_H */
