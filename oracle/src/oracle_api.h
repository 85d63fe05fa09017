/* Prototypes of the oracle's C functions that other oracle sources call.
 * TEST INFRASTRUCTURE ONLY (see oracle_common.h). */
#ifndef PIE_ORACLE_API_H
#define PIE_ORACLE_API_H
#include "oracle_common.h"

void orc_embed(const uint32_t* tokens, const uint16_t* table, uint16_t* y, int n_tokens, int hidden,
               int vocab);
void orc_rmsnorm(uint16_t* x, const uint16_t* residual, const uint16_t* w, uint16_t* y, int rows,
                 int hidden, float eps);
void orc_rope_table(const int32_t* positions, const float* inv_freq, float* table, int n_tokens,
                    int d);
void orc_rope_table_scaled(const int32_t* positions, const float* inv_freq, float* table, int n_tokens,
                           int d, float mscale);
void orc_qkv_rope_kvwrite(const uint16_t* packed, uint16_t* q_out, uint16_t* k_pages,
                          uint16_t* v_pages, const uint16_t* q_norm_w, const uint16_t* k_norm_w,
                          const float* table, const int64_t* kv_slots, int n_tokens, int hq, int hk,
                          int d, int interleaved, float eps);
void orc_swiglu(const uint16_t* gate_up, uint16_t* y, int n_tokens, int inter);
void orc_argmax_bf16(const uint16_t* logits, uint32_t* out, int rows, int vocab);
void orc_gemm_bf16(const uint16_t* act, const uint16_t* w, const uint16_t* y_in, float* y_f32,
                   uint16_t* y_bf16, double* abs_sum, int M, int N, int K, int beta, int mode);
void orc_gemm_w4a16(const uint16_t* act, const uint32_t* packed, const uint16_t* scale,
                    const uint16_t* y_in, float* y_f32, uint16_t* y_bf16, double* abs_sum, int M,
                    int N, int K, int group, int beta, int mode);
void orc_gemm_w8a16(const uint16_t* act, const int8_t* q, const float* scale_inv,
                    const uint16_t* y_in, float* y_f32, uint16_t* y_bf16, double* abs_sum, int M,
                    int N, int K, int beta, int mode);
void orc_gemm_fp8(const uint16_t* act, const uint8_t* q, const float* scale_inv,
                  const uint16_t* y_in, float* y_f32, uint16_t* y_bf16, double* abs_sum, int M,
                  int N, int K, int beta, int mode);
void orc_attn_rows(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                   float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                   const uint32_t* row_begin, const int32_t* row_len, int rows, int hq, int hk,
                   int d, int ps, float sm_scale, int mode);
void orc_attn_rows_masked(const uint16_t* q, const uint16_t* k_pages, const uint16_t* v_pages,
                          float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                          const uint32_t* row_begin, const int32_t* row_len, int rows, int hq,
                          int hk, int d, int ps, float sm_scale, int mode, const uint8_t* allow,
                          const int64_t* allow_off);
void orc_brle_allow(const uint32_t* runs, size_t n_runs, int pos, int n_kv, int window,
                    uint8_t* out);
void orc_topk_softmax(const uint16_t* logits, int32_t* topk_idx, float* topk_w, int N, int E, int K);
void orc_topk_softmax_opt(const uint16_t* logits, int32_t* topk_idx, float* topk_w, int N, int E, int K,
                          int renorm);
void orc_moe_combine(const uint16_t* y_routes, const float* topk_w, uint16_t* out, int N, int K,
                     int H, int add);
void orc_pcg32_sequence(uint64_t seed, uint64_t stream, uint32_t* out, int n);
float orc_pcg32_first_uniform(uint64_t seed);
void orc_apply_brle_logit_mask(float* logits, int V, const uint32_t* runs, size_t n_runs);
void orc_softmax_temperature(const float* logits, int V, float temperature, float* probs);
int orc_sample_token(const float* logits, int V, int kind, float temperature, uint32_t top_k,
                     float top_p, float min_p, float u, uint32_t* token, float* margin);
int orc_distribution(const float* logits, int V, float temperature, uint32_t k, uint32_t* ids,
                     float* vals);
int orc_logprobs_at(const float* logits, int V, const uint32_t* labels, int n, float* out);
float orc_entropy(const float* logits, int V);
#endif
