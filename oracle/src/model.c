/*
 * Oracle: one forward pass of the llama-like decoder over a paged KV cache — the control
 * flow and op sequence of the reference.  TEST INFRASTRUCTURE ONLY (see oracle_common.h).
 *
 * Graph: driver/portable/src/graph_qwen3.cpp:225-896 (norm -> QKV -> [qk-norm] -> RoPE ->
 * KV write at the token's slot -> attention over the request's pages -> o_proj + residual ->
 * norm -> SwiGLU FFN + residual; tail: final norm, lm_head on the sampled rows only, argmax).
 * Rounding points: those of the reference's kernel-by-kernel CUDA forward
 * (driver/cuda/src/model/llama_like.cpp:364-762): every inter-op activation is bf16, fp32
 * inside an op, residual add fused into the projection with one rounding (:626-628,:703-705).
 * Quantised linears use the fused evaluation order (scale applied to fp32 partial sums).
 * MoE layers (qwen3_moe): router GEMM -> top-k softmax -> per-route gate/up -> SwiGLU (bf16) ->
 * per-route down, rounded to bf16 per route -> weighted sum onto the residual — the composition
 * of driver/cuda/src/model/kimi_forward.cpp:662-714 (graph form
 * driver/portable/src/graph_common.cpp:237-345).
 *
 * The composition is pinned by tests/test_oracle_model.py: every op is one of the separately
 * pinned oracle functions, and the whole pass is compared with an independent numpy fp64
 * transformer on a tiny model (cosine of the logits, the tolerance precedent of
 * driver/cuda/tests/parity_qwen3.py:160-181).
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "oracle_api.h"

#include "model_types.h"

static void orc_linear(const OrcModel* m, const OrcLinear* w, const uint16_t* act, uint16_t* y,
                       int M, int N, int K, int beta) {
    float* tmp = (float*)malloc(sizeof(float) * (size_t)M * N);
    switch (m->quant) {
        case 0:
            orc_gemm_w4a16(act, (const uint32_t*)w->data, (const uint16_t*)w->scale, y, tmp, y, NULL,
                           M, N, K, m->group, beta, 0);
            break;
        case 1:
            orc_gemm_w8a16(act, (const int8_t*)w->data, (const float*)w->scale, y, tmp, y, NULL, M, N,
                           K, beta, 0);
            break;
        case 2:
            orc_gemm_fp8(act, (const uint8_t*)w->data, (const float*)w->scale, y, tmp, y, NULL, M, N, K,
                         beta, 0);
            break;
        default:
            orc_gemm_bf16(act, (const uint16_t*)w->data, y, tmp, y, NULL, M, N, K, beta, 0);
            break;
    }
    free(tmp);
}

/* Expert e's [N, K] slice of a stacked linear. */
static OrcLinear orc_expert_slice(const OrcModel* m, const OrcLinear* w, int e, int N, int K) {
    OrcLinear s;
    const size_t nk = (size_t)e * N * K;
    switch (m->quant) {
        case 0:
            s.data = (const unsigned char*)w->data + nk / 2;
            s.scale = (const unsigned char*)w->scale + (size_t)e * N * (K / m->group) * 2;
            break;
        case 1:
        case 2:
            s.data = (const unsigned char*)w->data + nk;
            s.scale = (const unsigned char*)w->scale + (size_t)e * N * 4;
            break;
        default:
            s.data = (const unsigned char*)w->data + nk * 2;
            s.scale = NULL;
            break;
    }
    return s;
}

/* Test diagnostic: the smallest gap between the last selected and the first rejected router
 * logit, relative to the largest logit magnitude of that token, over every (layer, token) routed
 * since the last reset.  A gap at bf16 resolution
 * means another summation order may pick another expert there: the parity tests flag such a
 * forward as a near-tie instead of holding it to the logit bar. */
#define ORC_ROUTER_GAP_ROWS 8192
static float g_router_min_gap = 3.4e38f;
static float g_router_row_gap[ORC_ROUTER_GAP_ROWS]; /* the same, per row of the forward (min over layers) */
void orc_router_gap_reset(void) {
    g_router_min_gap = 3.4e38f;
    for (int i = 0; i < ORC_ROUTER_GAP_ROWS; ++i) g_router_row_gap[i] = 3.4e38f;
}
float orc_router_gap_get(void) { return g_router_min_gap; }
void orc_router_gap_rows(float* out, int n) {
    for (int i = 0; i < n; ++i) out[i] = i < ORC_ROUTER_GAP_ROWS ? g_router_row_gap[i] : 0.f;
}
static void orc_router_gap_note(const uint16_t* logits, int N, int E, int K) {
    if (K < 1 || K >= E || E > 512) return;
    for (int n = 0; n < N; ++n) {
        float v[512];
        for (int j = 0; j < E; ++j) v[j] = orc_bf16_to_f32(logits[(size_t)n * E + j]);
        for (int k = 0; k <= K; ++k) { /* partial selection sort: v[0..K] descending */
            int b = k;
            for (int j = k + 1; j < E; ++j)
                if (v[j] > v[b]) b = j;
            const float t = v[k]; v[k] = v[b]; v[b] = t;
        }
        float mag = 0.f; /* the row's largest magnitude: the error of a logit scales with the
                            size of the sum's terms, not with the logit's own value */
        for (int j = 0; j < E; ++j) mag = fabsf(v[j]) > mag ? fabsf(v[j]) : mag;
        const float gap = (v[K - 1] - v[K]) / (mag > 1e-20f ? mag : 1e-20f);
        if (gap < g_router_min_gap) g_router_min_gap = gap;
        if (n < ORC_ROUTER_GAP_ROWS && gap < g_router_row_gap[n]) g_router_row_gap[n] = gap;
    }
}

/* Test diagnostic: when set, row 0 of the last layer's intermediates of the next forward is
 * copied out: q after RoPE [hq*d], attention output [hq*d], SwiGLU output [I] (dense models),
 * residual stream after the layer [H].  Any pointer may be NULL. */
static uint16_t *g_cap_q = NULL, *g_cap_attn = NULL, *g_cap_act = NULL, *g_cap_x = NULL;
void orc_debug_capture(uint16_t* q, uint16_t* attn, uint16_t* act, uint16_t* x) {
    g_cap_q = q; g_cap_attn = attn; g_cap_act = act; g_cap_x = x;
}

/* x[t] += sum_k w[t,k] * down_e(swiglu(gateup_e(xn[t]))) over the token's top-k experts. */
static void orc_moe_ffn(const OrcModel* m, int l, const uint16_t* xn, uint16_t* x, int N) {
    const int H = m->hidden, E = m->num_experts, K = m->top_k, Ie = m->expert_intermediate;
    uint16_t* logits = (uint16_t*)malloc((size_t)N * E * 2);
    float* lf = (float*)malloc((size_t)N * E * 4);
    int32_t* idx = (int32_t*)malloc((size_t)N * K * 4);
    float* wts = (float*)malloc((size_t)N * K * 4);
    uint16_t* yr = (uint16_t*)malloc((size_t)N * K * H * 2);
    orc_gemm_bf16(xn, m->router[l], NULL, lf, logits, NULL, N, E, H, 0, 0);
    orc_topk_softmax_opt(logits, idx, wts, N, E, K, m->raw_topk ? 0 : 1);
    orc_router_gap_note(logits, N, E, K);
#pragma omp parallel for schedule(dynamic)
    for (int r = 0; r < N * K; ++r) {
        const int t = r / K, e = idx[r];
        uint16_t* gu = (uint16_t*)malloc((size_t)2 * Ie * 2);
        uint16_t* act = (uint16_t*)malloc((size_t)Ie * 2);
        const OrcLinear wg = orc_expert_slice(m, &m->wgu[l], e, 2 * Ie, H);
        const OrcLinear wd = orc_expert_slice(m, &m->wdown[l], e, H, Ie);
        orc_linear(m, &wg, xn + (size_t)t * H, gu, 1, 2 * Ie, H, 0);
        orc_swiglu(gu, act, 1, Ie);
        orc_linear(m, &wd, act, yr + (size_t)r * H, 1, H, Ie, 0);
        free(gu);
        free(act);
    }
    orc_moe_combine(yr, wts, x, N, K, H, 1);
    free(logits); free(lf); free(idx); free(wts); free(yr);
}

/*
 * tokens/positions/kv_slots/row_begin/row_len: [N] as produced by the planner; k_pages/v_pages:
 * [L] pools [pages, ps, hk, d], updated in place; sample_rows [S] -> out_tokens [S] and, when
 * non-NULL, logits_bf16 [S, V].  allow / allow_off: optional per-row key visibility (custom
 * attention masks), as orc_attn_rows_masked takes them.
 */
void orc_kv_quant_rows(const uint16_t* x, uint8_t* codes, float* scales, float* dequant, int rows,
                       int d, int fmt);
void orc_attn_rows_f32kv(const uint16_t* q, const float* k_pages, const float* v_pages,
                         float* o_f32, uint16_t* o_bf16, float* lse, const uint32_t* page_indices,
                         const uint32_t* row_begin, const int32_t* row_len, int rows, int hq,
                         int hk, int d, int ps, float sm_scale, int mode, const uint8_t* allow,
                         const int64_t* allow_off);

/* kv_format != 0: a one-byte KV-cache format (1 fp8_e4m3, 2 int8_per_token_head,
 * 3 fp8_per_token_head, 4 fp8_e5m2, 5 fp4 blocks).  The step's rotated K / V rows are quantised per (token, head) as
 * kv_paged.cu:155-297 does and the pools k_f32 / v_f32 [L][pages, ps, hk, d] hold the values the
 * attention reads back, float(code) * scale (attention_naive_paged.cu:56-112). */
static void orc_llama_forward_impl(const OrcModel* m, uint16_t* const* k_pages, uint16_t* const* v_pages,
                       int kv_format, float* const* k_f32, float* const* v_f32,
                       const uint32_t* tokens, const int32_t* positions, const int64_t* kv_slots,
                       const uint32_t* row_begin, const int32_t* row_len,
                       const uint32_t* page_indices, int N, const uint32_t* sample_rows, int S,
                       int page_size, uint32_t* out_tokens, uint16_t* logits_bf16,
                       const uint8_t* allow, const int64_t* allow_off) {
    const int H = m->hidden, d = m->head_dim, hq = m->q_heads, hk = m->kv_heads;
    const int I = m->intermediate, V = m->vocab;
    const int qkv_dim = (hq + 2 * hk) * d;
    uint16_t* x = (uint16_t*)malloc((size_t)N * H * 2);
    uint16_t* xn = (uint16_t*)malloc((size_t)N * H * 2);
    uint16_t* qkv = (uint16_t*)malloc((size_t)N * qkv_dim * 2);
    uint16_t* q = (uint16_t*)malloc((size_t)N * hq * d * 2);
    uint16_t* attn = (uint16_t*)malloc((size_t)N * hq * d * 2);
    float* attn_f = (float*)malloc((size_t)N * hq * d * 4);
    uint16_t* gu = (uint16_t*)malloc((size_t)N * 2 * I * 2);
    uint16_t* act = (uint16_t*)malloc((size_t)N * I * 2);
    float* tab = (float*)malloc((size_t)N * d * 4);
    const size_t kvrow = (size_t)hk * d;
    uint16_t *k_rows = NULL, *v_rows = NULL;
    uint8_t* codes = NULL;
    float *scales = NULL, *deq = NULL;
    int64_t* iota = NULL;
    if (kv_format) {
        k_rows = (uint16_t*)malloc((size_t)N * kvrow * 2);
        v_rows = (uint16_t*)malloc((size_t)N * kvrow * 2);
        codes = (uint8_t*)malloc((size_t)N * kvrow);
        scales = (float*)malloc((size_t)N * hk * ((d + 15) / 16) * 4);   /* (fp4: one per 16-element block) */
        deq = (float*)malloc((size_t)N * kvrow * 4);
        iota = (int64_t*)malloc((size_t)N * 8);
        for (int i = 0; i < N; ++i) iota[i] = i;
    }

    orc_embed(tokens, m->embed, x, N, H, V);
    orc_rope_table_scaled(positions, m->inv_freq, tab, N, d, m->rope_mscale > 0.f ? m->rope_mscale : 1.0f);
    for (int l = 0; l < m->layers; ++l) {
        orc_rmsnorm(x, NULL, m->attn_norm[l], xn, N, H, m->rms_eps);
        orc_linear(m, &m->wqkv[l], xn, qkv, N, qkv_dim, H, 0);
        if (kv_format) {
            orc_qkv_rope_kvwrite(qkv, q, k_rows, v_rows, m->has_qk_norm ? m->q_norm[l] : NULL,
                                 m->has_qk_norm ? m->k_norm[l] : NULL, tab, iota, N, hq, hk, d,
                                 m->rope_interleaved, m->rms_eps);
            for (int kv = 0; kv < 2; ++kv) {
                orc_kv_quant_rows(kv ? v_rows : k_rows, codes, scales, deq, N * hk, d, kv_format);
                float* pool = kv ? v_f32[l] : k_f32[l];
                for (int t = 0; t < N; ++t)
                    if (kv_slots[t] >= 0)
                        memcpy(pool + (size_t)kv_slots[t] * kvrow, deq + (size_t)t * kvrow, kvrow * 4);
            }
            orc_attn_rows_f32kv(q, k_f32[l], v_f32[l], attn_f, attn, NULL, page_indices, row_begin,
                                row_len, N, hq, hk, d, page_size, -1.f, 0, allow, allow_off);
        } else {
            orc_qkv_rope_kvwrite(qkv, q, k_pages[l], v_pages[l], m->has_qk_norm ? m->q_norm[l] : NULL,
                                 m->has_qk_norm ? m->k_norm[l] : NULL, tab, kv_slots, N, hq, hk, d,
                                 m->rope_interleaved, m->rms_eps);
            orc_attn_rows_masked(q, k_pages[l], v_pages[l], attn_f, attn, NULL, page_indices, row_begin,
                                 row_len, N, hq, hk, d, page_size, -1.f, 0, allow, allow_off);
        }
        orc_linear(m, &m->wo[l], attn, x, N, H, hq * d, 1);
        orc_rmsnorm(x, NULL, m->ffn_norm[l], xn, N, H, m->rms_eps);
        if (m->num_experts > 0) {
            orc_moe_ffn(m, l, xn, x, N);
        } else {
            orc_linear(m, &m->wgu[l], xn, gu, N, 2 * I, H, 0);
            orc_swiglu(gu, act, N, I);
            orc_linear(m, &m->wdown[l], act, x, N, H, I, 1);
        }
        if (l == m->layers - 1) {
            if (g_cap_q) memcpy(g_cap_q, q, (size_t)hq * d * 2);
            if (g_cap_attn) memcpy(g_cap_attn, attn, (size_t)hq * d * 2);
            if (g_cap_act && m->num_experts == 0) memcpy(g_cap_act, act, (size_t)I * 2);
            if (g_cap_x) memcpy(g_cap_x, x, (size_t)H * 2);
        }
    }
    if (S > 0) {
        uint16_t* xs = (uint16_t*)malloc((size_t)S * H * 2);
        uint16_t* xsn = (uint16_t*)malloc((size_t)S * H * 2);
        uint16_t* lg = logits_bf16 ? logits_bf16 : (uint16_t*)malloc((size_t)S * V * 2);
        float* lgf = (float*)malloc((size_t)S * V * 4);
        orc_embed(sample_rows, x, xs, S, H, N); /* row gather */
        orc_rmsnorm(xs, NULL, m->final_norm, xsn, S, H, m->rms_eps);
        orc_gemm_bf16(xsn, m->lm_head, NULL, lgf, lg, NULL, S, V, H, 0, 0);
        orc_argmax_bf16(lg, out_tokens, S, V);
        free(xs);
        free(xsn);
        free(lgf);
        if (!logits_bf16) free(lg);
    }
    free(x); free(xn); free(qkv); free(q); free(attn); free(attn_f); free(gu); free(act); free(tab);
    free(k_rows); free(v_rows); free(codes); free(scales); free(deq); free(iota);
}

void orc_llama_forward(const OrcModel* m, uint16_t* const* k_pages, uint16_t* const* v_pages,
                       const uint32_t* tokens, const int32_t* positions, const int64_t* kv_slots,
                       const uint32_t* row_begin, const int32_t* row_len,
                       const uint32_t* page_indices, int N, const uint32_t* sample_rows, int S,
                       int page_size, uint32_t* out_tokens, uint16_t* logits_bf16,
                       const uint8_t* allow, const int64_t* allow_off) {
    orc_llama_forward_impl(m, k_pages, v_pages, 0, NULL, NULL, tokens, positions, kv_slots, row_begin,
                           row_len, page_indices, N, sample_rows, S, page_size, out_tokens,
                           logits_bf16, allow, allow_off);
}

void orc_llama_forward_kvq(const OrcModel* m, int kv_format, float* const* k_f32, float* const* v_f32,
                           const uint32_t* tokens, const int32_t* positions, const int64_t* kv_slots,
                           const uint32_t* row_begin, const int32_t* row_len,
                           const uint32_t* page_indices, int N, const uint32_t* sample_rows, int S,
                           int page_size, uint32_t* out_tokens, uint16_t* logits_bf16,
                           const uint8_t* allow, const int64_t* allow_off) {
    orc_llama_forward_impl(m, NULL, NULL, kv_format, k_f32, v_f32, tokens, positions, kv_slots,
                           row_begin, row_len, page_indices, N, sample_rows, S, page_size, out_tokens,
                           logits_bf16, allow, allow_off);
}
