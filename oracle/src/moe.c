/*
 * Oracle: MoE routing and combine.  TEST INFRASTRUCTURE ONLY (see oracle_common.h).
 *
 * orc_topk_softmax follows topk_softmax_bf16_kernel (driver/cuda/src/kernels/topk_softmax.cu:
 * 19-86): softmax over the experts in fp32 (max, exp, sum, multiply by 1/Z), K passes of argmax
 * with exclusion where a strictly greater value wins (so the lowest index wins ties), weights
 * divided by their sum accumulated in selection order.  Same selection rule as the graph form
 * softmax -> top_k -> gather -> divide by the sum (driver/portable/src/graph_common.cpp:262-283),
 * which divides only under norm_topk (:279-283): orc_topk_softmax_opt with renorm = 0 returns the
 * chosen experts' softmax probabilities as they are.
 * The reference sums the exponentials in a strided tree; here the sum is sequential — results
 * agree to fp32 rounding.
 *
 * orc_moe_combine follows token_batched_weighted_sum[_add]_bf16_kernel
 * (driver/cuda/src/kernels/moe_dispatch.cu:152-196): fp32 accumulation of weight * bf16 route
 * output in top-k order (nvcc contracts `acc += w * v` into an FMA), one rounding, optionally
 * added onto the bf16 residual before that rounding.
 *
 * Pinned by tests/test_oracle_moe.py: against numpy float64 softmax + stable argsort on
 * separated logits (with and without the division), constructed ties, weights summing to one,
 * and a float64 weighted sum.
 */
#include "oracle_api.h"

void orc_topk_softmax(const uint16_t* logits, int32_t* topk_idx, float* topk_w, int N, int E, int K) {
    orc_topk_softmax_opt(logits, topk_idx, topk_w, N, E, K, 1);
}

void orc_topk_softmax_opt(const uint16_t* logits, int32_t* topk_idx, float* topk_w, int N, int E, int K,
                          int renorm) {
    for (int n = 0; n < N; ++n) {
        const uint16_t* row = logits + (size_t)n * E;
        float probs[512];
        float mx = -3.4e38f;
        for (int j = 0; j < E; ++j) {
            probs[j] = orc_bf16_to_f32(row[j]);
            if (probs[j] > mx) mx = probs[j];
        }
        float sum = 0.f;
        for (int j = 0; j < E; ++j) {
            probs[j] = expf(probs[j] - mx);
            sum += probs[j];
        }
        const float inv_z = 1.f / sum;
        for (int j = 0; j < E; ++j) probs[j] *= inv_z;
        float w_sum = 0.f;
        for (int k = 0; k < K; ++k) {
            int best_i = -1;
            float best_v = -1.f;
            for (int j = 0; j < E; ++j)
                if (probs[j] > best_v) {
                    best_v = probs[j];
                    best_i = j;
                }
            topk_idx[(size_t)n * K + k] = best_i;
            topk_w[(size_t)n * K + k] = best_v;
            w_sum += best_v;
            probs[best_i] = -1.f;
        }
        if (!renorm) continue;
        const float inv_w = 1.f / w_sum;
        for (int k = 0; k < K; ++k) topk_w[(size_t)n * K + k] *= inv_w;
    }
}

/* y_routes: [N*K, H] in (token, k) order. */
void orc_moe_combine(const uint16_t* y_routes, const float* topk_w, uint16_t* out, int N, int K,
                     int H, int add) {
    for (int n = 0; n < N; ++n)
        for (int h = 0; h < H; ++h) {
            float acc = 0.f;
            for (int k = 0; k < K; ++k)
                acc = fmaf(topk_w[(size_t)n * K + k],
                           orc_bf16_to_f32(y_routes[((size_t)n * K + k) * H + h]), acc);
            uint16_t* o = out + (size_t)n * H + h;
            *o = orc_f32_to_bf16(add ? orc_bf16_to_f32(*o) + acc : acc);
        }
}
