/* The model description the oracle's forward passes take (weights in the driver's storage
 * formats).  TEST INFRASTRUCTURE ONLY (see oracle_common.h). */
#ifndef PIE_ORACLE_MODEL_TYPES_H
#define PIE_ORACLE_MODEL_TYPES_H
#include "oracle_common.h"

typedef struct {
    const void* data;
    const void* scale; /* int4: bf16 [N, K/G]; int8/fp8: f32 [N]; bf16: NULL */
} OrcLinear;

typedef struct {
    int hidden, layers, q_heads, kv_heads, head_dim, intermediate, vocab;
    float rms_eps;
    int rope_interleaved, has_qk_norm;
    int quant; /* 0 int4b8, 1 int8, 2 fp8, 3 bf16 */
    int group;
    const uint16_t* embed;
    const uint16_t* lm_head;
    const uint16_t* final_norm;
    const float* inv_freq;
    const uint16_t* const* attn_norm; /* [L] */
    const uint16_t* const* ffn_norm;
    const uint16_t* const* q_norm;
    const uint16_t* const* k_norm;
    const OrcLinear* wqkv; /* [L] */
    const OrcLinear* wo;
    const OrcLinear* wgu;
    const OrcLinear* wdown;
    /* MoE (num_experts > 0): wgu / wdown hold the experts stacked along the rows,
     * [E * 2*Ie, H] (per expert: gate rows then up rows) and [E * H, Ie]. */
    int num_experts, top_k, expert_intermediate;
    const uint16_t* const* router; /* [L] bf16 [E, H] */
    float rope_mscale;             /* cos and sin are multiplied by it (YaRN's attention factor; 1 otherwise) */
    int raw_topk;                  /* MoE: 1 = the chosen experts' probabilities are not divided by their sum
                                      (norm_topk = false, driver/portable/src/graph_common.cpp:279-283) */
} OrcModel;

#endif
