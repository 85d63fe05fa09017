/*
 * Oracle: the forward pass of model.c evaluated without the bf16 rounding points, in two forms.
 * TEST INFRASTRUCTURE ONLY (see oracle_common.h).
 *
 *   mode 1 ("P", portable-faithful): the rounding points of the reference's portable CPU driver.
 *     The residual stream and every activation between ops are F32 (ggml get_rows / mul_mat /
 *     rms_norm / flash_attn_ext produce F32 and the graph never casts back:
 *     driver/portable/src/graph_qwen3.cpp:85,287-291,551,572,723); K and V are rounded to F16 at
 *     the pool write (the pool's type, driver/portable/src/executor/executor.cpp:351,359);
 *     activations meeting bf16 weights are rounded to bf16 first, as ggml's mul_mat does.
 *     Quantised weights are dequantised exactly and multiplied in F32 (the portable driver has no
 *     counterpart of these storage formats, so that part is this oracle's definition).
 *   mode 2 (truth): the same graph in double with nothing rounded — the value both drivers
 *     approximate.  Format error and kernel error separate against it: a GPU result and the
 *     mode-C oracle are each compared with this one.
 *
 * KV pools are double arrays [pages, page_size, hk, d] in both modes (mode 1 stores F16-rounded
 * values in them).  Pinned by tests/test_oracle_model.py against an independent numpy fp64
 * transformer: mode 2 to 1e-9 of the logits, mode 1 to F32 / F16 accuracy.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "model_types.h"

float orc_fp8_e4m3_to_f32(uint8_t v);

/* f32 -> IEEE binary16 -> f32, round to nearest even, overflow to infinity, subnormals kept. */
float orc_round_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = x & 0x80000000u;
    x &= 0x7FFFFFFFu;
    if (x >= 0x7F800000u) return f;                 /* inf / nan */
    float r;
    if (x >= 0x477FF000u) {                         /* >= 65520: rounds past the largest half */
        r = INFINITY;
    } else if (x < 0x38800000u) {                   /* < 2^-14: half subnormals, quantum 2^-24 */
        float a;
        memcpy(&a, &x, 4);
        r = rintf(a * 16777216.0f) / 16777216.0f;
    } else {                                        /* 10 mantissa bits kept of 23 */
        x += 0xFFFu + ((x >> 13) & 1u);
        x &= ~0x1FFFu;
        memcpy(&r, &x, 4);
    }
    uint32_t u;
    memcpy(&u, &r, 4);
    u |= sign;
    memcpy(&r, &u, 4);
    return r;
}

void orc_round_f16_array(const float* in, float* out, size_t n) {
    for (size_t i = 0; i < n; ++i) out[i] = orc_round_f16(in[i]);
}

#define REAL double
#define FN(name) hp64_##name
#define HP_KV_F16 0
#define HP_ACT_BF16_FOR_BF16_WEIGHTS 0
#include "model_hp_body.h"
#undef REAL
#undef FN
#undef HP_KV_F16
#undef HP_ACT_BF16_FOR_BF16_WEIGHTS

#define REAL float
#define FN(name) hp32_##name
#define HP_KV_F16 1
#define HP_ACT_BF16_FOR_BF16_WEIGHTS 1
#include "model_hp_body.h"
#undef REAL
#undef FN
#undef HP_KV_F16
#undef HP_ACT_BF16_FOR_BF16_WEIGHTS

/* mode: 1 = F32 activations + F16 KV, 2 = double.  logits_out [S, V] double (may be NULL). */
void orc_llama_forward_hp(const OrcModel* m, int mode, double* const* k_pool, double* const* v_pool,
                          const uint32_t* tokens, const int32_t* positions, const int64_t* kv_slots,
                          const uint32_t* row_begin, const int32_t* row_len,
                          const uint32_t* page_indices, int N, const uint32_t* sample_rows, int S,
                          int page_size, uint32_t* out_tokens, double* logits_out,
                          const uint8_t* allow, const int64_t* allow_off) {
    if (mode == 1)
        hp32_forward(m, k_pool, v_pool, tokens, positions, kv_slots, row_begin, row_len, page_indices, N,
                     sample_rows, S, page_size, out_tokens, logits_out, allow, allow_off);
    else
        hp64_forward(m, k_pool, v_pool, tokens, positions, kv_slots, row_begin, row_len, page_indices, N,
                     sample_rows, S, page_size, out_tokens, logits_out, allow, allow_off);
}
