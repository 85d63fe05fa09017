/*
 * CPU oracle for the Pie driver forward-pass kernels — TEST INFRASTRUCTURE ONLY.
 *
 * This directory restates, in plain C, the arithmetic of the reference for the
 * hot path.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load it, and only as the checker or the reported CPU baseline; the
 * product (pie_amd/) never links or imports anything from here.
 */
#ifndef PIE_ORACLE_COMMON_H
#define PIE_ORACLE_COMMON_H

#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#ifdef __cplusplus
extern "C" {
#endif

static inline float orc_bf16_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Round-to-nearest-even, NaN kept quiet (what __float2bfloat16 does). */
static inline uint16_t orc_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static inline float orc_round_bf16(float f) { return orc_bf16_to_f32(orc_f32_to_bf16(f)); }

#ifdef __cplusplus
}
#endif
#endif
