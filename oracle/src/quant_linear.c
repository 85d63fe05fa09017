/*
 * Oracle: quantised weight formats and the weight-only linear (GEMV/GEMM).
 * TEST INFRASTRUCTURE ONLY (see oracle_common.h).
 *
 * Follows the reference CUDA driver's explicit kernels:
 *   int4b8 unpack + dequant   driver/cuda/src/kernels/dequant_wna16.cu:11-38
 *   fused W4A16 decode dot    driver/cuda/src/kernels/dequant_wna16.cu:96-110
 *   int8 per-channel quant    driver/cuda/src/kernels/quant_bf16_to_fp8.cu:273-323
 *   int8 dequant              driver/cuda/src/kernels/quant_bf16_to_fp8.cu:142-155
 *   W8A16 fused GEMV          driver/cuda/src/kernels/argmax.cu:846-854
 *
 * Pinned by tests/test_oracle_quant.py: literal nibble-order known answers,
 * pack/unpack round trips over all 16 nibble values in all 8 positions, fp64
 * numpy matmul on the dequantised weights, one-hot activations, linearity in
 * the scales, and the round-half-even int8 known answers of
 * driver/portable/tests/test_kv_cache_quant.cpp.
 */
#include "oracle_common.h"

/* q[n,k] = nibble(k%8 of word k/8) - 8.  dequant_wna16.cu:31-36. */
void orc_unpack_w4(const uint32_t* packed, int8_t* q, int out_dim, int in_dim) {
    const int words = in_dim / 8;
    for (int n = 0; n < out_dim; ++n)
        for (int k = 0; k < in_dim; ++k) {
            const uint32_t word = packed[(size_t)n * words + k / 8];
            q[(size_t)n * in_dim + k] = (int8_t)((int)((word >> (4 * (k % 8))) & 0xF) - 8);
        }
}

/* Inverse of the format, for building fixtures: nibble = q + 8. */
void orc_pack_w4(const int8_t* q, uint32_t* packed, int out_dim, int in_dim) {
    const int words = in_dim / 8;
    for (int n = 0; n < out_dim; ++n)
        for (int w = 0; w < words; ++w) {
            uint32_t word = 0;
            for (int j = 0; j < 8; ++j)
                word |= ((uint32_t)(q[(size_t)n * in_dim + w * 8 + j] + 8) & 0xFu) << (4 * j);
            packed[(size_t)n * words + w] = word;
        }
}

/* out[n,k] = bf16(float(q) * float(scale[n, k/G])).  dequant_wna16.cu:28-37. */
void orc_dequant_w4a16(const uint32_t* packed, const uint16_t* scale, uint16_t* out, int out_dim,
                       int in_dim, int group) {
    const int words = in_dim / 8, groups = in_dim / group;
    for (int n = 0; n < out_dim; ++n)
        for (int k = 0; k < in_dim; ++k) {
            const uint32_t word = packed[(size_t)n * words + k / 8];
            const float q = (float)((int)((word >> (4 * (k % 8))) & 0xF) - 8);
            const float s = orc_bf16_to_f32(scale[(size_t)n * groups + k / group]);
            out[(size_t)n * in_dim + k] = orc_f32_to_bf16(q * s);
        }
}

/*
 * y[m,n] = sum_k act[m,k] * w(n,k) (+ beta*y_in[m,n]), three evaluations:
 *   mode 0  fused fp32: acc += x * (q * s), k ascending (dequant_wna16.cu:96-110)
 *   mode 1  dequant-then-GEMM: w = bf16(q*s), fp32 accumulation
 *           (gemm_act_x_w dequant fallback, driver/cuda/src/ops/gemm.cpp:1213-1236)
 *   mode 2  fp64 ground truth of the exact product x*q*s
 * y_f32 receives the unrounded value, y_bf16 (optional) its bf16 rounding,
 * abs_sum (optional) sum_k |x*w| for error bounds.
 */
void orc_gemm_w4a16(const uint16_t* act, const uint32_t* packed, const uint16_t* scale,
                    const uint16_t* y_in, float* y_f32, uint16_t* y_bf16, double* abs_sum, int M,
                    int N, int K, int group, int beta, int mode) {
    const int words = K / 8, groups = K / group;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m) {
            float accf = 0.f;
            double accd = 0.0, absd = 0.0;
            for (int k = 0; k < K; ++k) {
                const uint32_t word = packed[(size_t)n * words + k / 8];
                const float q = (float)((int)((word >> (4 * (k % 8))) & 0xF) - 8);
                const float s = orc_bf16_to_f32(scale[(size_t)n * groups + k / group]);
                const float x = orc_bf16_to_f32(act[(size_t)m * K + k]);
                if (mode == 0) {
                    accf += x * (q * s);
                } else if (mode == 1) {
                    accf += x * orc_round_bf16(q * s);
                } else {
                    accd += (double)x * (double)q * (double)s;
                }
                absd += fabs((double)x * (double)q * (double)s);
            }
            double v = (mode == 2) ? accd : (double)accf;
            const size_t o = (size_t)m * N + n;
            if (beta) v += (double)orc_bf16_to_f32(y_in[o]);
            y_f32[o] = (float)v;
            if (y_bf16) y_bf16[o] = orc_f32_to_bf16((float)v);
            if (abs_sum) abs_sum[o] = absd;
        }
    }
}

/*
 * int8 per-output-channel quantiser: absmax over the row; scale_inv = absmax/127
 * (1 when the row is all zero); q = clamp(rintf(w * 127/absmax), -128, 127).
 * quant_bf16_to_fp8.cu:273-323.  rintf is round-half-to-even.
 */
void orc_quant_int8_per_channel(const uint16_t* w_bf16, int8_t* q, float* scale_inv, int rows,
                                int cols) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        float absmax = 0.f;
        for (int c = 0; c < cols; ++c) {
            const float v = fabsf(orc_bf16_to_f32(w_bf16[(size_t)r * cols + c]));
            if (v > absmax) absmax = v;
        }
        const float scale = absmax > 0.f ? 127.f / absmax : 1.f;
        scale_inv[r] = absmax > 0.f ? absmax / 127.f : 1.f;
        for (int c = 0; c < cols; ++c) {
            float v = rintf(orc_bf16_to_f32(w_bf16[(size_t)r * cols + c]) * scale);
            if (v > 127.f) v = 127.f;
            if (v < -128.f) v = -128.f;
            q[(size_t)r * cols + c] = (int8_t)v;
        }
    }
}

/* out = bf16(float(q) * scale_inv[row]).  quant_bf16_to_fp8.cu:142-155. */
void orc_dequant_int8_per_channel(const int8_t* q, const float* scale_inv, uint16_t* out, int rows,
                                  int cols) {
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c)
            out[(size_t)r * cols + c] = orc_f32_to_bf16((float)q[(size_t)r * cols + c] * scale_inv[r]);
}

/*
 * W8A16: y[m,n] = (sum_k f32(a[m,k]) * f32(q[n,k])) * scale_inv[n] (+ beta*y_in)
 *   mode 0  fp32 sum, scale applied once after it (argmax.cu:846-854)
 *   mode 1  dequant-then-GEMM: w = bf16(q*s), fp32 accumulation (gemm.cpp:1213-1236)
 *   mode 2  fp64 ground truth
 */
void orc_gemm_w8a16(const uint16_t* act, const int8_t* q, const float* scale_inv,
                    const uint16_t* y_in, float* y_f32, uint16_t* y_bf16, double* abs_sum, int M,
                    int N, int K, int beta, int mode) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m) {
            float accf = 0.f;
            double accd = 0.0, absd = 0.0;
            const float s = scale_inv[n];
            for (int k = 0; k < K; ++k) {
                const float x = orc_bf16_to_f32(act[(size_t)m * K + k]);
                const float w = (float)q[(size_t)n * K + k];
                if (mode == 0) accf += x * w;
                else if (mode == 1) accf += x * orc_round_bf16(w * s);
                else accd += (double)x * (double)w;
                absd += fabs((double)x * (double)w * (double)s);
            }
            double v;
            if (mode == 0) v = (double)(accf * s);
            else if (mode == 1) v = (double)accf;
            else v = accd * (double)s;
            const size_t o = (size_t)m * N + n;
            if (beta) v += (double)orc_bf16_to_f32(y_in[o]);
            y_f32[o] = (float)v;
            if (y_bf16) y_bf16[o] = orc_f32_to_bf16((float)v);
            if (abs_sum) abs_sum[o] = absd;
        }
    }
}

/*
 * OCP fp8 e4m3fn byte -> f32: sign, 4-bit exponent (bias 7), 3-bit mantissa, subnormals at
 * exponent 0, no infinities, 0x7F/0xFF = NaN (the hardware conversion; the reference's host
 * table at driver/portable/src/rust_loader.cpp:783-793 maps the NaN code to 0 instead — a
 * code no satfinite quantiser emits).
 */
float orc_fp8_e4m3_to_f32(uint8_t v) {
    const float sign = (v & 0x80) ? -1.0f : 1.0f;
    const int exp = (v >> 3) & 0x0f, mant = v & 0x07;
    if (exp == 0) return sign * ldexpf((float)mant / 8.0f, -6);
    if (exp == 0x0f && mant == 0x07) return NAN;
    return sign * ldexpf(1.0f + (float)mant / 8.0f, exp - 7);
}

void orc_fp8_decode(const uint8_t* src, float* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = orc_fp8_e4m3_to_f32(src[i]);
}

/* f32 -> e4m3fn, round to nearest even, saturating to +-448 (__NV_SATFINITE). */
uint8_t orc_f32_to_fp8_e4m3(float f) {
    if (f != f) return 0x7F;
    const uint8_t sign = signbit(f) ? 0x80 : 0x00;
    const float a = fabsf(f);
    if (a >= 448.0f) return sign | 0x7E;
    uint8_t best = 0;
    float best_err = INFINITY;
    for (int c = 0; c <= 0x7E; ++c) {
        const float err = fabsf(orc_fp8_e4m3_to_f32((uint8_t)c) - a);
        if (err < best_err || (err == best_err && (c & 1) == 0)) {
            best_err = err;
            best = (uint8_t)c;
        }
    }
    return sign | best;
}

/* Per-row fp8 quantiser: scale_inv = absmax/448 (1 if the row is zero),
 * q = e4m3_satfinite(w * 448/absmax).  quant_bf16_to_fp8.cu:181-226. */
void orc_quant_fp8_per_channel(const uint16_t* w_bf16, uint8_t* q, float* scale_inv, int rows,
                               int cols) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        float absmax = 0.f;
        for (int c = 0; c < cols; ++c) {
            const float v = fabsf(orc_bf16_to_f32(w_bf16[(size_t)r * cols + c]));
            if (v > absmax) absmax = v;
        }
        const float inv = absmax > 0.f ? 448.0f / absmax : 1.f;
        scale_inv[r] = absmax > 0.f ? absmax / 448.0f : 1.f;
        for (int c = 0; c < cols; ++c)
            q[(size_t)r * cols + c] =
                orc_f32_to_fp8_e4m3(orc_bf16_to_f32(w_bf16[(size_t)r * cols + c]) * inv);
    }
}

/*
 * fp8 weight-only linear, per-row scale:
 *   mode 0  fused: (sum_k x * f32(fp8)) * scale_inv[n], fp32 sum
 *   mode 1  dequant-then-GEMM: w = bf16(f32(fp8) * s) (dequant_fp8.cu:25-39), fp32 accumulation
 *   mode 2  fp64 ground truth
 */
void orc_gemm_fp8(const uint16_t* act, const uint8_t* q, const float* scale_inv,
                  const uint16_t* y_in, float* y_f32, uint16_t* y_bf16, double* abs_sum, int M,
                  int N, int K, int beta, int mode) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m) {
            float accf = 0.f;
            double accd = 0.0, absd = 0.0;
            const float s = scale_inv[n];
            for (int k = 0; k < K; ++k) {
                const float x = orc_bf16_to_f32(act[(size_t)m * K + k]);
                const float w = orc_fp8_e4m3_to_f32(q[(size_t)n * K + k]);
                if (mode == 0) accf += x * w;
                else if (mode == 1) accf += x * orc_round_bf16(w * s);
                else accd += (double)x * (double)w;
                absd += fabs((double)x * (double)w * (double)s);
            }
            double v;
            if (mode == 0) v = (double)(accf * s);
            else if (mode == 1) v = (double)accf;
            else v = accd * (double)s;
            const size_t o = (size_t)m * N + n;
            if (beta) v += (double)orc_bf16_to_f32(y_in[o]);
            y_f32[o] = (float)v;
            if (y_bf16) y_bf16[o] = orc_f32_to_bf16((float)v);
            if (abs_sum) abs_sum[o] = absd;
        }
    }
}
