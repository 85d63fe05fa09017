/*
 * Oracle: the small per-layer ops of the llama-like decoder.  TEST INFRASTRUCTURE ONLY
 * (see oracle_common.h).
 *
 * Each function restates one explicit kernel of the reference CUDA driver, with its
 * rounding points (fp32 inside the op, one bf16 rounding at the output):
 *   embed                 driver/cuda/src/kernels/embed.cu:8-23
 *   rmsnorm               driver/cuda/src/kernels/rmsnorm.cu:14-54
 *   residual_add_rmsnorm  driver/cuda/src/kernels/rmsnorm.cu:56-98
 *   rope table            driver/cuda/src/kernels/rope.cu:35-53
 *   qk-norm + rope + KV   driver/cuda/src/kernels/split_packed.cu:62-178, rope.cu:14-33
 *   swiglu                driver/cuda/src/kernels/swiglu.cu:9-22
 *   argmax                driver/cuda/src/kernels/argmax.cu:36-80
 *   llama3 inv_freq       driver/portable/src/model.cpp:1414-1448
 *
 * Pinned by tests/test_oracle_layer_ops.py against textbook closed forms in numpy fp64
 * (norm definition, rotation-matrix identities: norm preservation, position 0 = identity,
 * relative-position property of q.k), tie rules and literal small cases.
 */
#include "oracle_common.h"

void orc_embed(const uint32_t* tokens, const uint16_t* table, uint16_t* y, int n_tokens, int hidden,
               int vocab) {
    for (int n = 0; n < n_tokens; ++n) {
        const size_t row = tokens[n] < (uint32_t)vocab ? tokens[n] : 0;
        memcpy(y + (size_t)n * hidden, table + row * hidden, (size_t)hidden * 2);
    }
}

/* residual may be NULL (plain norm).  With a residual, x is updated in place to bf16(x + r). */
void orc_rmsnorm(uint16_t* x, const uint16_t* residual, const uint16_t* w, uint16_t* y, int rows,
                 int hidden, float eps) {
    for (int r = 0; r < rows; ++r) {
        uint16_t* xr = x + (size_t)r * hidden;
        float ss = 0.f;
        for (int i = 0; i < hidden; ++i) {
            if (residual) {
                const float sum = orc_bf16_to_f32(xr[i]) + orc_bf16_to_f32(residual[(size_t)r * hidden + i]);
                xr[i] = orc_f32_to_bf16(sum);
            }
            const float v = orc_bf16_to_f32(xr[i]);
            ss += v * v;
        }
        const float inv_rms = 1.0f / sqrtf(ss / (float)hidden + eps);
        for (int i = 0; i < hidden; ++i)
            y[(size_t)r * hidden + i] =
                orc_f32_to_bf16(orc_bf16_to_f32(xr[i]) * inv_rms * orc_bf16_to_f32(w[i]));
    }
}

/* inv_freq[i] = theta^(-2i/d), optionally scaled by the llama3 wavelength bands
 * (factor <= 0 disables scaling).  Mirrors compute_llama3_freq_factors: the stored factor
 * divides the base frequency. */
void orc_rope_inv_freq(float* inv_freq, int d, float theta, float factor, float low_freq_factor,
                       float high_freq_factor, int original_max_pos) {
    const int half = d / 2;
    const double pi = 3.14159265358979323846;
    for (int i = 0; i < half; ++i) {
        const double base = pow((double)theta, -2.0 * (double)i / (double)d);
        double f = base;
        if (factor > 0.f) {
            const double low_wavelen = (double)original_max_pos / (double)low_freq_factor;
            const double high_wavelen = (double)original_max_pos / (double)high_freq_factor;
            const double wavelen = 2.0 * pi / base;
            if (wavelen < high_wavelen) {
                f = base;
            } else if (wavelen > low_wavelen) {
                f = base / (double)factor;
            } else {
                const double smooth = ((double)original_max_pos / wavelen - (double)low_freq_factor) /
                                      ((double)high_freq_factor - (double)low_freq_factor);
                f = (1.0 - smooth) * base / (double)factor + smooth * base;
            }
        }
        inv_freq[i] = (float)f;
    }
}

void orc_rope_table_scaled(const int32_t* positions, const float* inv_freq, float* table, int n_tokens,
                           int d, float mscale) {
    const int half = d / 2;
    for (int n = 0; n < n_tokens; ++n)
        for (int i = 0; i < half; ++i) {
            const float ang = (float)positions[n] * inv_freq[i];
            table[(size_t)n * d + i] = cosf(ang) * mscale;
            table[(size_t)n * d + i + half] = sinf(ang) * mscale;
        }
}

void orc_rope_table(const int32_t* positions, const float* inv_freq, float* table, int n_tokens,
                    int d) {
    orc_rope_table_scaled(positions, inv_freq, table, n_tokens, d, 1.0f);
}

/* YaRN frequencies (launch_rope_yarn_original_bf16, driver/cuda/src/kernels/rope.cu:495-507,
 * 552-589; transformers' _compute_yarn_parameters): pairs below low_dim keep theta^(-2i/d), pairs
 * above high_dim are divided by the factor, a linear ramp between; low / high from the number of
 * rotations beta_fast / beta_slow a pair makes over the original context. */
void orc_rope_inv_freq_yarn(float* inv_freq, int d, float theta, float factor, float beta_fast,
                            float beta_slow, int original_max_pos) {
    const int half = d / 2;
    const double pi = 3.14159265358979323846;
    const double ln_theta = log((double)theta);
    double lo = floor(d * log((double)original_max_pos / ((double)beta_fast * 2.0 * pi)) / (2.0 * ln_theta));
    double hi = ceil(d * log((double)original_max_pos / ((double)beta_slow * 2.0 * pi)) / (2.0 * ln_theta));
    if (lo < 0.0) lo = 0.0;
    if (hi > (double)half - 1.0) hi = (double)half - 1.0;
    if (hi < lo) hi = lo;
    const double denom = hi == lo ? hi + 1e-3 - lo : hi - lo;
    for (int i = 0; i < half; ++i) {
        const double base = pow((double)theta, -2.0 * (double)i / (double)d);
        double ramp = ((double)i - lo) / denom;
        ramp = ramp < 0.0 ? 0.0 : (ramp > 1.0 ? 1.0 : ramp);
        inv_freq[i] = (float)(base * ((1.0 - ramp) + ramp / (double)factor));
    }
}

void orc_qkv_rope_kvwrite(const uint16_t* packed, uint16_t* q_out, uint16_t* k_pages,
                          uint16_t* v_pages, const uint16_t* q_norm_w, const uint16_t* k_norm_w,
                          const float* table, const int64_t* kv_slots, int n_tokens, int hq, int hk,
                          int d, int interleaved, float eps) {
    const int half = d / 2;
    const size_t stride = (size_t)(hq + 2 * hk) * d;
    for (int n = 0; n < n_tokens; ++n) {
        for (int head = 0; head < hq + 2 * hk; ++head) {
            const uint16_t* src = packed + n * stride + (size_t)head * d;
            const int is_q = head < hq, is_k = !is_q && head < hq + hk;
            const int64_t slot = kv_slots[n];
            if (!is_q && slot < 0) continue;
            if (!is_q && !is_k) {
                memcpy(v_pages + ((size_t)slot * hk + (head - hq - hk)) * d, src, (size_t)d * 2);
                continue;
            }
            const uint16_t* nw = is_q ? q_norm_w : k_norm_w;
            float inv_rms = 1.f;
            if (nw) {
                float ss = 0.f;
                for (int i = 0; i < d; ++i) ss += orc_bf16_to_f32(src[i]) * orc_bf16_to_f32(src[i]);
                inv_rms = 1.0f / sqrtf(ss / (float)d + eps);
            }
            uint16_t* dst = is_q ? q_out + ((size_t)n * hq + head) * d
                                 : k_pages + ((size_t)slot * hk + (head - hq)) * d;
            for (int i = 0; i < half; ++i) {
                const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
                float a = orc_bf16_to_f32(src[ia]), b = orc_bf16_to_f32(src[ib]);
                if (nw) {
                    a = a * inv_rms * orc_bf16_to_f32(nw[ia]);
                    b = b * inv_rms * orc_bf16_to_f32(nw[ib]);
                }
                const float c = table[(size_t)n * d + i], s = table[(size_t)n * d + i + half];
                dst[ia] = orc_f32_to_bf16(a * c - b * s);
                dst[ib] = orc_f32_to_bf16(b * c + a * s);
            }
        }
    }
}

void orc_swiglu(const uint16_t* gate_up, uint16_t* y, int n_tokens, int inter) {
    for (int n = 0; n < n_tokens; ++n)
        for (int i = 0; i < inter; ++i) {
            const float g = orc_bf16_to_f32(gate_up[(size_t)n * 2 * inter + i]);
            const float u = orc_bf16_to_f32(gate_up[(size_t)n * 2 * inter + inter + i]);
            const float silu = g / (1.f + expf(-g));
            y[(size_t)n * inter + i] = orc_f32_to_bf16(silu * u);
        }
}

void orc_argmax_bf16(const uint16_t* logits, uint32_t* out, int rows, int vocab) {
    for (int r = 0; r < rows; ++r) {
        float best = -INFINITY;
        int bi = 0;
        for (int i = 0; i < vocab; ++i) {
            const float v = orc_bf16_to_f32(logits[(size_t)r * vocab + i]);
            if (v > best) { best = v; bi = i; }  /* strict >: first (lowest) index wins */
        }
        out[r] = (uint32_t)bi;
    }
}

/* bf16 linear: y = act · W^T (+beta*y), fp32 accumulate (mode 0) or fp64 (mode 2). */
void orc_gemm_bf16(const uint16_t* act, const uint16_t* w, const uint16_t* y_in, float* y_f32,
                   uint16_t* y_bf16, double* abs_sum, int M, int N, int K, int beta, int mode) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < M; ++m) {
            float accf = 0.f;
            double accd = 0.0, absd = 0.0;
            for (int k = 0; k < K; ++k) {
                const float x = orc_bf16_to_f32(act[(size_t)m * K + k]);
                const float ww = orc_bf16_to_f32(w[(size_t)n * K + k]);
                if (mode == 0) accf += x * ww; else accd += (double)x * (double)ww;
                absd += fabs((double)x * (double)ww);
            }
            double v = mode == 0 ? (double)accf : accd;
            const size_t o = (size_t)m * N + n;
            if (beta) v += (double)orc_bf16_to_f32(y_in[o]);
            y_f32[o] = (float)v;
            if (y_bf16) y_bf16[o] = orc_f32_to_bf16((float)v);
            if (abs_sum) abs_sum[o] = absd;
        }
}
